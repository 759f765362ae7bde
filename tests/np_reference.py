"""Independent float64 numpy restatement of the decode step, used only to
cross-check the C oracle (two restatements written separately must agree).
Vectorised, so summation order differs from the oracle's serial loops; the
comparison is made against the oracle's double-precision shadow."""
import numpy as np


def f16_to_f32(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float32)


def quantize_q8(w, mode=0):
    """cuda_fused_infer.go:363-390 (mode 0) / metal_impl_darwin.m:5765-5780 (mode 1)."""
    w = np.asarray(w, np.float32)
    amax = np.abs(w).max(axis=1)
    s = (amax / np.float32(127.0)).astype(np.float32)
    q = np.zeros(w.shape, np.int8)
    nz = s > 0
    if mode == 0:
        with np.errstate(over="ignore", invalid="ignore"):
            inv = (np.float32(1.0) / s[nz]).astype(np.float32)
            t = (w[nz] * inv[:, None]).astype(np.float32)
        v = np.trunc(t)
        v[~np.isfinite(t)] = -128          # Go's int() of NaN/inf is the most negative integer
        q[nz] = np.clip(v, -128, 127).astype(np.int8)
    else:
        inv = (np.float32(127.0) / amax[nz]).astype(np.float32)
        v = np.clip((w[nz] * inv[:, None]).astype(np.float32), -127, 127).astype(np.float32)
        q[nz] = np.trunc(v + np.where(v > 0, np.float32(0.5), np.float32(-0.5)).astype(np.float32)).astype(np.int8)
    return q, s


def quantize_q4_0(w):
    """GGML quantize_row_q4_0_ref."""
    w = np.asarray(w, np.float32)
    rows, cols = w.shape
    x = w.reshape(-1, 32)
    idx = np.abs(x).argmax(axis=1)           # first maximum, as the strict '<' scan
    mx = x[np.arange(x.shape[0]), idx]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    y = (x * idv[:, None]).astype(np.float32) + np.float32(8.5)
    qi = np.minimum(np.trunc(y.astype(np.float32)).astype(np.int64).astype(np.int8), 15).astype(np.uint8)
    qs = (qi[:, :16] | (qi[:, 16:] << 4)).astype(np.uint8)
    out = np.empty((x.shape[0], 18), np.uint8)
    out[:, :2] = d.astype(np.float16).view(np.uint16).reshape(-1, 1).view(np.uint8).reshape(-1, 2)
    out[:, 2:] = qs
    return out.ravel()


def dequant_q4_0(blocks, rows, cols):
    b = np.asarray(blocks, np.uint8).reshape(-1, 18)
    d = b[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    lo = (b[:, 2:] & 0x0F).astype(np.int32) - 8
    hi = (b[:, 2:] >> 4).astype(np.int32) - 8
    vals = np.concatenate([lo, hi], axis=1).astype(np.float32) * d[:, None]
    return vals.astype(np.float32).reshape(rows, cols)


def rope_tables(maxSeq, headDim, theta):
    j = np.arange(headDim // 2, dtype=np.float64)
    freq = 1.0 / np.power(float(theta), 2.0 * j / headDim)
    ang = np.arange(maxSeq, dtype=np.float64)[:, None] * freq[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


class NpModel:
    """Decode step in float64 over dequantized float32 weights."""

    def __init__(self, shape_args, weights, vecs, maxSeq, kv_f16=False):
        self.kv_f16 = kv_f16       # K/V rows stored as float16 (numpy's own rounding)
        (self.dim, self.kvDim, self.headDim, self.nHeads, self.nKVHeads, self.ffnDim, self.vocab,
         self.nLayers, self.theta, self.eps) = shape_args
        self.W = {k: np.asarray(v, np.float64) for k, v in weights.items()}     # idx -> dequantized [N,K]
        self.V = {k: np.asarray(v, np.float64) for k, v in vecs.items()}        # idx -> vector
        self.cos, self.sin = rope_tables(maxSeq, self.headDim, self.theta)
        self.Kc = np.zeros((self.nLayers, maxSeq, self.kvDim))
        self.Vc = np.zeros((self.nLayers, maxSeq, self.kvDim))

    def rms(self, x, g):
        return x * (1.0 / np.sqrt(np.mean(x * x) + np.float64(np.float32(self.eps)))) * g

    def rope(self, x, pos, nH):
        hd, half = self.headDim, self.headDim // 2
        x = x.reshape(nH, hd).copy()
        c, s = self.cos[pos].astype(np.float64), self.sin[pos].astype(np.float64)
        a, b = x[:, :half].copy(), x[:, half:].copy()
        x[:, :half] = a * c - b * s
        x[:, half:] = a * s + b * c
        return x.reshape(-1)

    def step(self, hidden, pos, want_layers=False):
        x = np.asarray(hidden, np.float64).copy()
        hd, G = self.headDim, self.nHeads // self.nKVHeads
        layers = []
        for l in range(self.nLayers):
            b = l * 12
            n = self.rms(x, self.V[b + 0])
            q = self.W[b + 1] @ n
            k = self.W[b + 2] @ n
            v = self.W[b + 3] @ n
            if b + 4 in self.V:
                q = q + self.V[b + 4]
                k = k + self.V[b + 5]
                v = v + self.V[b + 6]
            q = self.rope(q, pos, self.nHeads)
            k = self.rope(k, pos, self.nKVHeads)
            if self.kv_f16:
                k = k.astype(np.float32).astype(np.float16).astype(np.float64)
                v = v.astype(np.float32).astype(np.float16).astype(np.float64)
            self.Kc[l, pos] = k
            self.Vc[l, pos] = v
            out = np.zeros(self.dim)
            for h in range(self.nHeads):
                kvh = h // G
                Kh = self.Kc[l, : pos + 1, kvh * hd:(kvh + 1) * hd]
                Vh = self.Vc[l, : pos + 1, kvh * hd:(kvh + 1) * hd]
                sc = (Kh @ q[h * hd:(h + 1) * hd]) / np.sqrt(hd)
                p = np.exp(sc - sc.max())
                p /= p.sum()
                out[h * hd:(h + 1) * hd] = p @ Vh
            x = x + self.W[b + 7] @ out
            n2 = self.rms(x, self.V[b + 8])
            g = self.W[b + 9] @ n2
            u = self.W[b + 10] @ n2
            m = g / (1.0 + np.exp(-g)) * u
            x = x + self.W[b + 11] @ m
            layers.append(x.copy())
        nf = self.rms(x, self.V[self.nLayers * 12])
        logits = self.W[self.nLayers * 12 + 1] @ nf
        return x, logits, (np.array(layers) if want_layers else None)

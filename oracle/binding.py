"""ctypes binding of the CPU oracle (oracle/mongoose_oracle.c).

TEST INFRASTRUCTURE ONLY.  The product (mongoose_amd/) never imports this.
"""
import ctypes
import os
import subprocess
from ctypes import POINTER, c_double, c_float, c_int, c_int8, c_uint8, c_uint16, c_void_p

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmongoose_oracle.so")


def build():
    subprocess.check_call(["make", "-s", "-C", HERE])
    return LIB_PATH


def _load():
    if not os.path.exists(LIB_PATH):
        build()
    return ctypes.CDLL(LIB_PATH)


lib = _load()
_f = POINTER(c_float)
_d = POINTER(c_double)


def _sig(name, restype, *argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)


_sig("orc_f32_to_f16", c_uint16, c_float)
_sig("orc_f16_to_f32", c_float, c_uint16)
_sig("orc_matmul", None, _f, _f, c_int, c_int, c_int, _f)
_sig("orc_rmsnorm", None, _f, _f, c_int, c_float)
_sig("orc_softmax", None, _f, c_int)
_sig("orc_quantize_q8", None, _f, c_int, c_int, c_int, POINTER(c_int8), _f)
_sig("orc_dequant_q8", None, POINTER(c_int8), _f, c_int, c_int, _f)
_sig("orc_quantize_q4_0", None, _f, c_int, c_int, POINTER(c_uint8))
_sig("orc_dequant_q4_0", None, POINTER(c_uint8), c_int, c_int, _f)
_sig("orc_rope_tables", None, c_int, c_int, c_double, _f, _f)
_sig("orc_create", c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_double, c_float)
_sig("orc_destroy", None, c_void_p)
_sig("orc_set_threads", None, c_void_p, c_int)
_sig("orc_num_weights", c_int, c_void_p)
_sig("orc_set_f32", c_int, c_void_p, c_int, _f, c_int)
_sig("orc_set_q8", c_int, c_void_p, c_int, POINTER(c_int8), _f)
_sig("orc_set_q4_0", c_int, c_void_p, c_int, POINTER(c_uint8))
_sig("orc_set_embed_f16", None, c_void_p, POINTER(c_uint16))
_sig("orc_set_embed_f32", None, c_void_p, _f)
_sig("orc_reset_kv", None, c_void_p)
_sig("orc_set_kv_f16", None, c_void_p, c_int)
_sig("orc_set_q4_act_quant", None, c_void_p, c_int)
_sig("orc_q8_quantize_act", None, _f, POINTER(c_uint8), c_int)
_sig("orc_embed", c_int, c_void_p, c_int, _f)
_sig("orc_argmax", c_int, _f, c_int)
for pfx, real in (("orc32", _f), ("orc64", _d)):
    _sig(pfx + "_rmsnorm_out", None, real, _f, c_int, c_float, real)
    _sig(pfx + "_q8_matvec", None, real, POINTER(c_int8), _f, real, c_int, c_int, c_int)
    _sig(pfx + "_q4_0_matvec", None, real, POINTER(c_uint8), real, c_int, c_int, c_int)
    _sig(pfx + "_q4_0_matvec_q8act", None, POINTER(c_uint8), POINTER(c_uint8), real, c_int, c_int, c_int)
    _sig(pfx + "_rope", None, real, _f, _f, c_int, c_int)
    _sig(pfx + "_decode_attention", None, real, real, real, real, c_int, c_int, c_int, c_int, c_int, real)
    _sig(pfx + "_silu_gate_mul", None, real, real, real, c_int)
    _sig(pfx + "_q4_matvec", None, real, POINTER(c_uint8), _f, real, c_int, c_int)
    _sig(pfx + "_fused_add_rmsnorm", None, real, real, _f, c_int, c_float, real)
    _sig(pfx + "_step", c_int, c_void_p, _f, c_int, c_int, c_int, _f, _f, _f)
    _sig(pfx + "_decode_token", c_int, c_void_p, c_int, c_int, _f, _f)


def fp(a):
    return a.ctypes.data_as(_f)


def dp(a):
    return a.ctypes.data_as(_d)


def i8p(a):
    return a.ctypes.data_as(POINTER(c_int8))


def u8p(a):
    return a.ctypes.data_as(POINTER(c_uint8))


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


# ---- array-level helpers ----
def quantize_q8(w, mode=0):
    w = f32(w)
    rows, cols = w.shape
    q = np.empty((rows, cols), np.int8)
    s = np.empty(rows, np.float32)
    lib.orc_quantize_q8(fp(w), rows, cols, mode, i8p(q), fp(s))
    return q, s


def dequant_q8(q, s):
    q = np.ascontiguousarray(q, np.int8)
    out = np.empty(q.shape, np.float32)
    lib.orc_dequant_q8(i8p(q), fp(f32(s)), q.shape[0], q.shape[1], fp(out))
    return out


def quantize_q4_0(w):
    w = f32(w)
    rows, cols = w.shape
    out = np.empty(rows * (cols // 32) * 18, np.uint8)
    lib.orc_quantize_q4_0(fp(w), rows, cols, u8p(out))
    return out


def dequant_q4_0(blocks, rows, cols):
    blocks = np.ascontiguousarray(blocks, np.uint8)
    out = np.empty((rows, cols), np.float32)
    lib.orc_dequant_q4_0(u8p(blocks), rows, cols, fp(out))
    return out


def rope_tables(maxSeq, headDim, theta):
    c = np.empty((maxSeq, headDim // 2), np.float32)
    s = np.empty((maxSeq, headDim // 2), np.float32)
    lib.orc_rope_tables(maxSeq, headDim, float(theta), fp(c), fp(s))
    return c, s


def _real(shadow):
    return ("orc64", np.float64, dp) if shadow else ("orc32", np.float32, fp)


def rmsnorm_out(x, g, eps, shadow=False):
    pfx, dt, p = _real(shadow)
    x = np.ascontiguousarray(x, dt)
    out = np.empty_like(x)
    getattr(lib, pfx + "_rmsnorm_out")(p(x), fp(f32(g)), x.size, eps, p(out))
    return out


def q8_matvec(act, q, s, shadow=False, threads=1):
    pfx, dt, p = _real(shadow)
    act = np.ascontiguousarray(act, dt)
    q = np.ascontiguousarray(q, np.int8)
    out = np.empty(q.shape[0], dt)
    getattr(lib, pfx + "_q8_matvec")(p(act), i8p(q), fp(f32(s)), p(out), q.shape[0], q.shape[1], threads)
    return out


def q4_0_matvec(act, blocks, N, K, shadow=False, threads=1):
    pfx, dt, p = _real(shadow)
    act = np.ascontiguousarray(act, dt)
    blocks = np.ascontiguousarray(blocks, np.uint8)
    out = np.empty(N, dt)
    getattr(lib, pfx + "_q4_0_matvec")(p(act), u8p(blocks), p(out), N, K, threads)
    return out


def q8_quantize_act(act):
    """fp32 activations [K] -> int8 blocks, (K/32)*40 bytes: float d, float d*sum(q), int8 q[32]."""
    act = f32(act)
    out = np.empty(act.size // 32 * 40, np.uint8)
    lib.orc_q8_quantize_act(fp(act), u8p(out), act.size)
    return out


def q4_0_matvec_q8act(q8, blocks, N, K, shadow=False, threads=1):
    """Raw GGUF Q4_0 rows against quantized activation blocks (the integer matvec)."""
    pfx, dt, p = _real(shadow)
    q8 = np.ascontiguousarray(q8, np.uint8)
    blocks = np.ascontiguousarray(blocks, np.uint8)
    out = np.empty(N, dt)
    getattr(lib, pfx + "_q4_0_matvec_q8act")(u8p(q8), u8p(blocks), p(out), N, K, threads)
    return out


def rope(x, cosRow, sinRow, nHeads, headDim, shadow=False):
    pfx, dt, p = _real(shadow)
    x = np.array(x, dtype=dt, order="C")
    getattr(lib, pfx + "_rope")(p(x), fp(f32(cosRow)), fp(f32(sinRow)), nHeads, headDim)
    return x


def decode_attention(Q, Kc, Vc, cacheLen, kvDim, nHeads, nKVHeads, headDim, shadow=False):
    pfx, dt, p = _real(shadow)
    Q = np.ascontiguousarray(Q, dt)
    Kc = np.ascontiguousarray(Kc, dt)
    Vc = np.ascontiguousarray(Vc, dt)
    out = np.empty(nHeads * headDim, dt)
    scores = np.empty(cacheLen, dt)
    getattr(lib, pfx + "_decode_attention")(p(Q), p(Kc), p(Vc), p(out), cacheLen, kvDim, nHeads, nKVHeads, headDim, p(scores))
    return out


def silu_gate_mul(g, u, shadow=False):
    pfx, dt, p = _real(shadow)
    g = np.ascontiguousarray(g, dt)
    u = np.ascontiguousarray(u, dt)
    out = np.empty_like(g)
    getattr(lib, pfx + "_silu_gate_mul")(p(g), p(u), p(out), g.size)
    return out


def q4_matvec(act, packed, scales, N, K, shadow=False):
    """Per-row-scale 4-bit matvec (mongoose_q4_matvec): packed [N, K/2] bytes, scales [N]."""
    pfx, dt, p = _real(shadow)
    act = np.ascontiguousarray(act, dt)
    packed = np.ascontiguousarray(packed, np.uint8)
    out = np.empty(N, dt)
    getattr(lib, pfx + "_q4_matvec")(p(act), u8p(packed), fp(f32(scales)), p(out), N, K)
    return out


def fused_add_rmsnorm(a, b, g, eps, shadow=False):
    pfx, dt, p = _real(shadow)
    a = np.ascontiguousarray(a, dt)
    b = np.ascontiguousarray(b, dt)
    out = np.empty_like(a)
    getattr(lib, pfx + "_fused_add_rmsnorm")(p(a), p(b), fp(f32(g)), a.size, eps, p(out))
    return out


def rmsnorm_inplace(x, g, eps):
    """cpu.go:36-47 (CPU.RMSNorm), in place on a copy."""
    x = np.array(x, dtype=np.float32, order="C")
    lib.orc_rmsnorm(fp(x), fp(f32(g)), x.size, eps)
    return x


class Oracle:
    """The decode step on the CPU; same slot map and step arguments as the product."""

    def __init__(self, dim, kvDim, headDim, nHeads, nKVHeads, ffnDim, vocab, nLayers, maxSeq, theta, eps, threads=1):
        self.h = lib.orc_create(dim, kvDim, headDim, nHeads, nKVHeads, ffnDim, vocab, nLayers, maxSeq, float(theta), float(eps))
        self.dim, self.vocab, self.nLayers = dim, vocab, nLayers
        lib.orc_set_threads(self.h, threads)

    def close(self):
        if self.h:
            lib.orc_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_f32(self, idx, data):
        a = f32(data).ravel()
        assert lib.orc_set_f32(self.h, idx, fp(a), a.size) == 0, f"slot {idx}"

    def set_q8(self, idx, q, s):
        assert lib.orc_set_q8(self.h, idx, i8p(np.ascontiguousarray(q, np.int8)), fp(f32(s))) == 0, f"slot {idx}"

    def set_q4_0(self, idx, blocks):
        assert lib.orc_set_q4_0(self.h, idx, u8p(np.ascontiguousarray(blocks, np.uint8))) == 0, f"slot {idx}"

    def set_embed_f16(self, table):
        a = np.ascontiguousarray(table).view(np.uint16)
        lib.orc_set_embed_f16(self.h, a.ctypes.data_as(POINTER(c_uint16)))

    def set_embed_f32(self, table):
        lib.orc_set_embed_f32(self.h, fp(f32(table)))

    def reset_kv(self):
        lib.orc_reset_kv(self.h)

    def set_kv_f16(self, on):
        lib.orc_set_kv_f16(self.h, 1 if on else 0)

    def set_q4_act_quant(self, on):
        lib.orc_set_q4_act_quant(self.h, 1 if on else 0)

    def embed(self, tok):
        out = np.empty(self.dim, np.float32)
        assert lib.orc_embed(self.h, int(tok), fp(out)) == 0
        return out

    def step(self, hidden, pos, l0=0, l1=None, shadow=False, want_logits=True, want_layers=False):
        l1 = self.nLayers if l1 is None else l1
        pfx = "orc64" if shadow else "orc32"
        h = f32(hidden)
        hout = np.empty(self.dim, np.float32)
        logits = np.empty(self.vocab, np.float32) if want_logits and l1 >= self.nLayers else None
        layers = np.empty((max(l1 - l0, 1), self.dim), np.float32) if want_layers else None
        rc = getattr(lib, pfx + "_step")(self.h, fp(h), pos, l0, l1, fp(hout),
                                         fp(logits) if logits is not None else None,
                                         fp(layers) if layers is not None else None)
        assert rc == 0
        return hout, logits, layers

    def decode_token(self, tok, pos, shadow=False, want_layers=False):
        pfx = "orc64" if shadow else "orc32"
        logits = np.empty(self.vocab, np.float32)
        layers = np.empty((self.nLayers, self.dim), np.float32) if want_layers else None
        nxt = getattr(lib, pfx + "_decode_token")(self.h, int(tok), pos, fp(logits),
                                                  fp(layers) if layers is not None else None)
        return nxt, logits, layers

"""Shared test helpers: deterministic synthetic models loaded into the CPU
oracle and/or the HIP context with identical quantized bytes."""
import numpy as np

from mongoose_amd import configs
from mongoose_amd import engine as E
from oracle import binding as ob

MATRIX_SLOTS = (1, 2, 3, 7, 9, 10, 11)


def slot_shape(s, idx):
    """(rows, cols) of a weight slot; cols == 1 for vectors (cuda_fused_infer.go:241-272)."""
    kv = configs.kv_dim(s)
    nL = s.nLayers
    if idx < nL * 12:
        w = idx % 12
        return {0: (s.dim, 1), 1: (s.dim, s.dim), 2: (kv, s.dim), 3: (kv, s.dim), 4: (s.dim, 1), 5: (kv, 1),
                6: (kv, 1), 7: (s.dim, s.dim), 8: (s.dim, 1), 9: (s.ffnDim, s.dim), 10: (s.ffnDim, s.dim),
                11: (s.dim, s.ffnDim)}[w]
    if idx == nL * 12:
        return (s.dim, 1)
    return (s.vocab, s.dim)


def gen_slot(s, seed, idx):
    """fp32 data of a slot: matrices and biases N(0, 0.02), norm gains 1 + N(0, 0.02)
    (not exactly 1, so that a dropped or misplaced gain would show)."""
    rows, cols = slot_shape(s, idx)
    a = E.synth_normal(seed, idx, 0.02, (rows, cols) if cols > 1 else (rows,))
    w = idx % 12 if idx < s.nLayers * 12 else -1
    if cols == 1 and (w in (0, 8) or idx == s.nLayers * 12):
        a = (a + np.float32(1.0)).astype(np.float32)
    return a


def all_slots(s):
    for idx in range(s.nLayers * 12 + 2):
        w = idx % 12 if idx < s.nLayers * 12 else -1
        if w in (4, 5, 6) and not s.bias:
            continue
        yield idx


def with_layers(s, n):
    return s._replace(nLayers=n, name=f"{s.name}-L{n}")


class Model:
    """Oracle and/or HIP context holding the same synthetic model."""

    def __init__(self, s, seed, maxSeq, eng=None, oracle=True, threads=8, fmt=None, keep_dequant=False, kv_f16=False):
        self.s, self.seed, self.maxSeq, self.eng = s, seed, maxSeq, eng
        fmt = fmt or s.fmt
        kv = configs.kv_dim(s)
        self.orc = ob.Oracle(s.dim, kv, s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab, s.nLayers, maxSeq,
                             s.theta, s.eps, threads=threads) if oracle else None
        if kv_f16 and self.orc:
            self.orc.set_kv_f16(True)
        self.hip = None
        if eng is not None:
            self.hip = E.NewHIPFusedInference(eng, s.dim, kv, s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab,
                                              s.nLayers, maxSeq, s.theta, s.eps)
            assert self.hip is not None, E.last_error()
            if kv_f16:
                assert self.hip.SetKVFormat(1) == 0, E.last_error()
            assert self.hip.SetLayerRange(0, s.nLayers) == 0, E.last_error()
        self.dequant = {} if keep_dequant else None
        self.vecs = {}
        for idx in all_slots(s):
            rows, cols = slot_shape(s, idx)
            data = gen_slot(s, seed, idx)
            if cols == 1:
                self.vecs[idx] = data
                if self.orc:
                    self.orc.set_f32(idx, data)
                if self.hip:
                    assert self.hip.SetWeight(idx, data) == 0, E.last_error()
                continue
            if fmt == "q8":
                q, sc = ob.quantize_q8(data, 0)
                if self.orc:
                    self.orc.set_q8(idx, q, sc)
                if self.hip:
                    assert self.hip.SetWeightQ8(idx, q, sc) == 0, E.last_error()
                if keep_dequant:
                    self.dequant[idx] = ob.dequant_q8(q, sc)
            else:
                blocks = ob.quantize_q4_0(data)
                if self.orc:
                    self.orc.set_q4_0(idx, blocks)
                if self.hip:
                    assert self.hip.SetWeightQ4_0(idx, blocks) == 0, E.last_error()
                if keep_dequant:
                    self.dequant[idx] = ob.dequant_q4_0(blocks, rows, cols)
        if not s.tied:
            # separate fp16 embedding table (the Q4_0 configuration keeps embeddings in fp16)
            emb = E.synth_normal(seed, 10_000_019, 0.02, (s.vocab, s.dim)).astype(np.float16)
            self.embed16 = emb
            if self.orc:
                self.orc.set_embed_f16(emb)
            if self.hip:
                assert self.hip.SetEmbeddingF16(emb) == 0, E.last_error()

    def prompt(self, n):
        return E.synth_tokens(self.seed, 20_000_003, self.s.vocab, n)

    def close(self):
        if self.hip:
            self.hip.Close()
        if self.orc:
            self.orc.close()


def rel_err(a, b):
    """max |a-b| / max |b|: error relative to the largest entry of the reference vector."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    den = np.abs(b).max()
    return float(np.abs(a - b).max() / den) if den > 0 else float(np.abs(a - b).max())


def oracle_generate(m, prompt, nDecode, want=None, shadow=False):
    """Greedy decode on the oracle; returns (tokens, per-position records)."""
    m.orc.reset_kv()
    toks, rec = [], {}
    tok = int(prompt[0])
    nP = len(prompt)
    for pos in range(nP - 1 + nDecode):
        nxt, logits, layers = m.orc.decode_token(tok, pos, shadow=shadow, want_layers=want is not None and pos in want)
        if want is not None and pos in want:
            rec[pos] = (logits.copy(), layers.copy())
        if pos + 1 < nP:
            tok = int(prompt[pos + 1])
        else:
            toks.append(nxt)
            tok = nxt
    return np.array(toks, np.int32), rec


def first_divergence(a, b):
    """Index of the first position where two token sequences differ, or None."""
    n = min(len(a), len(b))
    for i in range(n):
        if int(a[i]) != int(b[i]):
            return i
    return None if len(a) == len(b) else n


def assert_same_tokens_or_near_tie(m, prompt, toks, other, what, tol=1e-3):
    """Two correct evaluation orders of the same model give the same greedy tokens unless two logits
    are closer than the arithmetic can resolve.  Either the sequences are identical, or at their first
    difference the oracle's (double-precision) logits of the two candidate tokens differ by less than
    `tol` of the largest logit: the logit bar itself.  `toks` is the sequence the oracle is replayed on."""
    i = first_divergence(toks, other)
    if i is None:
        return None
    m.orc.reset_kv()
    stream = list(prompt) + [int(t) for t in toks[:i]]
    logits = None
    for pos, tok in enumerate(stream):
        _, logits, _ = m.orc.decode_token(int(tok), pos, shadow=True)
    a, b = int(toks[i]), int(other[i])
    gap = abs(float(logits[a]) - float(logits[b])) / float(np.abs(logits).max())
    assert gap < tol, f"{what}: sequences part at token {i} ({a} vs {b}) and the oracle's logits differ by {gap:.2e}"
    return i


def load_fast(s, seed, maxSeq, eng, oracle=True, threads=16, kv_f16=False):
    """A Model whose matrices are quantized by the library's parallel host quantizer (bit-identical to
    the oracle's, checked on the CPU) and shared with the oracle: for the multi-gigabyte shapes."""
    m = Model.__new__(Model)
    m.s, m.seed, m.maxSeq, m.eng = s, seed, maxSeq, eng
    kv = configs.kv_dim(s)
    m.orc = ob.Oracle(s.dim, kv, s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab, s.nLayers, maxSeq,
                      s.theta, s.eps, threads=threads) if oracle else None
    if kv_f16 and m.orc:
        m.orc.set_kv_f16(True)
    m.hip = E.NewHIPFusedInference(eng, s.dim, kv, s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab, s.nLayers,
                                   maxSeq, s.theta, s.eps)
    assert m.hip is not None, E.last_error()
    if kv_f16:
        assert m.hip.SetKVFormat(1) == 0, E.last_error()
    assert m.hip.SetLayerRange(0, s.nLayers) == 0, E.last_error()
    m.dequant, m.vecs = None, {}
    for idx in all_slots(s):
        rows, cols = slot_shape(s, idx)
        data = gen_slot(s, seed, idx)
        if cols == 1:
            m.vecs[idx] = data
            if m.orc:
                m.orc.set_f32(idx, data)
            assert m.hip.SetWeight(idx, data) == 0, E.last_error()
        elif s.fmt == "q8":
            q, sc = E.quantize_q8(data, 0)
            if m.orc:
                m.orc.set_q8(idx, q, sc)
            assert m.hip.SetWeightQ8(idx, q, sc) == 0, E.last_error()
        else:
            blocks = E.quantize_q4_0(data)
            if m.orc:
                m.orc.set_q4_0(idx, blocks)
            assert m.hip.SetWeightQ4_0(idx, blocks) == 0, E.last_error()
    if not s.tied:
        emb = E.synth_normal(seed, 10_000_019, 0.02, (s.vocab, s.dim)).astype(np.float16)
        m.embed16 = emb
        if m.orc:
            m.orc.set_embed_f16(emb)
        assert m.hip.SetEmbeddingF16(emb) == 0, E.last_error()
    return m

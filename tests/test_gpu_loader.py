"""The reference's own loading path on the GPU through the C ABI: SetWeight takes fp32, quantizes matrix
slots on the host (quantizeQ8, cuda_fused_infer.go:363-390) and uploads them (:241-272).  A model loaded
that way must behave bit for bit like one loaded with SetWeightQ8 from the oracle's quantized bytes, in both
rounding modes; and the fp32 embedding table (mg_set_embedding_f32) must be what the decode step gathers."""
import numpy as np
import pytest

from mongoose_amd import configs
from mongoose_amd import engine as E
from oracle import binding as ob
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _ctx(hip, s, maxSeq):
    f = E.NewHIPFusedInference(hip, s.dim, configs.kv_dim(s), s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab,
                               s.nLayers, maxSeq, s.theta, s.eps)
    assert f is not None, E.last_error()
    assert f.SetLayerRange(0, s.nLayers) == 0, E.last_error()
    return f


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("shape", [configs.TOY, H.with_layers(configs.QWEN, 2)._replace(vocab=3000)], ids=lambda s: s.name)
def test_set_weight_fp32_equals_set_weight_q8_of_oracle_bytes(hip, shape, mode):
    s = shape
    maxSeq = 12
    a, b = _ctx(hip, s, maxSeq), _ctx(hip, s, maxSeq)
    assert a.SetExecMode(1) == 0 and b.SetExecMode(1) == 0       # the same launches in both (one context a device owns the persistent one)
    assert a.SetQuantRounding(mode) == 0
    assert a.SetQuantRounding(2) != 0                            # only 0 and 1 exist
    orc = ob.Oracle(s.dim, configs.kv_dim(s), s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab, s.nLayers, maxSeq,
                    s.theta, s.eps, threads=8)
    differs = False
    for idx in H.all_slots(s):
        rows, cols = H.slot_shape(s, idx)
        data = H.gen_slot(s, 77, idx)
        assert a.SetWeight(idx, data) == 0, E.last_error()      # fp32 in: host quantizer inside the library
        if cols == 1:
            assert b.SetWeight(idx, data) == 0
            orc.set_f32(idx, data)
        else:
            q, sc = ob.quantize_q8(data, mode)                   # the oracle's quantizer, same rounding
            q0, _ = ob.quantize_q8(data, 0)
            differs = differs or not np.array_equal(q, q0)
            assert b.SetWeightQ8(idx, q, sc) == 0, E.last_error()
            orc.set_q8(idx, q, sc)
    assert differs == (mode == 1)                                # the switch does something
    prompt = E.synth_tokens(77, 20_000_003, s.vocab, 6)
    la, lb = np.empty(s.vocab, np.float32), np.empty(s.vocab, np.float32)
    for pos in range(6):
        ra, na = a.DecodeToken(int(prompt[pos]), pos, la)
        rb, nb = b.DecodeToken(int(prompt[pos]), pos, lb)
        assert ra == 0 and rb == 0, E.last_error()
        assert na == nb and np.array_equal(la, lb), pos          # same bytes on the device: same bits out
        nxt, lg, _ = orc.decode_token(int(prompt[pos]), pos, shadow=True)
        assert H.rel_err(la, lg) < 1e-3 and na == nxt, pos
    # greedy generation through the graph as well
    assert a.ResetKV() == 0 and b.ResetKV() == 0
    ra, ta = a.Generate(prompt[:4], 8, useGraph=True)
    rb, tb = b.Generate(prompt[:4], 8, useGraph=True)
    assert ra == 0 and rb == 0 and ta.tolist() == tb.tolist()
    assert a.WeightBytesPerToken() == b.WeightBytesPerToken()
    a.Close()
    b.Close()
    orc.close()


def test_fp32_embedding_table(hip):
    """mg_set_embedding_f32: the decode step gathers the fp32 row of the token (mongoose.cu:1052-1064 is the
    reference's fp32 gather) instead of the tied lm_head row; oracle: orc_set_embed_f32."""
    s = H.with_layers(configs.TOY, 2)
    m = H.Model(s, seed=88, maxSeq=16, eng=hip, threads=4)
    table = E.synth_normal(88, 10_000_033, 0.05, (s.vocab, s.dim))
    tied = [m.hip.DecodeToken(5, 0)[1]]
    assert m.hip.ResetKV() == 0
    assert m.hip.SetEmbeddingF32(table) == 0, E.last_error()
    m.orc.set_embed_f32(table)
    assert np.array_equal(m.orc.embed(9), table[9])
    prompt = m.prompt(5)
    ref, rec = H.oracle_generate(m, prompt, 8, want={0, 11}, shadow=True)
    for graph in (False, True):
        assert m.hip.ResetKV() == 0
        rc, toks = m.hip.Generate(prompt, 8, useGraph=graph)
        assert rc == 0, E.last_error()
        assert toks.tolist() == ref.tolist(), graph
    assert m.hip.ResetKV() == 0
    stream = list(prompt) + list(ref)
    logits = np.empty(s.vocab, np.float32)
    for pos in range(12):
        rc, _ = m.hip.DecodeToken(int(stream[pos]), pos, logits)
        assert rc == 0
        if pos in rec:
            assert H.rel_err(logits, rec[pos][0]) < 1e-3, pos
    # the batched prefill gathers from the same table
    assert m.hip.ResetKV() == 0
    rc, toks_pf = m.hip.GeneratePrefill(prompt, 8)
    assert rc == 0 and toks_pf.tolist() == ref.tolist()
    m.close()


def test_bench_matvec_helper_runs(hip):
    """mg_bench_matvec (the launch-shape sweep helper): returns a positive time for both formats and
    rejects bad arguments."""
    import ctypes
    from mongoose_amd.lib import lib
    us = ctypes.c_float(0)
    for wf in (0, 1):
        assert lib.mg_bench_matvec(wf, 896, 896, 0, 0, 0, 4, 20, ctypes.byref(us)) == 0
        assert 0.5 < us.value < 1000.0
    assert lib.mg_bench_matvec(0, 896, 896, 2, 1, 0, 2, 5, ctypes.byref(us)) == 0      # explicit configuration
    assert lib.mg_bench_matvec(2, 896, 896, 0, 0, 0, 1, 1, ctypes.byref(us)) != 0      # raw GGUF rows: not benchmarked
    assert lib.mg_bench_matvec(0, 896, 900, 0, 0, 0, 1, 1, ctypes.byref(us)) != 0      # K not a multiple of 32


def test_stream_object_outliving_its_context_is_inert(hip):
    """Destroying the context before its stream object leaves the latter refusing work, not dangling."""
    s = H.with_layers(configs.QWEN_Q4, 1)._replace(vocab=512)
    m = H.Model(s, seed=12, maxSeq=4, eng=hip, oracle=False)
    st = m.hip.StreamBuild()
    assert st is not None
    m.hip.Close()
    h = np.zeros(s.dim, np.float32)
    rc = st.StreamForwardToken(0, h, 1, [None] * 12, [0] * 7, None)
    assert rc == -4 and "destroyed" in E.last_error()
    st.Close()

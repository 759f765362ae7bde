"""The oracle's decode step against an independently written numpy float64
restatement (layer order, bias position, RoPE, GQA map, residuals, tail), and
the float path against its double shadow."""
import numpy as np
import pytest

from mongoose_amd import configs
from oracle import binding as ob
from tests import helpers as H
from tests import np_reference as npr


def _np_model(m, maxSeq, kv_f16=False):
    s = m.s
    args = (s.dim, configs.kv_dim(s), s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab, s.nLayers, s.theta, s.eps)
    return npr.NpModel(args, m.dequant, m.vecs, maxSeq, kv_f16=kv_f16)


MINI = configs.Shape("mini", 2, 128, 4, 2, 32, 160, 96, 1e-5, 1e4, True, True, "q8")
MINI_Q4 = MINI._replace(name="mini-q4", fmt="q4_0", tied=False, bias=False)


@pytest.mark.parametrize("shape", [MINI, MINI_Q4], ids=lambda s: s.name)
def test_step_matches_numpy_restatement(shape):
    maxSeq = 12
    m = H.Model(shape, seed=7, maxSeq=maxSeq, eng=None, oracle=True, threads=1, keep_dequant=True)
    ref = _np_model(m, maxSeq)
    prompt = m.prompt(maxSeq)
    m.orc.reset_kv()
    for pos in range(maxSeq):
        h = m.orc.embed(prompt[pos])
        if shape.tied:
            # tied Q8 embedding = dequantized lm_head row
            assert (h == m.dequant[shape.nLayers * 12 + 1][prompt[pos]]).all()
        else:
            assert (h == m.embed16[prompt[pos]].astype(np.float32)).all()
        hout64, logits64, layers64 = m.orc.step(h, pos, shadow=True, want_layers=True)
        x, logits, layers = ref.step(h, pos, want_layers=True)
        assert H.rel_err(layers64, layers) < 1e-6, pos       # outputs are cast to float
        assert H.rel_err(logits64, logits) < 1e-6, pos
        assert H.rel_err(hout64, x) < 1e-6
    m.close()


def test_fp16_kv_option_matches_numpy_float16_rows():
    """K/V rows rounded to fp16 when written: the oracle's conversion against numpy.float16 inside the
    independent model; and the option changes the result (it is not a no-op)."""
    maxSeq = 10
    m = H.Model(MINI, seed=13, maxSeq=maxSeq, eng=None, oracle=True, threads=1, keep_dequant=True, kv_f16=True)
    plain = H.Model(MINI, seed=13, maxSeq=maxSeq, eng=None, oracle=True, threads=1)
    ref = _np_model(m, maxSeq, kv_f16=True)
    prompt = m.prompt(maxSeq)
    differs = False
    for pos in range(maxSeq):
        h = m.orc.embed(prompt[pos])
        hout64, logits64, _ = m.orc.step(h, pos, shadow=True)
        x, logits, _ = ref.step(h, pos)
        assert H.rel_err(logits64, logits) < 1e-6 and H.rel_err(hout64, x) < 1e-6, pos
        _, logits_plain, _ = plain.orc.step(h, pos, shadow=True)
        differs = differs or H.rel_err(logits64, logits_plain) > 1e-6
    assert differs
    m.close()
    plain.close()


def test_float_step_tracks_double_shadow():
    maxSeq = 10
    m = H.Model(MINI, seed=11, maxSeq=maxSeq, oracle=True, threads=1)
    m2 = H.Model(MINI, seed=11, maxSeq=maxSeq, oracle=True, threads=1)
    prompt = m.prompt(maxSeq)
    for pos in range(maxSeq):
        h = m.orc.embed(prompt[pos])
        a, la, _ = m.orc.step(h, pos)
        b, lb, _ = m2.orc.step(h, pos, shadow=True)
        assert H.rel_err(a, b) < 2e-5 and H.rel_err(la, lb) < 2e-5
    m.close()
    m2.close()


def test_partial_ranges_compose():
    # layers [0,1) then [1,2) == [0,2): the layer-range arguments of PartialStep
    m = H.Model(MINI, seed=3, maxSeq=4, oracle=True, threads=1)
    m2 = H.Model(MINI, seed=3, maxSeq=4, oracle=True, threads=1)
    h = m.orc.embed(5)
    full, lg, _ = m.orc.step(h, 0)
    mid, none_logits, _ = m2.orc.step(h, 0, 0, 1)
    assert none_logits is None
    end, lg2, _ = m2.orc.step(mid, 0, 1, 2)
    assert (full == end).all() and (lg == lg2).all()
    m.close()
    m2.close()


def test_threads_do_not_change_results():
    m1 = H.Model(MINI, seed=5, maxSeq=4, oracle=True, threads=1)
    m4 = H.Model(MINI, seed=5, maxSeq=4, oracle=True, threads=4)
    h = m1.orc.embed(9)
    a = m1.orc.step(h, 0)
    b = m4.orc.step(h, 0)
    assert (a[0] == b[0]).all() and (a[1] == b[1]).all()
    m1.close()
    m4.close()


# ---------------------------------------------------------------------------
# Step-level checks that the mathematics fixes (independent of tests/np_reference.py)
# ---------------------------------------------------------------------------
def _oracle_from(shape, maxSeq, mats, vecs):
    """Oracle with explicitly given fp32 matrices (quantized to Q8 here) and vectors."""
    kv = configs.kv_dim(shape)
    o = ob.Oracle(shape.dim, kv, shape.headDim, shape.nHeads, shape.nKVHeads, shape.ffnDim, shape.vocab,
                  shape.nLayers, maxSeq, shape.theta, shape.eps, threads=1)
    deq = {}
    for idx, w in mats.items():
        q, s = ob.quantize_q8(w, 0)
        o.set_q8(idx, q, s)
        deq[idx] = ob.dequant_q8(q, s)
    for idx, v in vecs.items():
        o.set_f32(idx, v)
    return o, deq


def _random_layer(shape, rng, l=0):
    kv = configs.kv_dim(shape)
    d, f = shape.dim, shape.ffnDim
    n = lambda *sh: (rng.standard_normal(sh) * 0.1).astype(np.float32)
    mats = {l * 12 + 1: n(d, d), l * 12 + 2: n(kv, d), l * 12 + 3: n(kv, d), l * 12 + 7: n(d, d),
            l * 12 + 9: n(f, d), l * 12 + 10: n(f, d), l * 12 + 11: n(d, f)}
    vecs = {l * 12 + 0: (1 + n(d)).astype(np.float32), l * 12 + 8: (1 + n(d)).astype(np.float32)}
    return mats, vecs


def test_zero_output_projections_leave_the_residual_stream_unchanged():
    """x += Wo.attn and x += Wdown.ffn are the only writes to the residual stream
    (cuda_fused_infer.go:434-435, 442-443): with both matrices zero a layer is the identity, bit for bit,
    whatever the other weights are, at every position."""
    shape = configs.Shape("id", 2, 64, 2, 1, 32, 96, 40, 1e-5, 1e4, True, True, "q8")
    rng = np.random.default_rng(5)
    mats, vecs = {}, {}
    for l in range(shape.nLayers):
        m, v = _random_layer(shape, rng, l)
        m[l * 12 + 7][:] = 0
        m[l * 12 + 11][:] = 0
        v[l * 12 + 4] = rng.standard_normal(shape.dim).astype(np.float32)
        mats.update(m)
        vecs.update(v)
    vecs[shape.nLayers * 12] = np.ones(shape.dim, np.float32)
    mats[shape.nLayers * 12 + 1] = (rng.standard_normal((shape.vocab, shape.dim)) * 0.1).astype(np.float32)
    o, _ = _oracle_from(shape, 6, mats, vecs)
    for pos in range(6):
        h = rng.standard_normal(shape.dim).astype(np.float32)
        for shadow in (False, True):
            out, _, layers = o.step(h, pos, shadow=shadow, want_layers=True)
            assert (out == h).all() and (layers == h).all()
    o.close()


def test_bias_is_added_before_rope_closed_form():
    """One head, Wq = Wk = 0: q and k are the biases alone, so with the bias added BEFORE the rotation
    (cuda_fused_stream.go:319-321) the score of positions (P, t) is
        [ sum_j (bq_j bk_j + bq_j' bk_j') cos((P-t) f_j) - (bq_j' bk_j - bq_j bk_j') sin((P-t) f_j) ] / sqrt(hd)
    (j' = j + hd/2, f_j = theta^(-2j/hd)): a function of P - t only.  With the bias added after the
    rotation every score would be bq.bk / sqrt(hd) and the softmax uniform.  Wo = identity and
    Wdown = 0 expose the attention output as hidden_out - hidden_in."""
    hd = 32
    shape = configs.Shape("one-head", 1, hd, 1, 1, hd, 32, 16, 1e-5, 1e4, True, True, "q8")
    rng = np.random.default_rng(11)
    mats, vecs = _random_layer(shape, rng)
    mats[1][:] = 0
    mats[2][:] = 0
    mats[7] = np.eye(hd, dtype=np.float32)
    mats[11][:] = 0
    bq = rng.standard_normal(hd).astype(np.float32)
    bk = rng.standard_normal(hd).astype(np.float32)
    bv = rng.standard_normal(hd).astype(np.float32)
    vecs.update({4: bq, 5: bk, 6: bv, 12: np.ones(hd, np.float32)})
    mats[13] = (rng.standard_normal((shape.vocab, hd)) * 0.1).astype(np.float32)
    P = 7
    o, deq = _oracle_from(shape, P + 1, mats, vecs)
    hs = rng.standard_normal((P + 1, hd)).astype(np.float64)
    outs = [o.step(hs[t].astype(np.float32), t, shadow=True)[0] for t in range(P + 1)]
    hs = hs.astype(np.float32).astype(np.float64)
    # value rows: v_t = Wv . rmsnorm(h_t, g1) + bv, in double from the dequantized matrix
    g1 = vecs[0].astype(np.float64)
    nrm = hs / np.sqrt((hs * hs).mean(axis=1, keepdims=True) + shape.eps) * g1
    v = nrm @ deq[3].astype(np.float64).T + bv
    half = hd // 2
    f = shape.theta ** (-2.0 * np.arange(half) / hd)
    q0, q1, k0, k1 = bq[:half].astype(np.float64), bq[half:].astype(np.float64), bk[:half].astype(np.float64), bk[half:].astype(np.float64)
    wo = deq[7].astype(np.float64)
    for pos in (0, 3, P):
        t = np.arange(pos + 1)
        ang = (pos - t)[:, None] * f[None, :]
        s_before = ((q0 * k0 + q1 * k1) * np.cos(ang) - (q1 * k0 - q0 * k1) * np.sin(ang)).sum(axis=1) / np.sqrt(hd)
        p = np.exp(s_before - s_before.max())
        p /= p.sum()
        want = hs[pos] + wo @ (p @ v[:pos + 1])
        assert H.rel_err(outs[pos], want) < 2e-6, pos              # the cos/sin tables are stored as floats
        if pos > 0:
            uniform = hs[pos] + wo @ v[:pos + 1].mean(axis=0)       # what bias-after-rotation would give
            assert H.rel_err(outs[pos], uniform) > 1e-3, pos
    o.close()


def test_no_logits_before_the_last_layer():
    """cuda_fused_infer.go:446: the final norm and lm_head run only when layerEnd reaches nLayers."""
    m = H.Model(MINI, seed=3, maxSeq=4, oracle=True, threads=1)
    h = m.orc.embed(5)
    for pfx in ("orc32", "orc64"):
        logits = np.full(MINI.vocab, -123.0, np.float32)
        hout = np.empty(MINI.dim, np.float32)
        rc = getattr(ob.lib, pfx + "_step")(m.orc.h, ob.fp(h), 0, 0, MINI.nLayers - 1, ob.fp(hout), ob.fp(logits), None)
        assert rc == 0 and (logits == -123.0).all()
        rc = getattr(ob.lib, pfx + "_step")(m.orc.h, ob.fp(h), 0, 0, MINI.nLayers, ob.fp(hout), ob.fp(logits), None)
        assert rc == 0 and not (logits == -123.0).any()
    m.close()


def test_threaded_attention_changes_nothing():
    """Heads are shared out over the oracle's threads; each head's arithmetic is untouched."""
    shape = MINI._replace(nHeads=4, nKVHeads=2)
    a = H.Model(shape, seed=21, maxSeq=40, oracle=True, threads=1)
    b = H.Model(shape, seed=21, maxSeq=40, oracle=True, threads=3)
    prompt = a.prompt(40)
    for pos in range(40):
        h = a.orc.embed(prompt[pos])
        for shadow in (False, True):
            x, y = a.orc.step(h, pos, shadow=shadow), b.orc.step(h, pos, shadow=shadow)
            assert (x[0] == y[0]).all() and (x[1] == y[1]).all()
    a.close()
    b.close()


def test_step_with_integer_q4_0_matvecs_tracks_the_fp32_activation_step():
    """orc_set_q4_act_quant: every Q4_0 matrix sees int8 activation blocks (cuda_fused_infer_q4.go:611-673).  Same
    step otherwise, so the logits stay within the activation rounding of the fp32-activation step and are not equal."""
    from mongoose_amd import configs
    from tests import helpers as H
    s = H.with_layers(configs.TOY, 2)._replace(fmt="q4_0", name="toy-q4")
    a = H.Model(s, seed=5, maxSeq=8, threads=4)
    b = H.Model(s, seed=5, maxSeq=8, threads=4)
    b.orc.set_q4_act_quant(True)
    prompt = a.prompt(4)
    for pos in range(4):
        h = a.orc.embed(prompt[pos])
        _, la, _ = a.orc.step(h, pos, shadow=True)
        _, lb, _ = b.orc.step(h, pos, shadow=True)
        _, lb32, _ = b.orc.step(h, pos)
        err = H.rel_err(lb, la)
        assert 1e-5 < err < 5e-2, (pos, err)
        assert H.rel_err(lb32, lb) < 1e-4
    a.close()
    b.close()

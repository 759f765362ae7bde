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

"""Decode attention in its long-context regimes on the GPU against the CPU oracle, through the fused launches
(exec mode 1: split-KV attention kernel with the last-workgroup combine, the workgroup shapes the context
picks by maxSeq -- one, two or all query heads of a GQA group per workgroup -- and several tiles inside a
split) and through the persistent layer launch (exec mode 3: its grouped attention phase, per-head merge of
tens of splits), head sizes 64 and 128, and a last split that is only partly filled.  Every test pins the
exec mode and asserts which launch ran.

Every position is stepped on both sides (the oracle needs its own K/V rows), the model is one layer
with a small FFN and vocabulary so that the oracle's time goes into the attention itself; logits and
the hidden state are compared with the oracle's double-precision shadow at the stated bars
(hidden 1e-4, logits 1e-3 relative).  The reference semantics are kernels/mongoose.cu:856-933."""
import numpy as np
import pytest

from mongoose_amd import configs
from mongoose_amd import engine as E
from tests import helpers as H

pytestmark = pytest.mark.gpu

HID_TOL = 1e-4
LOGIT_TOL = 1e-3


def _walk(m, maxSeq, check, modes=(None,)):
    """Steps positions 0..maxSeq-1 on the oracle (double shadow) and on the GPU, compares at the positions in
    `check`.  One GPU context per entry of `modes` (exec mode 1: the fused launches with their split-KV
    attention kernel; 3: the persistent layer launch with its own attention phase; None: whatever a new
    context picks), all fed the same hidden vectors, so the oracle is stepped once.  Each context is asserted
    to run the launch its mode names."""
    s = m.s
    prompt = m.prompt(maxSeq)
    m.orc.reset_kv()
    ctxs = []
    for i, mode in enumerate(modes):
        c = m if i == 0 else H.load_fast(s, seed=m.seed, maxSeq=maxSeq, eng=m.eng, oracle=False)
        if mode is not None:
            assert c.hip.SetExecMode(mode) == 0
        ctxs.append(c)
    for c, mode in zip(ctxs, modes):             # (the launch has one owner a device: claimed in this order)
        if mode is not None:
            assert c.hip.FlowInUse() == (mode == 3), f"exec mode {mode}: wrong launch in use"
        assert c.hip.ResetKV() == 0
    worst_h = worst_l = 0.0
    for pos in range(maxSeq):
        h = m.orc.embed(prompt[pos])
        want = pos in check
        hid64, lg, _ = m.orc.step(h, pos, shadow=True, want_logits=want)
        for c, mode in zip(ctxs, modes):
            logits = np.empty(s.vocab, np.float32) if want else None
            assert c.hip.PartialStep(h, pos, 0, s.nLayers, None, logits) == 0, E.last_error()
            if want:
                print(f"  {s.name}: mode {mode}: compare at pos {pos}", flush=True)
                eh, el = H.rel_err(c.hip.ExportHidden(), hid64), H.rel_err(logits, lg)
                worst_h, worst_l = max(worst_h, eh), max(worst_l, el)
                assert el < LOGIT_TOL, (mode, pos, el)
                assert eh < HID_TOL, (mode, pos, eh)
                assert int(np.argmax(logits)) == int(np.argmax(lg)), (mode, pos)
    for c, mode in zip(ctxs, modes):
        if mode is not None:
            assert c.hip.FlowInUse() == (mode == 3)
    for c in ctxs[1:]:
        c.close()
    return worst_h, worst_l


def test_llama3_head_geometry_split_kv_to_4096(hip):
    """Llama-3-8B's attention geometry -- head size 128, 32 query heads over 8 KV heads, fp32 KV rows -- up to
    position 4095 with maxSeq 4100.  The persistent launch cannot cover that context with 8 KV heads (32 partial
    slots of 128 positions), so a new context runs the fused launches: the split-KV attention kernel with
    128-row tiles, 33 splits, two query heads a workgroup.  One layer, FFN and vocabulary cut; compared at the
    first tile's end, split boundaries and 4095."""
    s = H.with_layers(configs.LLAMA3_8B, 1)._replace(name="l3-geom", ffnDim=512, vocab=1024, tied=True)
    m = H.load_fast(s, seed=51, maxSeq=4100, eng=hip, threads=16)
    assert not m.hip.FlowInUse(), "maxSeq 4100 at 8 KV heads is past what the persistent launch covers"
    _walk(m, 4100, {0, 127, 128, 129, 1023, 1024, 2047, 2048, 4095, 4099})
    m.close()


def test_context_past_8192_whole_gqa_group_per_workgroup_head64(hip):
    """maxSeq > 8192, 14 query heads on 2 KV heads (the Qwen grouping), head size 64, through both launches.
    Exec mode 1, the fused launches: the attention kernel's workgroups take a whole GQA group in chunks of four
    query heads (the second chunk holds three), 256-row tiles, 33 splits of one tile.  Exec mode 3, the
    persistent launch: grouped attention phase, 128-position tiles, up to 65 splits merged per head.  Positions
    in the first split, across boundaries, deep in the cache and in the partly filled last split."""
    s = configs.Shape("g7-hd64-long", 1, 896, 14, 2, 64, 256, 512, 1e-6, 1e6, True, True, "q8")
    m = H.load_fast(s, seed=52, maxSeq=8300, eng=hip, threads=16)
    _walk(m, 8300, {0, 127, 128, 255, 256, 1000, 4095, 4096, 8191, 8192, 8299}, modes=(1, 3))
    m.close()


def test_context_past_8192_head128_two_tiles_per_split(hip):
    """Head size 128 with maxSeq > 8192, four query heads per KV head, through both launches.  Exec mode 1: a
    split of the fused attention kernel is two 128-row tiles (the loop over tiles inside a split), the four query
    heads of a KV head in one workgroup.  Exec mode 3: the persistent launch's grouped attention phase at heads
    of 128, up to 65 splits."""
    s = configs.Shape("g4-hd128-long", 1, 1024, 8, 2, 128, 256, 512, 1e-5, 5e5, False, True, "q8")
    m = H.load_fast(s, seed=53, maxSeq=8300, eng=hip, threads=16)
    _walk(m, 8300, {0, 127, 128, 255, 256, 257, 383, 384, 5000, 8191, 8192, 8299}, modes=(1, 3))
    m.close()


def test_context_past_16384_head64_two_tiles_per_split(hip):
    """Head size 64 with maxSeq > 16384, through both launches; one KV head with seven query heads keeps the
    oracle's attention affordable at 16.5k positions.  Exec mode 1: 512 positions a split of the fused attention
    kernel, i.e. two 256-row tiles per workgroup.  Exec mode 3: the persistent launch with 129 splits of 128
    positions for its one KV head."""
    s = configs.Shape("g7-hd64-xlong", 1, 448, 7, 1, 64, 64, 256, 1e-6, 1e6, True, True, "q8")
    m = H.load_fast(s, seed=54, maxSeq=16500, eng=hip, threads=16)
    _walk(m, 16500, {0, 127, 128, 255, 256, 511, 512, 513, 767, 768, 9000, 16383, 16384, 16499}, modes=(1, 3))
    m.close()


@pytest.mark.parametrize("name,shape,maxSeq", [
    ("hd64", configs.Shape("g7-hd64-modes", 1, 896, 14, 2, 64, 256, 512, 1e-6, 1e6, True, True, "q8"), 8300),
    ("hd128", configs.Shape("g4-hd128-modes", 1, 1024, 8, 2, 128, 256, 512, 1e-5, 5e5, False, True, "q8"), 8300),
])
def test_fused_split_kv_matches_per_op_single_split(hip, name, shape, maxSeq):
    """The same long cache through the fused launches (split-KV, combine) and through the reference-order
    per-op launches (exec mode 0: one workgroup column per head group, no splits): two contexts are fed
    identical hidden vectors position by position, so both hold the same K/V rows; logits agree to rounding
    at positions spanning several splits.  GPU only, so the cache is filled quickly."""
    a = H.load_fast(shape, seed=55, maxSeq=maxSeq, eng=hip, oracle=False)
    b = H.load_fast(shape, seed=55, maxSeq=maxSeq, eng=hip, oracle=False)
    assert a.hip.SetExecMode(1) == 0
    assert b.hip.SetExecMode(0) == 0
    rng = np.random.default_rng(7)
    check = {0, 300, 2049, 6000, maxSeq - 1}
    for pos in range(maxSeq):
        h = rng.standard_normal(shape.dim).astype(np.float32)
        want = pos in check
        la = np.empty(shape.vocab, np.float32) if want else None
        lb = np.empty(shape.vocab, np.float32) if want else None
        assert a.hip.PartialStep(h, pos, 0, 1, None, la) == 0, E.last_error()
        assert b.hip.PartialStep(h, pos, 0, 1, None, lb) == 0, E.last_error()
        if want:
            print(f"  {name}: fused vs per-op at pos {pos}", flush=True)
            assert H.rel_err(la, lb) < 1e-5, pos
            assert H.rel_err(a.hip.ExportHidden(), b.hip.ExportHidden()) < 1e-5, pos
    a.close()
    b.close()

"""Graphs over a range of layers: the reference's CUDAGraph interface (cuda_graph.go:286-739).

CaptureGraph(cfg, pos) / Launch(pos) / UpdateAndLaunch / UploadHidden / ReadHidden / ValidateGraphCapture against
PartialStep on the same hidden states and positions: the graph replays the launches PartialStep issues, with the
position read from device memory instead of baked into the arguments, so the outputs are bit-identical.  The
reference's own criterion (largest difference < 1e-3, cuda_graph.go:590-597) is ValidateGraphCapture's.
"""
import numpy as np
import pytest

from mongoose_amd import configs
from mongoose_amd import engine as E
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _hiddens(s, n, seed):
    rng = np.random.default_rng(seed)
    return [rng.standard_normal(s.dim).astype(np.float32) for _ in range(n)]


@pytest.mark.parametrize("mode", [1, 3])
def test_graph_over_layer_ranges_equals_partial_step(hip, mode):
    s = configs.TOY
    m = H.Model(s, seed=21, maxSeq=32, eng=hip, threads=8)
    assert m.hip.SetExecMode(mode) == 0
    assert E.HasGraphKernel()
    assert m.hip.TestMinimalCapture()
    hs = _hiddens(s, 6, 1)
    for l0, l1 in ((0, s.nLayers), (0, 2), (2, s.nLayers), (1, 2)):
        # eager: the range at positions 0..5, each on its own input
        assert m.hip.ResetKV() == 0
        want = []
        for pos, h in enumerate(hs):
            assert m.hip.PartialStep(h, pos, l0, l1, None, None) == 0, E.last_error()
            want.append(m.hip.ExportHidden())
        # oracle on the same inputs, for the full range
        if (l0, l1) == (0, s.nLayers):
            m.orc.reset_kv()
            for pos, h in enumerate(hs):
                hid, _, _ = m.orc.step(h, pos, shadow=True)
                assert H.rel_err(want[pos], hid) < 1e-4
        # the graph: one capture, a launch per position
        assert m.hip.ResetKV() == 0
        g = m.hip.CaptureGraph(E.GraphCaptureConfig(LayerStart=l0, LayerEnd=l1, StreamCount=1), 0)
        assert g is not None, E.last_error()
        for pos, h in enumerate(hs):
            assert m.hip.UploadHidden(h) == 0
            if pos % 2 == 0:
                assert g.Launch(pos) == 0, E.last_error()
            else:
                assert m.hip.UpdateAndLaunch(g, pos)
            got = m.hip.ReadHidden()
            assert got is not None, E.last_error()
            assert np.array_equal(got, want[pos]), (l0, l1, pos, H.rel_err(got, want[pos]))
        g.Destroy()
    ok, md = m.hip.ValidateGraphCapture(hs[0], 0, s.nLayers)
    assert ok and md < 1e-3
    ok, md = m.hip.ValidateMultiStreamGraph(hs[0], 0, s.nLayers, 2)
    assert ok and md < 1e-3
    m.close()


def test_capture_config_errors_and_stale_graphs(hip):
    s = configs.TOY
    m = H.Model(s, seed=22, maxSeq=16, eng=hip, oracle=False)
    C = E.GraphCaptureConfig
    assert m.hip.CaptureGraph(C(0, s.nLayers, StreamCount=3), 0) is None and "StreamCount" in E.last_error()
    assert m.hip.CaptureGraph(C(0, s.nLayers, StreamCount=2, PipelineBreak=0), 0) is None and "PipelineBreak" in E.last_error()
    assert m.hip.CaptureGraph(C(0, s.nLayers + 1), 0) is None
    assert m.hip.CaptureGraph(C(2, 2), 0) is None
    assert m.hip.CaptureGraph(C(0, s.nLayers), 16) is None and "pos" in E.last_error()
    g2 = m.hip.CaptureGraph(C(0, s.nLayers, StreamCount=2, PipelineBreak=2), 0)          # the two-stage form
    assert g2 is not None, E.last_error()
    h = _hiddens(s, 1, 2)[0]
    assert m.hip.PartialStep(h, 0, 0, s.nLayers, None, None) == 0
    want = m.hip.ExportHidden()
    assert m.hip.ResetKV() == 0
    assert m.hip.UploadHidden(h) == 0 and g2.Launch(0) == 0
    assert np.array_equal(m.hip.ReadHidden(), want)
    assert g2.Launch(16) != 0                                                            # position outside the cache
    # a graph captured in one mode, launched after the mode changed: re-captured, same result to rounding
    assert m.hip.SetExecMode(3) == 0
    assert m.hip.ResetKV() == 0
    assert m.hip.UploadHidden(h) == 0 and g2.Launch(0) == 0, E.last_error()
    assert H.rel_err(m.hip.ReadHidden(), want) < 1e-5
    # exec mode 0 takes its positions from the host: no capture
    assert m.hip.SetExecMode(0) == 0
    assert m.hip.CaptureGraph(C(0, s.nLayers), 0) is None and "mode 0" in E.last_error()
    # a graph outlives its context as a dead handle
    m.hip.Close()
    assert g2.Launch(0) != 0 and "destroyed" in E.last_error()
    g2.Destroy()
    m.hip = None
    m.close()

"""mg_q8_gemm_noalloc: the multi-row Q8 product with its split planes in the library's static scratch
array (no allocation, no workspace) against mongoose_q8_gemm with a caller's workspace -- same kernels on
the same values, so the results must agree bit for bit.  Two calls in a row, the second with a smaller
input (the array then still holds the first call's planes), then an accumulate call and the size limit."""
import numpy as np
import pytest

from mongoose_amd import engine as E
from mongoose_amd.lib import lib
from oracle import binding as ob
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _up(eng, a):
    return eng.UploadRawBytes(np.ascontiguousarray(a))


def _run_both(hip, T, N, K, seed, bias, accumulate):
    rng = np.random.default_rng(seed)
    w = E.synth_normal(seed, N * 7 + K, 0.02, (N, K))
    q, s = ob.quantize_q8(w)
    act = rng.standard_normal((T, K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32) if bias else None
    y0 = rng.standard_normal((T, N)).astype(np.float32)
    dq, ds, da = _up(hip, q), _up(hip, s), _up(hip, act)
    db = _up(hip, b) if bias else None
    wsBytes = 4 * ((T + 127) // 128 * 128) * ((K + 63) // 64 * 64)
    # a workspace full of NaN patterns: nothing may depend on what it held
    ws = _up(hip, np.full(wsBytes, 0xFF, np.uint8))
    outs = []
    for which in (0, 1):
        dy = _up(hip, y0)
        if which == 0:
            E.KQ8Gemm(da, dq, ds, db, dy, T, N, K, accumulate, ws, wsBytes)
        else:
            assert E.KQ8GemmNoAlloc(da, dq, ds, db, dy, T, N, K, accumulate) == 0, E.last_error()
        E.KSync()
        assert E.HIPCheck() == 0
        outs.append(hip.DownloadRawBytes(dy, T * N * 4).view(np.float32).reshape(T, N).copy())
        dy.Release()
    for t in (dq, ds, da, ws) + ((db,) if bias else ()):
        t.Release()
    # and against the oracle's row-by-row matvec (double shadow), to the per-op bar
    deq = ob.dequant_q8(q, s).astype(np.float64)
    want = act.astype(np.float64) @ deq.T
    if bias:
        want += b
    if accumulate:
        want += y0
    return outs[0], outs[1], want


def test_noalloc_gemm_matches_workspace_gemm_two_calls_in_a_row(hip):
    assert lib.mg_q8_gemm_noalloc_max_bytes() == 8 << 20
    # first call: the largest K that fits 128 rows; second call: smaller in both T and K (K % 64 == 32)
    for (T, N, K, bias, acc) in [(100, 1000, 4096, True, False), (37, 300, 1376, False, False), (5, 64, 96, True, True)]:
        print(f"noalloc gemm T={T} N={N} K={K}", flush=True)
        a, b, want = _run_both(hip, T, N, K, seed=T + K, bias=bias, accumulate=acc)
        assert np.array_equal(a, b), (T, N, K)
        assert H.rel_err(b, want) < 1e-4, (T, N, K)


def test_noalloc_gemm_rejects_sizes_beyond_its_scratch(hip):
    d = hip.Zeros([64])
    # 4 * 128 * 16448 > 8 MiB ; 4 * 640 * 4096 > 8 MiB
    for (T, K) in [(1, 16416), (513, 4096)]:
        rc = lib.mg_q8_gemm_noalloc(d.DevicePtr(), d.DevicePtr(), d.DevicePtr(), None, d.DevicePtr(), T, 1, K, 0, None)
        assert rc == -2 and "exceed" in E.last_error(), (T, K, E.last_error())
    assert lib.mg_q8_gemm_noalloc(d.DevicePtr(), d.DevicePtr(), d.DevicePtr(), None, d.DevicePtr(), 4, 4, 48, 0, None) == -2
    # the exact limit is accepted
    T, K, N = 512, 4096, 8
    assert 4 * T * K == 8 << 20
    w = np.zeros((N, K), np.int8)
    dq, ds = hip.UploadRawBytes(w), hip.UploadRawBytes(np.ones(N, np.float32))
    da, dy = hip.Zeros([T * K]), hip.Zeros([T * N])
    assert E.KQ8GemmNoAlloc(da, dq, ds, None, dy, T, N, K, False) == 0, E.last_error()
    E.KSync()
    assert E.HIPCheck() == 0
    assert (hip.ToHost(dy) == 0).all()
    for t in (d, dq, ds, da, dy):
        t.Release()

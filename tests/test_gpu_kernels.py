"""Per-op parity on the GPU: each C-ABI launch against the CPU oracle on the
same seeded inputs.  Integer/byte results (dequantized weights, gathers,
copies) must be bit-exact; floating-point reductions are compared with the
oracle's float path and its double shadow at 1e-5 relative (stated per test),
far inside the 1e-4 per-layer bar."""
import numpy as np
import pytest

from mongoose_amd import engine as E
from oracle import binding as ob
from tests import helpers as H

pytestmark = pytest.mark.gpu
rng = np.random.default_rng(2024)

# (N, K) of every matvec in the five benchmark configurations
MATVEC_SHAPES = [
    (512, 512), (1376, 512), (512, 1376), (256, 512),                 # toy
    (896, 896), (128, 896), (4864, 896), (896, 4864),                 # qwen (lm_head below)
    (2048, 2048), (256, 2048), (5632, 2048), (2048, 5632), (32000, 2048),   # tinyllama
    (4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336),         # llama-3-8b
]


def _up(eng, a):
    return eng.UploadRawBytes(np.ascontiguousarray(a))


def _down(eng, t, dtype, n):
    return eng.DownloadRawBytes(t, n * np.dtype(dtype).itemsize).view(dtype)


def _check():
    E.KSync()
    assert E.HIPCheck() == 0


@pytest.mark.parametrize("N,K", MATVEC_SHAPES + [(151936, 896)])
def test_q8_matvec_rowscale(hip, N, K):
    print(f"q8 matvec N={N} K={K}", flush=True)
    w = E.synth_normal(5, N * 131 + K, 0.02, (N, K))
    q, s = ob.quantize_q8(w)
    act = rng.standard_normal(K).astype(np.float32)
    dq, ds, da = _up(hip, q), _up(hip, s), _up(hip, act)
    dout = hip.Zeros([N])
    E.KQ8MatvecRowScale(da, dq, ds, dout, N, K)
    _check()
    got = hip.ToHost(dout)
    ref32 = ob.q8_matvec(act, q, s, threads=8)
    ref64 = ob.q8_matvec(act, q, s, shadow=True, threads=8)
    assert H.rel_err(got, ref64) < 1e-5          # tolerance: 1e-5 of the largest output
    assert H.rel_err(got, ref32) < 1e-5
    for t in (dq, ds, da, dout):
        t.Release()


def test_q8_matvec_reference_scale_convention(hip):
    # mongoose_q8_matvec keeps the reference kernel's scales[r]/127 (mongoose.cu:1561)
    N, K = 640, 896
    w = E.synth_normal(6, 1, 0.02, (N, K))
    q, s = ob.quantize_q8(w)
    absmax = (s * np.float32(127.0)).astype(np.float32)
    act = rng.standard_normal(K).astype(np.float32)
    dq, ds, da, dout = _up(hip, q), _up(hip, absmax), _up(hip, act), hip.Zeros([N])
    E.KQ8Matvec(da, dq, ds, dout, N, K)
    _check()
    ref = ob.q8_matvec(act, q, (absmax / np.float32(127.0)).astype(np.float32), shadow=True)
    assert H.rel_err(hip.ToHost(dout), ref) < 1e-5


@pytest.mark.parametrize("N,K", [(7, 24), (33, 100), (5, 8)])
def test_q8_matvec_ragged_shapes(hip, N, K):
    # K not a multiple of 16 takes the generic kernel; N not a multiple of the row group
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    q, s = ob.quantize_q8(w)
    act = rng.standard_normal(K).astype(np.float32)
    dq, ds, da, dout = _up(hip, q), _up(hip, s), _up(hip, act), hip.Zeros([N])
    E.KQ8MatvecRowScale(da, dq, ds, dout, N, K)
    _check()
    assert H.rel_err(hip.ToHost(dout), ob.q8_matvec(act, q, s, shadow=True)) < 1e-5


def test_q8_matvec_empty_is_noop(hip):
    E.KQ8MatvecRowScale(None, None, None, None, 0, 896)
    _check()


@pytest.mark.parametrize("N,K", [(896, 896), (128, 896), (4864, 896), (896, 4864), (1024, 4096), (33, 64), (151936, 896)])
def test_q4_0_matvec_raw_and_planar(hip, N, K):
    print(f"q4_0 matvec N={N} K={K}", flush=True)
    w = E.synth_normal(8, N * 17 + K, 0.02, (N, K))
    blocks = ob.quantize_q4_0(w)
    act = rng.standard_normal(K).astype(np.float32)
    ref64 = ob.q4_0_matvec(act, blocks, N, K, shadow=True, threads=8)
    draw, da, dout = _up(hip, blocks), _up(hip, act), hip.Zeros([N])
    E.KQ4_0Matvec(da, draw, dout, N, K)
    _check()
    assert H.rel_err(hip.ToHost(dout), ref64) < 1e-5
    # device repack -> split layout -> fast kernel
    dplanar = hip.UploadRawBytes(np.zeros(blocks.size, np.uint8))
    E.KQ4_0Repack(draw, dplanar, N, K)
    dout2 = hip.Zeros([N])
    E.KQ4_0MatvecPlanar(da, dplanar, dout2, N, K)
    _check()
    assert H.rel_err(hip.ToHost(dout2), ref64) < 1e-5
    planar = hip.DownloadRawBytes(dplanar)
    b = blocks.reshape(-1, 18)
    assert (planar[: b.shape[0] * 16].reshape(-1, 16) == b[:, 2:]).all()
    assert (planar[b.shape[0] * 16:].reshape(-1, 2) == b[:, :2]).all()
    for t in (draw, da, dout, dplanar, dout2):
        t.Release()


def test_dequantized_weights_bit_exact(hip):
    rows, cols = 300, 896
    w = E.synth_normal(9, 3, 0.02, (rows, cols))
    q, s = ob.quantize_q8(w)
    dq, ds, dout = _up(hip, q), _up(hip, s), hip.Zeros([rows * cols])
    E.KDequantQ8RowScale(dq, ds, dout, rows, cols)
    _check()
    got = hip.ToHost(dout).reshape(rows, cols)
    assert (got.view(np.uint32) == ob.dequant_q8(q, s).view(np.uint32)).all()
    # reference convention (absmax scales, /127): mongoose.cu:1475-1487
    absmax = np.abs(w).max(axis=1).astype(np.float32)
    ds2 = _up(hip, absmax)
    E.KDequantInt8ToFP32(dq, ds2, dout, rows, cols)
    _check()
    ref = q.astype(np.float32) * (absmax / np.float32(127.0)).astype(np.float32)[:, None]
    assert (hip.ToHost(dout).reshape(rows, cols).view(np.uint32) == ref.view(np.uint32)).all()
    # Q4_0
    blocks = ob.quantize_q4_0(w)
    db = _up(hip, blocks)
    E.KDequantQ4_0(db, dout, rows, cols)
    _check()
    got4 = hip.ToHost(dout).reshape(rows, cols)
    assert (got4.view(np.uint32) == ob.dequant_q4_0(blocks, rows, cols).view(np.uint32)).all()


@pytest.mark.parametrize("dim,eps", [(512, 1e-5), (896, 1e-6), (4096, 1e-5), (100, 1e-5)])
def test_rmsnorm_out(hip, dim, eps):
    x = rng.standard_normal((3, dim)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    dx, dg, do = _up(hip, x), _up(hip, g), hip.Zeros([3 * dim])
    E.KRMSNormOutEps(dx, do, dg, 3, dim, eps)
    _check()
    got = hip.ToHost(do).reshape(3, dim)
    for r in range(3):
        assert H.rel_err(got[r], ob.rmsnorm_out(x[r], g, eps, shadow=True)) < 1e-6     # tolerance 1e-6
    E.KRMSNormOut(dx, do, dg, 3, dim)          # hard-coded 1e-6, mongoose.cu:170
    _check()
    assert H.rel_err(hip.ToHost(do).reshape(3, dim)[1], ob.rmsnorm_out(x[1], g, 1e-6, shadow=True)) < 1e-6


def test_rope_matches_oracle(hip):
    hd, nH, seq = 64, 14, 5
    dim = hd * nH
    c, s = ob.rope_tables(seq, hd, 1e6)
    x = rng.standard_normal((seq, dim)).astype(np.float32)
    dx, dc, ds = _up(hip, x), _up(hip, c), _up(hip, s)
    E.KRoPE(dx, dc, ds, seq, dim, hd, nH)
    _check()
    got = _down(hip, dx, np.float32, seq * dim).reshape(seq, dim)
    for p in range(seq):
        ref = ob.rope(x[p], c[p], s[p], nH, hd)
        assert np.abs(got[p] - ref).max() <= 1e-6          # one fma's rounding at most
    # decode form: seqLen 1 with the table pointer advanced to the position (cuda_fused_infer.go:423-426)
    dx1 = _up(hip, x[3])
    E.KRoPE(dx1, E.ptrAdd(dc.DevicePtr(), 3 * (hd // 2) * 4), E.ptrAdd(ds.DevicePtr(), 3 * (hd // 2) * 4), 1, dim, hd, nH)
    _check()
    assert (_down(hip, dx1, np.float32, dim) == got[3]).all()


@pytest.mark.parametrize("nH,nKV,hd,T", [(8, 8, 64, 1), (8, 8, 64, 72), (14, 2, 64, 216), (32, 4, 64, 300),
                                         (32, 8, 128, 700), (12, 1, 64, 40), (6, 2, 64, 257)])
def test_decode_attention(hip, nH, nKV, hd, T):
    print(f"attention nH={nH} nKV={nKV} hd={hd} T={T}", flush=True)
    dim, kvDim = nH * hd, nKV * hd
    Q = rng.standard_normal(dim).astype(np.float32)
    Kc = rng.standard_normal((T, kvDim)).astype(np.float32)
    Vc = rng.standard_normal((T, kvDim)).astype(np.float32)
    dq, dk, dv, do = _up(hip, Q), _up(hip, Kc), _up(hip, Vc), hip.Zeros([dim])
    E.KDecodeAttention(dq, dk, dv, do, T, dim, kvDim, nH, nKV)
    _check()
    got = hip.ToHost(do)
    ref = ob.decode_attention(Q, Kc, Vc, T, kvDim, nH, nKV, hd, shadow=True)
    assert H.rel_err(got, ref) < 1e-5            # tolerance 1e-5
    if T == 1:
        G = nH // nKV
        for h in range(nH):
            assert (got[h * hd:(h + 1) * hd] == Vc[0, (h // G) * hd:(h // G + 1) * hd]).all()


def test_elementwise_ops(hip):
    n = 4864
    g = (rng.standard_normal(n) * 3).astype(np.float32)
    u = rng.standard_normal(n).astype(np.float32)
    dg, du, do = _up(hip, g), _up(hip, u), hip.Zeros([n])
    E.KSiLUGateMul(dg, du, do, n)
    _check()
    assert H.rel_err(hip.ToHost(do), ob.silu_gate_mul(g, u, shadow=True)) < 1e-6
    E.KAddInPlace(dg, du, n)
    _check()
    assert (_down(hip, dg, np.float32, n) == g + u).all()
    # kv cache write: cache[pos*kvDim + i] = src[i]
    kvDim, maxSeq = 256, 8
    cache = hip.Zeros([maxSeq * kvDim])
    src = _up(hip, u[:kvDim])
    E.KKVCacheWrite(cache, src, 5, kvDim)
    _check()
    c = hip.ToHost(cache).reshape(maxSeq, kvDim)
    assert (c[5] == u[:kvDim]).all() and np.count_nonzero(np.delete(c, 5, axis=0)) == 0
    # embedding gather, copy, zero
    table = rng.standard_normal((50, 64)).astype(np.float32)
    toks = np.array([3, 49, 0, 3], np.int32)
    dt, dtok, dout = _up(hip, table), _up(hip, toks), hip.Zeros([4 * 64])
    E.KEmbedGather2(dout, dt, dtok, 4, 64)
    _check()
    assert (hip.ToHost(dout).reshape(4, 64) == table[toks]).all()
    E.KCopy(dout, dt, 4 * 64 * 4)
    _check()
    assert (hip.ToHost(dout).reshape(4, 64) == table[:4]).all()
    E.KZero(dout, 4 * 64 * 4 - 4)
    _check()
    z = hip.ToHost(dout)
    assert (z[:-1] == 0).all() and z[-1] == table[3, 63]


# ---- the symbols the tensor-typed helpers bind (kernel_tensor.go:23-40) ----
@pytest.mark.parametrize("N,K", [(896, 896), (128, 4864), (33, 70), (5, 2), (1000, 1376)])
def test_q4_rowscale_matvec(hip, N, K):
    """mongoose_q4_matvec (mongoose.cu:1598-1640): per-row-scale 4-bit, sequential nibble pairs, (nib-8)*s/7.
    Shapes with word-aligned rows and without (K/2 not a multiple of 4), a single byte per row."""
    packed = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    scales = rng.uniform(0.01, 0.3, N).astype(np.float32)
    act = rng.standard_normal(K).astype(np.float32)
    dw, ds, da = _up(hip, packed), _up(hip, scales), _up(hip, act)
    dout = hip.Zeros([N])
    E.TQ8Matvec(da, E.Q8Weight(dw, ds, N, K, Q4=True), dout)      # the route TQ8Matvec takes for Q4 weights
    _check()
    got = hip.ToHost(dout)
    assert H.rel_err(got, ob.q4_matvec(act, packed, scales, N, K, shadow=True)) < 1e-5
    assert H.rel_err(got, ob.q4_matvec(act, packed, scales, N, K)) < 1e-5
    for t in (dw, ds, da, dout):
        t.Release()


@pytest.mark.parametrize("seqLen,dim", [(1, 896), (3, 512), (2, 4096), (1, 100)])
def test_rmsnorm_in_place_and_fused_add(hip, seqLen, dim):
    """mongoose_rmsnorm (mongoose.cu:16-50, in place) and mongoose_fused_add_rmsnorm (:372-404), eps 1e-6 as
    the CUDA kernels hard-code; the _eps form against another eps; out aliasing an input."""
    x = rng.standard_normal((seqLen, dim)).astype(np.float32)
    y = rng.standard_normal((seqLen, dim)).astype(np.float32)
    g = (1.0 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    dx, dy, dg = _up(hip, x), _up(hip, y), _up(hip, g)
    dout = hip.Zeros([seqLen * dim])
    E.KFusedAddRMSNorm(dx, dy, dout, dg, seqLen, dim)
    _check()
    got = hip.ToHost(dout).reshape(seqLen, dim)
    for r in range(seqLen):
        assert H.rel_err(got[r], ob.fused_add_rmsnorm(x[r], y[r], g, 1e-6, shadow=True)) < 1e-6
    E.KFusedAddRMSNormEps(dx, dy, dout, dg, seqLen, dim, 0.25)
    _check()
    got = hip.ToHost(dout).reshape(seqLen, dim)
    for r in range(seqLen):
        assert H.rel_err(got[r], ob.fused_add_rmsnorm(x[r], y[r], g, 0.25, shadow=True)) < 1e-6
    E.KFusedAddRMSNorm(dx, dy, dy, dg, seqLen, dim)                # out aliases b
    _check()
    got = _down(hip, dy, np.float32, seqLen * dim).reshape(seqLen, dim)
    for r in range(seqLen):
        assert H.rel_err(got[r], ob.fused_add_rmsnorm(x[r], y[r], g, 1e-6, shadow=True)) < 1e-6
    E.TRMSNorm(dx, dg, seqLen, dim)                                # in place
    _check()
    got = _down(hip, dx, np.float32, seqLen * dim).reshape(seqLen, dim)
    for r in range(seqLen):
        assert H.rel_err(got[r], ob.rmsnorm_out(x[r], g, 1e-6, shadow=True)) < 1e-6
        assert H.rel_err(got[r], ob.rmsnorm_inplace(x[r], g, 1e-6)) < 1e-5     # the float path's serial sum of 4096 squares
    for t in (dx, dy, dg, dout):
        t.Release()


def test_zero_fill_unaligned(hip):
    """mongoose_zero on a range that starts and ends off a word boundary touches exactly its bytes."""
    buf = np.full(64, 0xAB, np.uint8)
    d = _up(hip, buf)
    E.KZero(d.DevicePtr() + 3, 22)
    _check()
    got = hip.DownloadRawBytes(d, 64)
    want = buf.copy()
    want[3:25] = 0
    assert np.array_equal(got, want)
    d.Release()


# ---------------------------------------------------------------------------
# The integer ("dp4a") forms of the Q4_0 matvec (kernels.go:66-70, 985-1017).
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("K,B", [(32, 1), (896, 1), (4864, 1), (14336, 1), (896, 5)])
def test_q8_quantize_act_bytes_equal_the_oracle(hip, K, B):
    """Activation blocks (40 bytes per 32 values): the same bytes as the oracle's, zero blocks and single spikes
    included; the batch form quantizes B contiguous vectors."""
    x = rng.standard_normal(K * B).astype(np.float32)
    x[:32] = 0.0
    if K >= 96:
        x[32:64] = 0.0
        x[40] = 7.25
    want = np.concatenate([ob.q8_quantize_act(x[b * K:(b + 1) * K]) for b in range(B)])
    dx = _up(hip, x)
    dq = hip.UploadRawBytes(np.full(want.size, 0xAA, np.uint8))
    if B == 1:
        E.KQ8QuantizeAct(dx, dq, K)
    else:
        E.KQ8QuantizeActBatch(dx, dq, K, B)
    _check()
    assert np.array_equal(hip.DownloadRawBytes(dq), want)
    dx.Release()
    dq.Release()


@pytest.mark.parametrize("N,K", [(896, 896), (128, 896), (4864, 896), (896, 4864), (1001, 64), (4096, 14336)])
def test_q4_0_matvec_dp4a_forms(hip, N, K):
    """mongoose_q4_0_matvec_dp4a (quantizes into the caller's scratch), _preq (takes quantized blocks) and _batch against
    the oracle's integer matvec at 1e-5 (the integer block sums are exact; the floats differ by summation order), and
    against the fp32-activation matvec within the activation rounding (what the reference's own check logs,
    cuda_fused_infer_q4.go:633-662)."""
    print(f"q4_0 dp4a N={N} K={K}", flush=True)
    w = E.synth_normal(18, N * 19 + K, 0.02, (N, K))
    blocks = ob.quantize_q4_0(w)
    B = 3
    acts = rng.standard_normal(K * B).astype(np.float32)
    q8 = [ob.q8_quantize_act(acts[b * K:(b + 1) * K]) for b in range(B)]
    ref = [ob.q4_0_matvec_q8act(q8[b], blocks, N, K, shadow=True, threads=8) for b in range(B)]
    dw, da = _up(hip, blocks), _up(hip, acts)
    dscratch = hip.UploadRawBytes(np.zeros(K // 32 * 40, np.uint8))
    dout = hip.Zeros([N])
    E.KQ4_0MatvecDP4A(da, dw, dout, dscratch, N, K)
    _check()
    got = hip.ToHost(dout)
    assert H.rel_err(got, ref[0]) < 1e-5
    assert np.array_equal(hip.DownloadRawBytes(dscratch), q8[0])
    exact = ob.q4_0_matvec(acts[:K], blocks, N, K, shadow=True, threads=8)
    assert H.rel_err(got, exact) < 3e-2
    dout2 = hip.Zeros([N])
    E.KQ4_0MatvecDP4APreq(dw, dscratch, dout2, N, K)
    _check()
    assert np.array_equal(hip.ToHost(dout2), got)
    dq8 = hip.UploadRawBytes(np.zeros(K // 32 * 40 * B, np.uint8))
    E.KQ8QuantizeActBatch(da, dq8, K, B)
    doutB = hip.Zeros([B * N])
    E.KQ4_0MatvecDP4ABatch(dw, dq8, doutB, N, K, B)
    _check()
    gotB = hip.ToHost(doutB).reshape(B, N)
    for b in range(B):
        assert H.rel_err(gotB[b], ref[b]) < 1e-5, b
    assert np.array_equal(gotB[0], got)
    for t in (dw, da, dscratch, dout, dout2, dq8, doutB):
        t.Release()

"""Pins the CPU oracle: the reference's own known-answer tests (cpu_test.go),
then closed forms, invariants, brute force and an independently written numpy
restatement for everything the reference holds no vector for."""
import numpy as np
import pytest

from oracle import binding as ob
from tests import np_reference as npr

rng = np.random.default_rng(1234)


# ---- cpu_test.go KATs -------------------------------------------------------
def test_matmul_2x3_3x2():
    # cpu_test.go:17-29
    a = np.array([1, 2, 3, 4, 5, 6], np.float32)
    b = np.array([7, 8, 9, 10, 11, 12], np.float32)
    out = np.zeros(4, np.float32)
    ob.lib.orc_matmul(ob.fp(a), ob.fp(b), 2, 3, 2, ob.fp(out))
    assert np.abs(out - np.array([58, 64, 139, 154], np.float32)).max() <= 0.001


def test_matmul_identity():
    # cpu_test.go:31-42
    eye = np.eye(3, dtype=np.float32).ravel()
    x = np.arange(1, 10, dtype=np.float32)
    out = np.zeros(9, np.float32)
    ob.lib.orc_matmul(ob.fp(x), ob.fp(eye), 3, 3, 3, ob.fp(out))
    assert np.abs(out - x).max() <= 0.001


def test_softmax_invariants():
    # cpu_test.go:57-76
    x = np.array([1, 2, 3], np.float32)
    ob.lib.orc_softmax(ob.fp(x), 3)
    assert abs(float(x.sum()) - 1.0) <= 0.001
    assert ((x >= 0) & (x <= 1)).all()
    assert x[2] > x[1] > x[0]
    # closed form
    ref = np.exp(np.array([1, 2, 3], np.float64))
    ref /= ref.sum()
    assert np.abs(x - ref).max() < 1e-7


def test_rmsnorm_kat():
    # cpu_test.go:78-92
    x = np.array([1, 2, 3, 4], np.float32)
    w = np.ones(4, np.float32)
    ob.lib.orc_rmsnorm(ob.fp(x), ob.fp(w), 4, 1e-5)
    rms = np.sqrt((x.astype(np.float64) ** 2).mean())
    assert abs(rms - 1.0) <= 0.1
    # closed form: x / sqrt(7.5 + 1e-5)
    ref = np.array([1, 2, 3, 4], np.float64) / np.sqrt(7.5 + np.float64(np.float32(1e-5)))
    assert np.abs(x - ref).max() < 1e-6


def test_rmsnorm_out_gain_and_eps():
    x = rng.standard_normal(896).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(896)).astype(np.float32)
    for eps in (1e-5, 1e-6):
        ref = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean() + np.float64(np.float32(eps))) * g
        assert np.abs(ob.rmsnorm_out(x, g, eps) - ref).max() < 5e-6
        assert np.abs(ob.rmsnorm_out(x, g, eps, shadow=True) - ref).max() < 1e-12
    # eps matters when the input is tiny: a dropped eps would blow this up
    tiny = np.full(64, 1e-4, np.float32)
    out = ob.rmsnorm_out(tiny, np.ones(64, np.float32), 1e-5)
    assert np.allclose(out, 1e-4 / np.sqrt(1e-8 + 1e-5), rtol=1e-5)


# ---- fp16 -------------------------------------------------------------------
def test_f16_decode_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([ob.lib.orc_f16_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(ref)
    assert (np.isnan(got) == nan).all()
    assert (got[~nan].view(np.uint32) == ref[~nan].view(np.uint32)).all()


def test_f16_encode_matches_numpy_rne():
    # every fp16 value, its neighbours' midpoints (ties) and random floats
    halfs = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = ((halfs[:-1].astype(np.float64) + halfs[1:].astype(np.float64)) / 2).astype(np.float32)
    rnd = (rng.standard_normal(20000) * 10.0 ** rng.uniform(-9, 5, 20000)).astype(np.float32)
    special = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                        np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -26, 6.1e-5], np.float32)
    xs = np.concatenate([halfs, -halfs, mids, -mids, rnd, special])
    with np.errstate(over="ignore"):
        ref = xs.astype(np.float16).view(np.uint16)
    got = np.array([ob.lib.orc_f32_to_f16(float(x)) for x in xs], np.uint16)
    assert (got == ref).all(), np.nonzero(got != ref)[0][:10]


# ---- Q8 quantizer -----------------------------------------------------------
@pytest.mark.parametrize("mode", [0, 1])
def test_q8_quantizer_vs_numpy_and_invariants(mode):
    w = (rng.standard_normal((37, 896)) * 0.02).astype(np.float32)
    w[3] = 0.0                        # zero row
    w[4] = 0.5                        # all equal
    w[5] = 0.0
    w[5, 17] = -3.0                   # single spike
    w[6] = 1e-41                      # denormals
    q, s = ob.quantize_q8(w, mode)
    qn, sn = npr.quantize_q8(w, mode)
    assert (s.view(np.uint32) == sn.view(np.uint32)).all()
    assert (q == qn).all()
    assert (q[3] == 0).all() and s[3] == 0
    nz = s > 0
    nz[6] = False     # denormal scale: 1/s overflows, the reference's result there is -128 everywhere (mode 0)
    assert np.abs(q[nz].astype(np.int32)).max() <= 127
    # the row extreme maps to +-127 (up to the one-step truncation slack)
    top = np.abs(q[nz].astype(np.int32)).max(axis=1)
    assert ((top == 127) | (top == 126)).all()
    assert (q[5, 17] in (-127, -126)) and np.count_nonzero(q[5]) == 1
    # scale convention: absmax/127 (cuda_fused_infer.go:373-374)
    assert np.allclose(s, np.abs(w).max(axis=1) / 127.0, rtol=1e-6)
    # truncation never rounds away from zero; rounding is within half a step
    deq = ob.dequant_q8(q, s)
    err = np.abs(deq - w)
    step = s[:, None]
    assert (err[nz] <= (step[nz] * (1.0001 if mode == 0 else 0.5001) + 1e-12)).all()
    if mode == 0:
        assert (np.abs(deq[nz]) <= np.abs(w[nz]) * (1 + 1e-6) + 1e-12).all()
    # dequant is one float multiply: exact
    assert (deq.view(np.uint32) == (q.astype(np.float32) * s[:, None]).view(np.uint32)).all()


# ---- Q4_0 -------------------------------------------------------------------
def test_q4_0_quantizer_vs_numpy_and_closed_form():
    w = (rng.standard_normal((16, 256)) * 0.02).astype(np.float32)
    w[0, :32] = 0.0                              # zero block
    w[1, :32] = np.linspace(-0.8, 0.7, 32)       # negative extreme -> d > 0
    w[2, :32] = np.linspace(-0.7, 0.8, 32)       # positive extreme -> d < 0
    blocks = ob.quantize_q4_0(w)
    assert (blocks == npr.quantize_q4_0(w)).all()
    b = blocks.reshape(-1, 18)
    # zero block: d == 0 (0/-8 is -0.0, bits 0x8000), every nibble == 8
    assert b[0, :2].copy().view(np.float16)[0] == 0 and (b[0, 2:] == 0x88).all()
    # signed extreme maps to nibble 0 (value -8*d == max) and d = max/-8
    d1 = b[8, :2].copy().view(np.float16)[0]
    assert d1 > 0 and np.isclose(float(d1), 0.8 / 8, rtol=1e-3)
    assert (b[8, 2] & 0x0F) == 0
    d2 = b[16, :2].copy().view(np.float16)[0]
    assert d2 < 0 and np.isclose(float(d2), -0.8 / 8, rtol=1e-3)
    assert (b[16, 2 + 15] >> 4) == 0             # element 31 is the high nibble of byte 15
    deq = ob.dequant_q4_0(blocks, 16, 256)
    assert (deq.view(np.uint32) == npr.dequant_q4_0(blocks, 16, 256).view(np.uint32)).all()
    # reconstruction error is at most one quantization step
    dabs = np.abs(b[:, :2].copy().view(np.float16).astype(np.float32)).reshape(16, 8)
    assert (np.abs(deq - w).reshape(16, 8, 32) <= dabs[:, :, None] * 1.001 + 1e-9).all()


def test_q4_0_dequant_brute_force_all_scales_and_nibbles():
    # all 2^16 fp16 scales x 16 nibble values (2^20 cases), both nibble positions
    scales = np.arange(65536, dtype=np.uint16)
    fin = np.isfinite(scales.view(np.float16))
    scales = scales[fin]
    n = scales.size
    blocks = np.zeros((n, 18), np.uint8)
    blocks[:, :2] = scales.view(np.uint8).reshape(-1, 2)
    for j in range(16):
        blocks[:, 2 + j] = (j | ((15 - j) << 4))
    deq = ob.dequant_q4_0(blocks.ravel(), n, 32)
    d = scales.view(np.float16).astype(np.float32)
    for j in range(16):
        assert (deq[:, j].view(np.uint32) == (np.float32(j - 8) * d).view(np.uint32)).all()
        assert (deq[:, 16 + j].view(np.uint32) == (np.float32(15 - j - 8) * d).view(np.uint32)).all()


# ---- matvec -----------------------------------------------------------------
def test_q8_matvec_is_matmul_on_dequantized_weights():
    w = (rng.standard_normal((24, 64)) * 0.02).astype(np.float32)
    q, s = ob.quantize_q8(w)
    act = rng.standard_normal(64).astype(np.float32)
    deq = ob.dequant_q8(q, s)
    ref = np.zeros(24, np.float32)
    bT = np.ascontiguousarray(deq.T)                       # [K, N], cpu.go MatMul layout
    ob.lib.orc_matmul(ob.fp(act), ob.fp(bT), 1, 64, 24, ob.fp(ref))
    got = ob.q8_matvec(act, q, s)
    assert (got.view(np.uint32) == ref.view(np.uint32)).all()
    assert np.abs(ob.q8_matvec(act, q, s, shadow=True) - deq.astype(np.float64) @ act).max() < 1e-14


def test_q4_0_matvec_is_matmul_on_dequantized_weights():
    w = (rng.standard_normal((12, 96)) * 0.02).astype(np.float32)
    blocks = ob.quantize_q4_0(w)
    act = rng.standard_normal(96).astype(np.float32)
    deq = ob.dequant_q4_0(blocks, 12, 96)
    ref = np.zeros(12, np.float32)
    bT = np.ascontiguousarray(deq.T)
    ob.lib.orc_matmul(ob.fp(act), ob.fp(bT), 1, 96, 12, ob.fp(ref))
    got = ob.q4_0_matvec(act, blocks, 12, 96)
    assert (got.view(np.uint32) == ref.view(np.uint32)).all()
    # element order: unit activations pick out single dequantized weights
    for k in (0, 15, 16, 31, 32, 95):
        e = np.zeros(96, np.float32)
        e[k] = 1.0
        assert (ob.q4_0_matvec(e, blocks, 12, 96) == deq[:, k]).all()


# ---- RoPE -------------------------------------------------------------------
def test_rope_tables_and_invariants():
    hd, nH, theta = 64, 4, 1e6
    c, s = ob.rope_tables(32, hd, theta)
    cn, sn = npr.rope_tables(32, hd, theta)
    assert np.abs(c - cn).max() < 1e-7 and np.abs(s - sn).max() < 1e-7
    assert (c[0] == 1).all() and (s[0] == 0).all()
    # frequency of pair j: theta^(-2j/hd); j=0 rotates by `pos` radians
    assert np.isclose(c[5, 0], np.cos(5.0), atol=1e-7) and np.isclose(s[5, 0], np.sin(5.0), atol=1e-7)
    assert np.isclose(s[7, 16], np.sin(7.0 * theta ** (-32 / 64)), atol=1e-9)
    x = rng.standard_normal(nH * hd)
    # pos 0 is the identity
    assert (ob.rope(x, c[0], s[0], nH, hd, shadow=True) == x).all()
    # rotate-half pairing (j, j+hd/2): a unit vector at j rotates into j+hd/2
    e = np.zeros(nH * hd)
    e[3] = 1.0
    r = ob.rope(e, c[9], s[9], nH, hd, shadow=True)
    assert np.isclose(r[3], c[9, 3]) and np.isclose(r[3 + 32], s[9, 3]) and np.count_nonzero(r) == 2
    # norm preserving per pair
    y = ob.rope(x, c[11], s[11], nH, hd, shadow=True).reshape(nH, hd)
    xx = x.reshape(nH, hd)
    assert np.allclose(y[:, :32] ** 2 + y[:, 32:] ** 2, xx[:, :32] ** 2 + xx[:, 32:] ** 2, rtol=1e-6)
    # relative-position property: <R_m q, R_n k> depends on m-n only
    q, k = rng.standard_normal(hd), rng.standard_normal(hd)
    d1 = ob.rope(q, c[10], s[10], 1, hd, shadow=True) @ ob.rope(k, c[4], s[4], 1, hd, shadow=True)
    d2 = ob.rope(q, c[16], s[16], 1, hd, shadow=True) @ ob.rope(k, c[10], s[10], 1, hd, shadow=True)
    assert abs(d1 - d2) < 1e-5 * max(1.0, abs(d1))


# ---- attention --------------------------------------------------------------
def test_attention_invariants_and_gqa():
    hd, nH, nKV = 64, 6, 2
    kvDim = nKV * hd
    T = 9
    Q = rng.standard_normal(nH * hd)
    Kc = rng.standard_normal((T, kvDim))
    Vc = rng.standard_normal((T, kvDim))
    # cacheLen 1: output is V exactly, whatever q and k are
    out = ob.decode_attention(Q, Kc, Vc, 1, kvDim, nH, nKV, hd, shadow=True).reshape(nH, hd)
    for h in range(nH):
        assert (out[h] == Vc[0, (h // 3) * hd:(h // 3 + 1) * hd]).all()
    # identical keys: uniform weights, output is the mean of V
    Ku = np.tile(Kc[0], (T, 1))
    out = ob.decode_attention(Q, Ku, Vc, T, kvDim, nH, nKV, hd, shadow=True).reshape(nH, hd)
    for h in range(nH):
        assert np.allclose(out[h], Vc[:, (h // 3) * hd:(h // 3 + 1) * hd].mean(axis=0), atol=1e-12)
    # brute force, including the 1/sqrt(hd) scale and kvHead = h // (nH/nKV)
    out = ob.decode_attention(Q, Kc, Vc, T, kvDim, nH, nKV, hd, shadow=True).reshape(nH, hd)
    for h in range(nH):
        kvh = h // (nH // nKV)
        sc = Kc[:, kvh * hd:(kvh + 1) * hd] @ Q[h * hd:(h + 1) * hd] / np.sqrt(hd)
        p = np.exp(sc - sc.max())
        p /= p.sum()
        assert np.allclose(out[h], p @ Vc[:, kvh * hd:(kvh + 1) * hd], atol=1e-12)
    # float path agrees with the shadow
    o32 = ob.decode_attention(Q.astype(np.float32), Kc.astype(np.float32), Vc.astype(np.float32), T, kvDim, nH, nKV, hd)
    assert np.abs(o32 - out.ravel()).max() < 1e-5


def test_silu_gate_mul_closed_form():
    g = np.linspace(-30, 30, 301)
    u = rng.standard_normal(301)
    ref = g / (1 + np.exp(-g)) * u
    assert np.abs(ob.silu_gate_mul(g, u, shadow=True) - ref).max() < 1e-12
    assert np.abs(ob.silu_gate_mul(g.astype(np.float32), u.astype(np.float32)) - ref).max() < 1e-5
    z = ob.silu_gate_mul(np.zeros(4), np.ones(4), shadow=True)
    assert (z == 0).all()


def test_argmax_lowest_index_on_ties():
    x = np.array([1, 5, 5, 2, 5], np.float32)
    assert ob.lib.orc_argmax(ob.fp(x), 5) == 1


# ---- per-row-scale 4-bit matvec (mongoose_q4_matvec, kernels/mongoose.cu:1598-1630) ----
def _dense_q4_rowscale(packed, scales, N, K):
    """Element 2k = low nibble of byte k, element 2k+1 = high nibble; value (nib-8) * (s/7), in float."""
    b = np.asarray(packed, np.uint8).reshape(N, K // 2)
    s7 = (np.asarray(scales, np.float32) / np.float32(7.0)).astype(np.float32)
    w = np.empty((N, K), np.float32)
    w[:, 0::2] = ((b & 0x0F).astype(np.int32) - 8).astype(np.float32) * s7[:, None]
    w[:, 1::2] = ((b >> 4).astype(np.int32) - 8).astype(np.float32) * s7[:, None]
    return w


def test_q4_rowscale_matvec_unit_activations_pick_single_nibbles():
    """A unit activation at element e returns, for every row, exactly that element's dequantized
    weight: pins which nibble is which element, the -8 offset and the /7."""
    N, K = 3, 8
    packed = np.array([[0x10, 0x32, 0x54, 0xF6], [0x8F, 0x08, 0x80, 0x77], [0xFF, 0x00, 0xA5, 0x5A]], np.uint8)
    scales = np.array([7.0, 3.5, 0.25], np.float32)
    for e in range(K):
        act = np.zeros(K, np.float32)
        act[e] = 1.0
        got = ob.q4_matvec(act, packed, scales, N, K)
        byte = packed[:, e // 2]
        nib = (byte & 0x0F) if e % 2 == 0 else (byte >> 4)
        want = (nib.astype(np.int32) - 8).astype(np.float32) * (scales / np.float32(7.0)).astype(np.float32)
        assert (got == want).all(), e
    # row 0 with scale 7: the weights are the integers nib - 8 themselves
    act = np.ones(K, np.float32)
    assert ob.q4_matvec(act, packed, scales, N, K)[0] == sum(n - 8 for n in (0, 1, 2, 3, 4, 5, 6, 15))


def test_q4_rowscale_matvec_equals_matmul_over_dequantized_weights():
    rng = np.random.default_rng(17)
    N, K = 37, 96
    packed = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    scales = rng.uniform(0.01, 0.2, N).astype(np.float32)
    act = rng.standard_normal(K).astype(np.float32)
    w = _dense_q4_rowscale(packed, scales, N, K)
    got64 = ob.q4_matvec(act, packed, scales, N, K, shadow=True)
    assert np.allclose(got64, w.astype(np.float64) @ act.astype(np.float64), rtol=1e-12, atol=1e-14)
    got32 = ob.q4_matvec(act, packed, scales, N, K)
    assert H_rel(got32, got64) < 1e-5
    # a zero scale row gives zero; K = 2 is the smallest row
    assert ob.q4_matvec(np.ones(2, np.float32), np.array([[0xF0]], np.uint8), np.array([0.0], np.float32), 1, 2)[0] == 0.0


def H_rel(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / np.abs(b).max())


def test_fused_add_rmsnorm_is_rmsnorm_of_the_sum():
    """kernels/mongoose.cu:372-404 against CPU.RMSNorm (cpu.go:36-47) applied to a + b."""
    rng = np.random.default_rng(23)
    n = 896
    a = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    g = (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    for eps in (1e-6, 1e-5, 0.5):
        got = ob.fused_add_rmsnorm(a, b, g, eps)
        want = ob.rmsnorm_inplace((a + b).astype(np.float32), g, eps)
        assert (got == want).all()
    # b = -a: the sum is zero and so is the output, whatever eps (> 0) is
    assert (ob.fused_add_rmsnorm(a, -a, g, 1e-6) == 0).all()
    # closed form in double
    s = a.astype(np.float64) + b.astype(np.float64)
    want64 = s / np.sqrt((s * s).mean() + 1e-6) * g
    assert H_rel(ob.fused_add_rmsnorm(a, b, g, 1e-6, shadow=True), want64) < 1e-12


# ---------------------------------------------------------------------------
# The integer ("dp4a") Q4_0 matvec: activation blocks and the block dot product
# (kernels.go:66-70, 985-1017; the CUDA bodies are absent from the reference, so these
# closed forms and the independent restatement are what pins the oracle's functions).
# ---------------------------------------------------------------------------
def _np_q8_blocks(x):
    """Independent numpy restatement of the activation quantizer: per 32 values d = amax/127 (float32),
    q = round half away from zero of x * (1/d), s = d * sum(q)."""
    x = np.asarray(x, np.float32).reshape(-1, 32)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    idv = np.zeros_like(d)
    nz = d != 0
    idv[nz] = (np.float32(1.0) / d[nz]).astype(np.float32)
    v = (x * idv[:, None]).astype(np.float32).astype(np.float64)
    q = (np.sign(v) * np.floor(np.abs(v) + 0.5)).astype(np.int32)
    s = (d * q.sum(axis=1).astype(np.float32)).astype(np.float32)
    return d, s, q.astype(np.int8)


def _split_q8(blocks):
    b = np.asarray(blocks, np.uint8).reshape(-1, 40)
    return b[:, :4].copy().view(np.float32)[:, 0], b[:, 4:8].copy().view(np.float32)[:, 0], b[:, 8:].copy().view(np.int8)


def test_q8_activation_blocks_closed_forms_and_numpy():
    rng = np.random.default_rng(77)
    x = rng.standard_normal(32 * 40).astype(np.float32)
    x[64:96] = 0.0                                  # a zero block
    x[96:128] = 0.0
    x[100] = -3.5                                   # a single spike: it alone maps to -127
    x[128:160] = 1e-30                              # tiny equal values: all +127
    d, s, q = _split_q8(ob.q8_quantize_act(x))
    nd, ns, nq = _np_q8_blocks(x)
    assert np.array_equal(d, nd) and np.array_equal(s, ns) and np.array_equal(q, nq)
    xb = x.reshape(-1, 32)
    assert d[2] == 0 and s[2] == 0 and not q[2].any()
    assert q[3][4] == -127 and np.count_nonzero(q[3]) == 1 and d[3] == np.float32(3.5) / np.float32(127)
    assert (q[4] == 127).all()
    for b in range(xb.shape[0]):
        if d[b] == 0:
            continue
        i = int(np.abs(xb[b]).argmax())
        assert abs(int(q[b][i])) == 127                               # the extreme maps to +-127
        assert np.abs(xb[b] - q[b].astype(np.float64) * d[b]).max() <= 0.5 * d[b] * (1 + 1e-6)
        assert s[b] == np.float32(d[b] * np.float32(q[b].astype(np.int64).sum()))


def test_integer_q4_0_matvec_is_the_fp32_matvec_on_the_quantized_activations():
    """sum_b d4 (d8 sumi - 8 s8) == sum_k deq(W)[r,k] * (q[k] d8[block of k]) in exact arithmetic: the double shadow of
    the integer form against the (pinned) fp32-activation matvec fed the dequantized activation blocks."""
    rng = np.random.default_rng(78)
    N, K = 37, 896
    w = rng.standard_normal((N, K)).astype(np.float32) * 0.02
    blocks = ob.quantize_q4_0(w)
    act = rng.standard_normal(K).astype(np.float32)
    q8 = ob.q8_quantize_act(act)
    d, s, q = _split_q8(q8)
    act_hat = (q.astype(np.float64) * d.astype(np.float64)[:, None]).reshape(-1)
    want = ob.q4_0_matvec(act_hat, blocks, N, K, shadow=True)
    got64 = ob.q4_0_matvec_q8act(q8, blocks, N, K, shadow=True)
    got32 = ob.q4_0_matvec_q8act(q8, blocks, N, K)
    den = np.abs(want).max()
    assert np.abs(got64 - want).max() / den < 1e-6          # s8 is d*sum rounded to float: 6e-8 of the -8 term
    assert np.abs(got32 - want).max() / den < 1e-5
    # and it is the fp32-activation result up to the activation rounding (half a step of 1/127 of the block maximum)
    exact = ob.q4_0_matvec(act, blocks, N, K, shadow=True)
    err = np.abs(got64 - exact).max() / np.abs(exact).max()
    assert 1e-5 < err < 3e-2, err


def test_integer_q4_0_matvec_element_order():
    """One activation per run: it quantizes to +127 with d = x/127, so row r gives d4 * (nib - 8) * x -- which picks
    the nibble that belongs to element k (low nibble of byte j = element j, high nibble = element j + 16)."""
    rng = np.random.default_rng(79)
    N, K = 3, 64
    w = rng.standard_normal((N, K)).astype(np.float32)
    blocks = ob.quantize_q4_0(w)
    deq = ob.dequant_q4_0(blocks, N, K)
    for k in (0, 1, 15, 16, 17, 31, 32, 47, 63):
        act = np.zeros(K, np.float32)
        act[k] = 2.5
        got = ob.q4_0_matvec_q8act(ob.q8_quantize_act(act), blocks, N, K, shadow=True)
        assert np.allclose(got, deq[:, k].astype(np.float64) * 2.5, rtol=1e-6, atol=1e-6), k     # a nibble of 8: zero up to the rounding of s = d * sum(q)

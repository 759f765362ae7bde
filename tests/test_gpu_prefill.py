"""Batched prefill (MFMA GEMM path) against the token-by-token decode step.

The reference has no batched prompt path: its semantics for a prompt are the
decode step applied position by position, which is what the oracle does here.
Bars: last-position logits within 1e-3 relative of the oracle (float path and
double shadow), greedy tokens identical, and the decode that continues from
the prefilled KV caches identical to the all-decode run (which checks every
cache row the prefill wrote).  The GEMM itself is compared with a float64
product at 2e-5 of the largest output (int8 weights are exact in bf16; the
two-term bf16 split of an activation leaves 2^-16 relative)."""
import numpy as np
import pytest

from mongoose_amd import configs
from mongoose_amd import engine as E
from oracle import binding as ob
from tests import helpers as H

pytestmark = pytest.mark.gpu
rng = np.random.default_rng(77)


def _up(eng, a):
    return eng.UploadRawBytes(np.ascontiguousarray(a))


@pytest.mark.parametrize("T,N,K,acc,bias", [
    (1, 128, 32, False, False), (5, 100, 64, False, True), (130, 300, 896, True, False),
    (128, 128, 4864, False, False), (257, 1376, 512, True, True), (512, 1024, 4096, False, False),
    # enough 256 x 256 tiles for the direct-to-LDS ring kernel: accumulate form, bias form, odd count of 32-wide K steps
    (512, 12288, 64, True, False), (300, 12800, 96, False, True),
])
def test_q8_gemm_against_float64(hip, T, N, K, acc, bias):
    print(f"q8 gemm T={T} N={N} K={K} acc={acc} bias={bias}", flush=True)
    w = E.synth_normal(9, T * 7 + N, 0.02, (N, K))
    q, s = ob.quantize_q8(w)
    a = rng.standard_normal((T, K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32) if bias else None
    y0 = rng.standard_normal((T, N)).astype(np.float32)
    plane = 2 * ((T + 127) // 128 * 128) * ((K + 63) // 64 * 64)
    dq, ds, da, dy = _up(hip, q), _up(hip, s), _up(hip, a), _up(hip, y0)
    db = _up(hip, b) if bias else None
    ws = hip.UploadRawBytes(np.zeros(2 * plane, np.uint8))
    E.KQ8Gemm(da, dq, ds, db, dy, T, N, K, acc, ws, 2 * plane)
    E.KSync()
    assert E.HIPCheck() == 0
    got = hip.DownloadRawBytes(dy, T * N * 4).view(np.float32).reshape(T, N)
    ref = (a.astype(np.float64) @ q.astype(np.float64).T) * s.astype(np.float64)[None, :]
    if bias:
        ref = ref + b.astype(np.float64)[None, :]
    if acc:
        ref = ref + y0.astype(np.float64)
    assert H.rel_err(got, ref) < 2e-5
    # row 0 is also what the decode matvec gives for the same activation
    if not acc and not bias:
        mv = ob.q8_matvec(a[0], q, s, shadow=True, threads=4)
        assert H.rel_err(got[0], mv) < 2e-5
    for t in (dq, ds, da, dy, ws) + ((db,) if bias else ()):
        t.Release()


def test_q8_gemm_rejects_bad_arguments(hip):
    t = hip.Zeros([64])
    E.KQ8Gemm(t, t, t, None, t, 1, 1, 31, False, t, 256)      # K not a multiple of 32
    E.KSync()
    assert E.HIPCheck() != 0
    E.KQ8Gemm(t, t, t, None, t, 1, 1, 32, False, t, 16)       # workspace too small
    E.KSync()
    assert E.HIPCheck() != 0
    assert E.HIPCheck() == 0                                    # the error is reported once
    t.Release()


def _oracle_prompt_logits(m, prompt, shadow):
    m.orc.reset_kv()
    logits = None
    for pos, tok in enumerate(prompt):
        _, logits, _ = m.orc.decode_token(int(tok), pos, shadow=shadow, want_layers=False)
    return logits.copy()


def _prefill_case(hip, s, seed, nPrompt, nDecode, maxSeq, kv_f16=False):
    m = H.Model(s, seed=seed, maxSeq=maxSeq, eng=hip, threads=8, kv_f16=kv_f16)
    prompt = m.prompt(nPrompt)
    lg32 = _oracle_prompt_logits(m, prompt, False)
    lg64 = _oracle_prompt_logits(m, prompt, True)
    assert m.hip.ResetKV() == 0
    rc, nxt, logits, ms = m.hip.Prefill(prompt, 0, wantLogits=True)
    assert rc == 0, E.last_error()
    assert ms > 0
    assert H.rel_err(logits, lg64) < 1e-3 and H.rel_err(logits, lg32) < 1e-3
    assert nxt == int(np.argmax(lg32)) == int(np.argmax(lg64))
    # the token-by-token GPU path gives the same logits to well inside the bar
    assert m.hip.ResetKV() == 0
    lg_dec = np.empty(s.vocab, np.float32)
    for pos, tok in enumerate(prompt):
        rc, _ = m.hip.DecodeToken(int(tok), pos, lg_dec if pos == len(prompt) - 1 else None)
        assert rc == 0, E.last_error()
    assert H.rel_err(logits, lg_dec) < 1e-4
    # decode continues from the prefilled caches exactly as from decoded ones
    toks_ref, _ = H.oracle_generate(m, prompt, nDecode)
    assert m.hip.ResetKV() == 0
    rc, toks_dec = m.hip.Generate(prompt, nDecode, useGraph=True)
    assert rc == 0, E.last_error()
    assert m.hip.ResetKV() == 0
    rc, toks_pf = m.hip.GeneratePrefill(prompt, nDecode)
    assert rc == 0, E.last_error()
    assert toks_pf.tolist() == toks_dec.tolist() == toks_ref.tolist()
    return m, prompt, logits


def test_prefill_toy_matches_decode(hip):
    m, prompt, logits = _prefill_case(hip, configs.TOY, seed=1, nPrompt=37, nDecode=24, maxSeq=72)
    # chunked: 20 positions, then the remaining 17 starting at pos0 = 20
    assert m.hip.ResetKV() == 0
    rc, _, _, _ = m.hip.Prefill(prompt[:20], 0)
    assert rc == 0, E.last_error()
    rc, nxt2, logits2, _ = m.hip.Prefill(prompt[20:], 20, wantLogits=True)
    assert rc == 0, E.last_error()
    assert H.rel_err(logits2, logits) < 1e-5
    # a single-token prefill is a decode step
    assert m.hip.ResetKV() == 0
    rc, n1, l1, _ = m.hip.Prefill(prompt[:1], 0, wantLogits=True)
    assert rc == 0, E.last_error()
    assert m.hip.ResetKV() == 0
    l2 = np.empty(m.s.vocab, np.float32)
    rc, n2 = m.hip.DecodeToken(int(prompt[0]), 0, l2)
    assert rc == 0 and n1 == n2 and H.rel_err(l1, l2) < 1e-5
    m.close()


def test_prefill_qwen_shape_with_bias(hip):
    """Qwen2.5-0.5B shape (GQA 14/2, head 64, QKV bias), 3 layers, 200-token prompt (two row tiles)."""
    s = H.with_layers(configs.QWEN, 3)
    m, _, _ = _prefill_case(hip, s, seed=3, nPrompt=200, nDecode=8, maxSeq=256)
    m.close()


def test_prefill_llama3_shape_one_layer(hip):
    """Llama-3-8B shape (head 128, GQA 32/8), 1 layer, 160-token prompt."""
    s = H.with_layers(configs.LLAMA3_8B, 1)
    m, _, _ = _prefill_case(hip, s, seed=4, nPrompt=160, nDecode=4, maxSeq=192)
    m.close()


def test_prefill_llama3_shape_two_row_tiles(hip):
    """Llama-3-8B layer shape with a 300-token prompt (vocab cut to 8192 so the oracle stays fast): two
    256-row tiles, which is where the gate|up GEMM has enough tiles to run unsplit and forms
    silu(gate)*up in its own epilogue, while q|k|v, Wo and down split K and finish in the
    row-wise kernels (RoPE + cache rows; residual + next norm + split)."""
    s = H.with_layers(configs.LLAMA3_8B, 1)._replace(vocab=8192)
    m, _, _ = _prefill_case(hip, s, seed=14, nPrompt=300, nDecode=2, maxSeq=320)
    m.close()


def test_prefill_wide_ffn_with_a_partial_column_tile(hip):
    """An FFN of 80.5 tiles of 128 columns at 300 rows: the gate|up GEMM runs unsplit on the 256 x 256 tiles and forms
    silu(gate)*up itself.  Whole tiles leave through LDS as 128-byte rows (row blocks past the planes' 384 rows are
    skipped), the last tile has 64 columns and stores element by element; the down projection then reads both."""
    s = configs.Shape("ffn-edge", 1, 256, 4, 2, 64, 10304, 512, 1e-5, 1e4, False, True, "q8")
    m, _, _ = _prefill_case(hip, s, seed=21, nPrompt=300, nDecode=2, maxSeq=320)
    m.close()


def test_prefill_fp16_kv(hip):
    """Prefill writing fp16 KV rows (head sizes 64 and 128) against the oracle with the same rounding."""
    m, _, _ = _prefill_case(hip, H.with_layers(configs.QWEN, 2), seed=7, nPrompt=70, nDecode=6, maxSeq=96, kv_f16=True)
    m.close()
    s = configs.Shape("l3-mini", 2, 512, 4, 1, 128, 1024, 512, 1e-5, 5e5, False, True, "q8")
    m, _, _ = _prefill_case(hip, s, seed=8, nPrompt=45, nDecode=6, maxSeq=64, kv_f16=True)
    m.close()


def test_prefill_buffer_growth_and_sequence_end(hip):
    """Row buffers grow with the prompt (small call first), and a prompt may run to the last position."""
    s = H.with_layers(configs.TOY, 2)
    maxSeq = 200
    m = H.Model(s, seed=12, maxSeq=maxSeq, eng=hip, threads=8)
    prompt = m.prompt(maxSeq)
    rc, n_small, _, _ = m.hip.Prefill(prompt[:5], 0)                  # allocates for 128 rows
    assert rc == 0, E.last_error()
    assert m.hip.ResetKV() == 0
    rc, nxt, logits, _ = m.hip.Prefill(prompt, 0, wantLogits=True)    # 200 rows: buffers are re-made; ends at maxSeq - 1
    assert rc == 0, E.last_error()
    lg64 = _oracle_prompt_logits(m, prompt, True)
    assert H.rel_err(logits, lg64) < 1e-3 and nxt == int(np.argmax(lg64))
    # the position after the last one does not exist
    assert m.hip.Prefill(prompt[:1], maxSeq)[0] == -2
    # prompt + decode may fill the sequence exactly: maxSeq - 3 prompt positions, 4 tokens (the last needs no cache row)
    assert m.hip.ResetKV() == 0
    rc, toks = m.hip.GeneratePrefill(prompt[:maxSeq - 3], 4)
    assert rc == 0, E.last_error()
    assert m.hip.ResetKV() == 0
    rc, toks_dec = m.hip.Generate(prompt[:maxSeq - 3], 4, useGraph=True)
    assert rc == 0 and toks.tolist() == toks_dec.tolist()
    assert m.hip.GeneratePrefill(prompt[:maxSeq - 3], 5)[0] == -2
    m.close()


def test_prefill_errors(hip):
    s = H.with_layers(configs.TOY, 1)
    m = H.Model(s, seed=2, maxSeq=32, eng=hip, oracle=False)
    assert m.hip.Prefill(np.zeros(33, np.int32), 0)[0] == -2          # longer than maxSeq
    assert m.hip.Prefill(np.zeros(4, np.int32), 30)[0] == -2          # runs past maxSeq
    assert m.hip.Prefill(np.array([s.vocab], np.int32), 0)[0] == -2   # token out of range
    assert m.hip.Prefill(np.zeros(4, np.int32), 0)[0] == 0
    m.close()


def test_prefill_qwen_q4_0_shape(hip):
    """Qwen shape with GGUF Q4_0 weights and an fp16 embedding table, 2 layers, 150-token prompt (large-tile path)."""
    s = H.with_layers(configs.QWEN_Q4, 2)
    m, _, _ = _prefill_case(hip, s, seed=5, nPrompt=150, nDecode=6, maxSeq=192)
    m.close()


def test_prefill_q4_0_short_prompt_and_k_tail(hip):
    """Toy shape in Q4_0 (ffn 1376: a K of 43 blocks, odd, so the last K step is half empty), 40-token prompt (small tiles)."""
    s = configs.TOY._replace(fmt="q4_0", name="toy-q4")
    m, _, _ = _prefill_case(hip, s, seed=6, nPrompt=40, nDecode=6, maxSeq=64)
    m.close()

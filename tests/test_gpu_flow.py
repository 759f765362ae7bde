"""The persistent layer launch (exec mode 3): all layers of a decode step in one launch whose workgroups hand
their vectors over through an exchange area in device memory.

* every vector a phase hands over (q, K row, V row, attention partials, hidden after the attention block, SwiGLU
  vector, layer output), read back from the exchange area, against a float64 numpy evaluation of the layer
  (cuda_fused_infer.go:414-444 order, kernels/mongoose.cu:145-174, 856-933, 949-956, 991-1006 arithmetic);
* tokens through the launch == the oracle's, through graph replay and eager launches, and == the fused launches';
* contexts that need several KV splits per head, up to every partial slot in use;
* heads of 128 with grouped KV heads;
* Q4_0 matrices (split layout, half-block chunks) through the same launch: every handed-over vector, tokens against
  the oracle, rows of one and of two chunks a lane, the ring variant, biases;
* the widest FFN the launch takes, an FFN whose staged pieces come out uneven, row lengths between the tuned shapes;
* whole tokens inside the launch (embedding gather, layers, final norm, lm_head, argmax) and runs of tokens in one launch:
  tokens against the oracle for every number of tokens a launch, bit-identical logits between one token a launch and
  many, across a KV-split boundary inside a run (the K/V rows a run writes are read by its later tokens on other XCDs);
* fp16 K/V rows through the launch;
* a new context uses the launch; the trace diagnostic, the tail's included;
* a wait that runs out: the launch still ends, the call reports it, the context continues with the fused launches.
"""
import numpy as np
import pytest

from mongoose_amd import configs
from mongoose_amd import engine as E
from oracle import binding as ob
from tests import helpers as H

pytestmark = pytest.mark.gpu

MG_E_STATE = -4


def _in_use(hipctx):
    return hipctx.FlowInUse()


@pytest.mark.parametrize("fmt", ["q8", "q4_0"])
def test_every_handed_over_vector_matches_numpy(hip, fmt):
    s = H.with_layers(configs.TOY, 1)
    m = H.Model(s, seed=1, maxSeq=72, eng=hip, threads=8, keep_dequant=True, fmt=fmt)
    assert m.hip.SetExecMode(3) == 0
    D = {k: v.astype(np.float64) for k, v in m.dequant.items()}
    hd, half = s.headDim, s.headDim // 2
    cosT, sinT = ob.rope_tables(72, hd, s.theta)

    def rms(x, g):
        x = x.astype(np.float64)
        return x / np.sqrt((x * x).mean() + s.eps) * g

    def rope(x, pos, nH):
        x = x.reshape(nH, hd).copy()
        c, sn = cosT[pos].astype(np.float64), sinT[pos].astype(np.float64)
        a, b = x[:, :half].copy(), x[:, half:].copy()
        x[:, :half] = a * c - b * sn
        x[:, half:] = a * sn + b * c
        return x.reshape(-1)

    rng = np.random.default_rng(0)
    Ks, Vs = [], []
    G = s.nHeads // s.nKVHeads
    for pos in range(5):
        h = rng.standard_normal(s.dim).astype(np.float32)
        assert m.hip.PartialStep(h, pos, 0, 1, None, None) == 0, E.last_error()
        x = m.hip.FlowExchange(0)
        assert x is not None, "the persistent launch is not in use"
        n = rms(h, m.vecs[0])
        q = rope(D[1] @ n, pos, s.nHeads)
        k = rope(D[2] @ n, pos, s.nKVHeads)
        v = D[3] @ n
        Ks.append(k)
        Vs.append(v)
        assert H.rel_err(x["q"], q) < 1e-5 and H.rel_err(x["k"], k) < 1e-5 and H.rel_err(x["v"], v) < 1e-5
        K = np.array(Ks).reshape(pos + 1, s.nKVHeads, hd)
        V = np.array(Vs).reshape(pos + 1, s.nKVHeads, hd)
        att = np.zeros(s.dim)
        for hh in range(s.nHeads):
            sc = (K[:, hh // G] @ q[hh * hd:(hh + 1) * hd]) / np.sqrt(hd)
            p = np.exp(sc - sc.max())
            att[hh * hd:(hh + 1) * hd] = (p / p.sum()) @ V[:, hh // G]
        got = x["pacc"][0] / np.repeat(x["pl"][0], hd)           # one KV split at these positions
        assert H.rel_err(got, att) < 1e-5
        x1 = h.astype(np.float64) + D[7] @ att
        assert H.rel_err(x["x1"], x1) < 1e-5
        n2 = rms(x1, m.vecs[8])
        g, u = D[9] @ n2, D[10] @ n2
        mm = g / (1 + np.exp(-g)) * u
        assert H.rel_err(x["m"], mm) < 1e-5
        x2 = x1 + D[11] @ mm
        assert H.rel_err(x["x2"], x2) < 1e-5
        assert H.rel_err(m.hip.ExportHidden(), x2) < 1e-5
    m.close()


@pytest.mark.parametrize("fmt", ["q8", "q4_0"])
def test_tokens_match_oracle_and_fused_launches(hip, fmt):
    s = configs.TOY
    m = H.Model(s, seed=3, maxSeq=72, eng=hip, threads=8, fmt=fmt)
    prompt = m.prompt(8)
    ref, _ = H.oracle_generate(m, prompt, 64)
    assert _in_use(m.hip), "a new context should use the persistent launch"
    out = {}
    for mode in (1, 3):
        assert m.hip.SetExecMode(mode) == 0
        for graph in (True, False):
            assert m.hip.ResetKV() == 0
            rc, t = m.hip.Generate(prompt, 64, useGraph=graph)
            assert rc == 0, E.last_error()
            out[(mode, graph)] = t.tolist()
        assert _in_use(m.hip) == (mode == 3)
    assert out[(3, True)] == ref.tolist(), H.first_divergence(out[(3, True)], ref)
    assert out[(3, False)] == ref.tolist()
    assert out[(1, True)] == ref.tolist() and out[(1, False)] == ref.tolist()
    # logits and hidden of a step through the launch against the oracle's
    assert m.hip.SetExecMode(3) == 0
    assert m.hip.ResetKV() == 0
    m.orc.reset_kv()
    stream = list(prompt) + list(ref)
    logits = np.empty(s.vocab, np.float32)
    for pos in range(12):
        h = m.orc.embed(stream[pos])
        hid, lg, _ = m.orc.step(h, pos, shadow=True)
        assert m.hip.PartialStep(h, pos, 0, s.nLayers, None, logits) == 0, E.last_error()
        assert H.rel_err(logits, lg) < 1e-4
        assert H.rel_err(m.hip.ExportHidden(), hid) < 1e-4
    m.close()


def _modes_agree(m, prompt, nDecode, what):
    """The same prompt and decode run through the fused launches (exec mode 1) and the persistent launch (3):
    identical greedy tokens, and -- tokens alone need not show a dropped or mis-weighted KV split -- the logits
    and the hidden state of one more step at the position after the run agree to rounding (the two differ in
    the order in which the splits' partials are merged, nothing else)."""
    out, last = {}, {}
    s = m.s
    for mode in (1, 3):
        assert m.hip.SetExecMode(mode) == 0
        assert m.hip.ResetKV() == 0
        rc, t = m.hip.GeneratePrefill(prompt, nDecode)
        assert rc == 0, E.last_error()
        assert _in_use(m.hip) == (mode == 3)
        out[mode] = t
        pos = len(prompt) + nDecode - 1                     # the cache holds positions 0 .. pos - 1
        if pos < m.maxSeq:
            logits = np.empty(s.vocab, np.float32)
            rc, _ = m.hip.DecodeToken(int(t[-1]), pos, logits)
            assert rc == 0, E.last_error()
            last[mode] = (logits, m.hip.ExportHidden())
    i = H.first_divergence(out[3], out[1])
    assert i is None, f"{what}: persistent launch and fused launches part at token {i}"
    if last:
        el, eh = H.rel_err(last[3][0], last[1][0]), H.rel_err(last[3][1], last[1][1])
        print(f"  {what}: modes 3 vs 1 at the next position: logits {el:.2e}, hidden {eh:.2e}", flush=True)
        assert el < 1e-5 and eh < 1e-5, f"{what}: logits {el:.2e} / hidden {eh:.2e} between the two launches"
    return out[3]


def test_kv_splits_heads_of_64(hip):
    """0.5B geometry (14 query heads on 2 KV heads, biases), 2 layers.  18 partial slots per head (256 CUs / 14 heads),
    i.e. contexts of up to 2304 positions: positions 600..640 use 5-6 splits of 128 positions, 2260..2300 all 18."""
    s = H.with_layers(configs.QWEN, 2)._replace(name="qwen-geom", vocab=2048)
    m = H.Model(s, seed=11, maxSeq=2304, eng=hip, oracle=False)
    print("flow: qwen geometry, positions 600..640", flush=True)
    _modes_agree(m, m.prompt(600), 40, "5-6 splits")
    print("flow: qwen geometry, positions 2260..2300 (18 splits)", flush=True)
    _modes_agree(m, m.prompt(2260), 40, "18 splits")
    m.close()
    # a longer context: one attention workgroup per (KV head, split) that takes the 7 query heads of its KV head in turn
    m = H.Model(s, seed=11, maxSeq=6000, eng=hip, oracle=False)
    print("flow: qwen geometry, grouped attention, positions 100..130, 2990..3020 and 5950..5990", flush=True)
    _modes_agree(m, m.prompt(100), 30, "grouped, 1 split")
    _modes_agree(m, m.prompt(2990), 30, "grouped, 24 splits")
    _modes_agree(m, m.prompt(5950), 40, "grouped, 47 splits")
    # The launch is handed the attention variant its positions need: the plain one (a workgroup per query head and split)
    # while 14 heads x splits fit the 256 workgroups, i.e. up to position 2303, the grouped one from there on.  Launches of
    # 8 tokens from position 2290: the first is plain, the second crosses the boundary inside the launch, the rest are
    # grouped; the same run as launches of 64 tokens is grouped throughout.
    for n in (8, 64):
        assert m.hip.SetTokensPerLaunch(n) == 0
        _modes_agree(m, m.prompt(2290), 40, f"plain to grouped at position 2304, {n} tokens a launch")
    m.close()
    # 2 KV heads x 128 positions x 128 workgroup rows = 16384 positions at most
    m = H.Model(s, seed=11, maxSeq=16385, eng=hip, oracle=False)
    assert m.hip.SetExecMode(3) == 0
    assert not _in_use(m.hip)
    m.close()


def test_q4_0_qwen_geometry_and_ring(hip):
    """Q4_0 matrices through the persistent launch at the 0.5B geometry (biases, 14 query heads on 2 KV heads, rows of
    896 = 56 half-block chunks, fp16 embedding table) and at rows of 4096 weights, which stream through the register
    ring: tokens against the oracle, then against the fused launches over positions that need several KV splits."""
    s = H.with_layers(configs.QWEN_Q4, 2)._replace(name="qwen-q4-geom", vocab=2048)
    m = H.Model(s, seed=21, maxSeq=400, eng=hip, threads=8)
    print("flow: qwen geometry, Q4_0, 6 + 10 against the oracle", flush=True)
    prompt = m.prompt(6)
    ref, _ = H.oracle_generate(m, prompt, 10)
    rc, t = m.hip.Generate(prompt, 10, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip), "Q4_0 layers should run in the persistent launch"
    assert t.tolist() == ref.tolist(), H.first_divergence(t, ref)
    print("flow: qwen geometry, Q4_0, positions 300..340 (3 splits)", flush=True)
    _modes_agree(m, m.prompt(300), 40, "Q4_0, 3 splits")
    m.close()
    s = H.with_layers(configs.LLAMA3_8B, 2)._replace(name="l3-q4-geom", ffnDim=4864, vocab=1024, tied=True)
    m = H.Model(s, seed=22, maxSeq=200, eng=hip, threads=16, fmt="q4_0")
    print("flow: rows of 4096 and 4864 weights (ring), Q4_0, 6 + 8 against the oracle", flush=True)
    prompt = m.prompt(6)
    ref, _ = H.oracle_generate(m, prompt, 8)
    rc, t = m.hip.Generate(prompt, 8, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip)
    assert t.tolist() == ref.tolist(), H.first_divergence(t, ref)
    _modes_agree(m, m.prompt(150), 30, "Q4_0 ring, 2 splits")
    m.close()
    # TinyLlama's row lengths (2048 = two chunks a lane, 5632 in the down projection), no ring
    s = H.with_layers(configs.TINYLLAMA, 2)._replace(name="tiny-q4-geom", vocab=1024, tied=True)
    m = H.Model(s, seed=23, maxSeq=64, eng=hip, threads=16, fmt="q4_0")
    print("flow: rows of 2048 and 5632 weights, Q4_0, 6 + 8 against the oracle", flush=True)
    prompt = m.prompt(6)
    ref, _ = H.oracle_generate(m, prompt, 8)
    rc, t = m.hip.Generate(prompt, 8, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip)
    assert t.tolist() == ref.tolist(), H.first_divergence(t, ref)
    m.close()


@pytest.mark.parametrize("fmt", ["q8", "q4_0"])
def test_prefetching_workgroups_change_nothing(hip, fmt):
    """Exec mode 3 sets 32 workgroups of the launch aside to read the coming weights into the L2s (0.5B geometry: a layer
    fits); mode 4 lets every workgroup compute.  A row is multiplied by one wave in the same order either way, so the
    logits are identical bit for bit, at one KV split and at several."""
    s = H.with_layers(configs.QWEN if fmt == "q8" else configs.QWEN_Q4, 3)._replace(vocab=2048)
    m = H.Model(s, seed=31, maxSeq=400, eng=hip, oracle=False)
    # (both modes on the same kernel variant: the one with this shape's sizes compiled in has the prefetching role
    # compiled in too, so mode 4 would take another variant, whose results differ by rounding)
    assert m.hip.SetFlowGeneric(True) == 0
    prompt = m.prompt(300)
    outs = {}
    for mode in (3, 4):
        assert m.hip.SetExecMode(mode) == 0
        assert m.hip.ResetKV() == 0
        assert _in_use(m.hip)
        logits = np.empty(s.vocab, np.float32)
        res = []
        for pos in range(300):
            last = pos in (0, 1, 127, 128, 298, 299)
            rc, nxt = m.hip.DecodeToken(int(prompt[pos]), pos, logits if last else None)
            assert rc == 0, E.last_error()
            if last:
                res.append((nxt, logits.copy()))
        outs[mode] = res
    for (n3, l3), (n4, l4) in zip(outs[3], outs[4]):
        assert n3 == n4 and np.array_equal(l3, l4)
    # and through graph replay after the switch back
    assert m.hip.SetExecMode(3) == 0
    assert m.hip.ResetKV() == 0
    rc, t3 = m.hip.Generate(prompt[:8], 24, useGraph=True)
    assert rc == 0, E.last_error()
    assert m.hip.SetExecMode(4) == 0
    assert m.hip.ResetKV() == 0
    rc, t4 = m.hip.Generate(prompt[:8], 24, useGraph=True)
    assert rc == 0, E.last_error()
    assert t3.tolist() == t4.tolist()
    m.close()


@pytest.mark.parametrize("name,positions,kv_f16", [("qwen2.5-0.5b", 300, False), ("qwen2.5-0.5b-q4_0", 300, False),
                                                   ("tinyllama-1.1b", 300, False), ("llama-3-8b", 1100, False),
                                                   ("llama-3-8b", 1100, True)])
def test_variants_with_a_shape_compiled_in_change_nothing(hip, name, positions, kv_f16):
    """A context of exactly the 0.5B, 1.1B or 8B shape takes a variant of the persistent launch with that shape's sizes as
    constants; mg_set_flow_generic keeps it on the variants whose sizes come with the launch.  Same formulas over the same
    rows; the compiler contracts and schedules the two differently, so logits agree to rounding (1e-5 of their largest, the
    bar between launches elsewhere in this file) and the greedy tokens are the same, token by token across the first KV
    split boundary and in runs of tokens inside one launch (8B shape: to past position 1024, where the launch changes to
    the grouped attention, with fp32 and with fp16 K/V rows)."""
    s = H.with_layers(configs.BY_NAME[name], 2)._replace(vocab=2048)
    m = H.Model(s, seed=41, maxSeq=positions + 40, eng=hip, oracle=False, kv_f16=kv_f16)
    prompt = m.prompt(8)
    outs = {}
    for generic in (0, 1):
        assert m.hip.SetFlowGeneric(generic) == 0
        assert m.hip.ResetKV() == 0
        assert _in_use(m.hip)
        rc, toks = m.hip.Generate(prompt, positions, useGraph=True)         # runs of 64 tokens a launch
        assert rc == 0, E.last_error()
        assert m.hip.FlowInUse()
        stream = list(prompt) + [int(t) for t in toks]
        assert m.hip.ResetKV() == 0
        logits = np.empty(s.vocab, np.float32)
        res = []
        for pos in range(140):                                              # a launch a token, logits read back
            last = pos in (0, 1, 127, 128, 139)
            rc, nxt = m.hip.DecodeToken(stream[pos], pos, logits if last else None)
            assert rc == 0, E.last_error()
            if last:
                res.append((nxt, logits.copy()))
        outs[generic] = (toks.tolist(), res)
    assert outs[0][0] == outs[1][0]
    for (n0, l0), (n1, l1) in zip(outs[0][1], outs[1][1]):
        assert n0 == n1 and H.rel_err(l0, l1) < 1e-5
    m.close()


def test_heads_of_128_grouped_kv(hip):
    """Llama-3-8B attention geometry (32 query heads of 128 on 8 KV heads, dim 4096: rows of two chunks a lane), 2
    layers, FFN and vocabulary cut: 8 partial slots, tile 128."""
    s = H.with_layers(configs.LLAMA3_8B, 2)._replace(name="l3-geom", ffnDim=1024, vocab=1024, tied=True)
    m = H.Model(s, seed=12, maxSeq=700, eng=hip, threads=16)
    print("flow: llama-3 geometry, 6 + 6 against the oracle", flush=True)
    prompt = m.prompt(6)
    ref, _ = H.oracle_generate(m, prompt, 6)
    assert m.hip.SetExecMode(3) == 0
    rc, t = m.hip.Generate(prompt, 6, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip)
    assert t.tolist() == ref.tolist()
    print("flow: llama-3 geometry, positions 300..330 (3 splits)", flush=True)
    _modes_agree(m, m.prompt(300), 30, "heads of 128")
    m.close()
    # past 8 x 128 positions: grouped attention (4 query heads a KV head), up to 32 splits
    m = H.Model(s, seed=12, maxSeq=4096, eng=hip, oracle=False)
    print("flow: llama-3 geometry, grouped attention, positions 4040..4090", flush=True)
    _modes_agree(m, m.prompt(4040), 50, "heads of 128, grouped")
    m.close()


def test_fp16_kv_rows_in_the_launch(hip):
    """fp16 K/V rows (SetKVFormat(1)) through the persistent launch: rounded where the q|k|v phase writes them (the
    cache and the copy it hands to the attention workgroups), widened where the attention phase reads them.  Tokens
    against the oracle with the same rounding (toy, and heads of 128 over several KV splits), then against the fused
    launches -- tokens, logits and hidden state -- at the 8B attention geometry with grouped attention at positions
    4040..4090."""
    m = H.Model(configs.TOY, seed=44, maxSeq=72, eng=hip, threads=8, kv_f16=True)
    prompt = m.prompt(8)
    ref, _ = H.oracle_generate(m, prompt, 40)
    rc, t = m.hip.Generate(prompt, 40, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip) and m.hip.FlowTailInUse(), "fp16 rows should not keep a context out of the launch"
    assert t.tolist() == ref.tolist(), H.first_divergence(t, ref)
    m.close()
    s = configs.Shape("l3-mini-f16", 2, 512, 4, 1, 128, 1024, 512, 1e-5, 5e5, False, True, "q8")
    m = H.Model(s, seed=45, maxSeq=600, eng=hip, threads=8, kv_f16=True)
    prompt = m.prompt(4)
    ref, _ = H.oracle_generate(m, prompt, 300)
    rc, t = m.hip.Generate(prompt, 300, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip)
    assert t.tolist() == ref.tolist(), H.first_divergence(t, ref)
    _modes_agree(m, m.prompt(500), 40, "fp16 rows, heads of 128, 4-5 splits")
    m.close()
    s = H.with_layers(configs.LLAMA3_8B, 2)._replace(name="l3-geom-f16", ffnDim=1024, vocab=1024, tied=True)
    m = H.Model(s, seed=46, maxSeq=4096, eng=hip, oracle=False, kv_f16=True)
    print("flow: llama-3 geometry, fp16 rows, grouped attention, positions 4040..4090", flush=True)
    _modes_agree(m, m.prompt(4040), 50, "fp16 rows, heads of 128, grouped")
    m.close()


@pytest.mark.parametrize("ffn", [15360, 9216])
def test_streamed_rows_wide_ffn(hip, ffn):
    """Rows of 4096 weights with the widest FFN the launch takes (15360: seven or eight staged pieces a thread for the
    down projection, seven or eight rounds of gate|up rows) and one whose pieces do not come out even (9216: four or five a thread):
    tokens against the oracle, then against the fused launches at two KV splits."""
    s = H.with_layers(configs.LLAMA3_8B, 2)._replace(name=f"l3-ffn{ffn}", ffnDim=ffn, vocab=1024, tied=True)
    m = H.Model(s, seed=31, maxSeq=200, eng=hip, threads=16)
    print(f"flow: rows of 4096, ffn {ffn}, 4 + 6 against the oracle", flush=True)
    prompt = m.prompt(4)
    ref, _ = H.oracle_generate(m, prompt, 6)
    rc, t = m.hip.Generate(prompt, 6, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip)
    assert t.tolist() == ref.tolist(), H.first_divergence(t, ref)
    _modes_agree(m, m.prompt(140), 20, f"ffn {ffn}, 2 splits")
    m.close()


@pytest.mark.parametrize("fmt", ["q8", "q4_0"])
@pytest.mark.parametrize("name,dim,heads,kv,hd,ffn", [
    ("rows-3072", 3072, 24, 8, 128, 8192),      # streamed rows whose second request a lane is half empty
    ("rows-1536", 1536, 24, 4, 64, 4096),       # two requests a lane, the second used by half the lanes
    ("rows-640", 640, 10, 2, 64, 1792),         # one request a lane, partly used
])
def test_row_lengths_between_the_tuned_ones(hip, fmt, name, dim, heads, kv, hd, ffn):
    """Row lengths that are not a whole number of 1024-weight requests: tokens against the oracle through the
    persistent launch, then against the fused launches at two KV splits."""
    s = configs.Shape(name, 2, dim, heads, kv, hd, ffn, 1024, 1e-5, 5e5, True, True, "q8")
    m = H.Model(s, seed=37, maxSeq=200, eng=hip, threads=16, fmt=fmt)
    print(f"flow: {name} {fmt}, 4 + 6 against the oracle", flush=True)
    prompt = m.prompt(4)
    ref, _ = H.oracle_generate(m, prompt, 6)
    rc, t = m.hip.Generate(prompt, 6, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip)
    H.assert_same_tokens_or_near_tie(m, prompt, t, ref, f"{name} {fmt}")
    _modes_agree(m, m.prompt(140), 20, f"{name} {fmt}, 2 splits")
    m.close()


@pytest.mark.parametrize("fmt", ["q8", "q4_0"])
def test_runs_of_tokens_in_one_launch(hip, fmt):
    """Whole tokens inside the persistent launch.  Toy model (8 + 64): the oracle's tokens whether a launch runs 1, 5 or 64
    tokens, through Generate and GeneratePrefill, and with the lm_head and argmax as launches of their own
    (SetFlowTail(0)).  0.5B geometry, 2 layers: a run of 80 tokens from position 90 crosses the boundary between the
    first and the second KV split at position 128 inside one launch -- every K/V row the run writes is read by the
    tokens after it -- and gives the tokens, and bit for bit the logits of the step after, of one token a launch."""
    s = configs.TOY
    m = H.Model(s, seed=41, maxSeq=80, eng=hip, threads=8, fmt=fmt)
    prompt = m.prompt(8)
    ref, _ = H.oracle_generate(m, prompt, 64)
    assert m.hip.FlowTailInUse(), "whole tokens should run inside the launch"
    for n in (1, 5, 64):
        assert m.hip.SetTokensPerLaunch(n) == 0
        assert m.hip.ResetKV() == 0
        rc, t = m.hip.Generate(prompt, 64, useGraph=True)
        assert rc == 0, E.last_error()
        assert t.tolist() == ref.tolist(), (n, H.first_divergence(t, ref))
    assert m.hip.ResetKV() == 0
    rc, t = m.hip.GeneratePrefill(prompt, 64)
    assert rc == 0, E.last_error()
    H.assert_same_tokens_or_near_tie(m, prompt, t, ref, f"prefill then a run of tokens, {fmt}")
    assert m.hip.SetFlowTail(False) == 0
    assert m.hip.FlowInUse() and not m.hip.FlowTailInUse()
    assert m.hip.ResetKV() == 0
    rc, t = m.hip.Generate(prompt, 64, useGraph=True)
    assert rc == 0, E.last_error()
    assert t.tolist() == ref.tolist()
    m.close()

    s = H.with_layers(configs.QWEN if fmt == "q8" else configs.QWEN_Q4, 2)._replace(name="qwen-geom-runs", vocab=2048)
    m = H.Model(s, seed=42, maxSeq=200, eng=hip, oracle=False, fmt=fmt)
    prompt = m.prompt(90)
    res = {}
    logits = np.empty(s.vocab, np.float32)
    for n in (1, 64):
        assert m.hip.SetTokensPerLaunch(n) == 0
        assert m.hip.ResetKV() == 0
        rc, t = m.hip.GeneratePrefill(prompt, 80)
        assert rc == 0, E.last_error()
        assert m.hip.FlowTailInUse()
        rc, _ = m.hip.DecodeToken(int(t[-1]), 169, logits)
        assert rc == 0, E.last_error()
        res[n] = (t.tolist(), logits.copy())
    assert res[1][0] == res[64][0], H.first_divergence(res[1][0], res[64][0])
    assert np.array_equal(res[1][1], res[64][1])
    m.close()


def test_new_context_uses_the_launch_and_trace(hip):
    s = H.with_layers(configs.TOY, 8)
    m = H.Model(s, seed=5, maxSeq=40, eng=hip, threads=8)
    prompt = m.prompt(4)
    ref, _ = H.oracle_generate(m, prompt, 16)
    rc, t = m.hip.Generate(prompt, 16, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip)
    assert t.tolist() == ref.tolist()
    rc, tr = m.hip.FlowTrace(True, read=False)
    assert rc == 0, E.last_error()
    rc, t2 = m.hip.Generate(prompt, 2, useGraph=False)
    assert rc == 0
    rc, tr = m.hip.FlowTrace(True, read=True)
    assert rc == 0 and tr.shape[0] == 8 and tr.shape[1] == len(m.hip.FLOW_TRACE_POINTS)
    # every workgroup passed the top of every layer, later in every later layer
    tops = tr[:, 0, :]
    assert (tops > 0).all() and (np.diff(tops.astype(np.int64), axis=0) > 0).all()
    # the tail of the token: after the last layer, in program order
    rc, tt = m.hip.FlowTailTrace()
    assert rc == 0 and tt.shape[0] == len(m.hip.FLOW_TAIL_TRACE_POINTS)
    assert (tt[0] >= tr[-1, -1, :]).all()
    top, staged, wave0, known, done, parts = [tt[i].astype(np.int64) for i in range(6)]
    assert (staged >= top).all() and (wave0 >= staged).all() and (done >= wave0).all() and (parts >= done).all() and (known >= parts).all()
    assert m.hip.FlowTrace(False)[0] == 0
    # a context in another mode has no such launch to trace
    assert m.hip.SetExecMode(1) == 0
    assert m.hip.FlowTrace(True)[0] == MG_E_STATE
    m.close()


def test_one_context_a_device_owns_the_launch(hip):
    s = configs.TOY
    a = H.Model(s, seed=8, maxSeq=24, eng=hip, oracle=False)
    b = H.Model(s, seed=8, maxSeq=24, eng=hip, oracle=False)
    prompt = a.prompt(4)
    assert _in_use(a.hip) and not _in_use(b.hip)
    rc, ta = a.hip.Generate(prompt, 8)
    assert rc == 0, E.last_error()
    rc, tb = b.hip.Generate(prompt, 8)                 # the fused launches
    assert rc == 0, E.last_error()
    assert ta.tolist() == tb.tolist()
    assert a.hip.SetExecMode(1) == 0                   # gives the launch up
    assert _in_use(b.hip) and not _in_use(a.hip)
    assert b.hip.ResetKV() == 0
    rc, tb2 = b.hip.Generate(prompt, 8)
    assert rc == 0 and tb2.tolist() == ta.tolist()
    b.close()
    assert a.hip.SetExecMode(3) == 0
    assert _in_use(a.hip)
    a.close()


def test_a_wait_that_runs_out_is_reported_and_the_context_goes_on(hip):
    s = configs.TOY
    m = H.Model(s, seed=7, maxSeq=40, eng=hip, threads=8)
    prompt = m.prompt(4)
    ref, _ = H.oracle_generate(m, prompt, 12)
    assert m.hip.SetExecMode(3) == 0
    assert m.hip.SetFlowWaitLimit(-1) == 0          # every wait not satisfied at once gives up; all workgroups still exit
    rc, _ = m.hip.Generate(prompt, 12, useGraph=False)
    assert rc != 0 and "persistent" in E.last_error(), (rc, E.last_error())
    assert not _in_use(m.hip)
    assert m.hip.SetFlowWaitLimit(5_000_000) == 0
    assert m.hip.ResetKV() == 0
    rc, t = m.hip.Generate(prompt, 12, useGraph=True)
    assert rc == 0, E.last_error()
    assert t.tolist() == ref.tolist()
    # asking for the mode by name arms the launch again; the same with a run of tokens in one launch: every workgroup
    # gives up its waits, runs through all the run's tokens and exits, and the call reports it
    assert m.hip.SetExecMode(3) == 0
    assert _in_use(m.hip) and m.hip.FlowTailInUse()
    assert m.hip.SetFlowWaitLimit(-1) == 0
    assert m.hip.ResetKV() == 0
    rc, _ = m.hip.Generate(prompt, 12, useGraph=True)
    assert rc != 0 and "persistent" in E.last_error(), (rc, E.last_error())
    assert not _in_use(m.hip)
    assert m.hip.SetFlowWaitLimit(5_000_000) == 0
    assert m.hip.SetExecMode(3) == 0
    assert m.hip.ResetKV() == 0
    rc, t = m.hip.Generate(prompt, 12, useGraph=True)
    assert rc == 0, E.last_error()
    assert _in_use(m.hip) and t.tolist() == ref.tolist()
    m.close()

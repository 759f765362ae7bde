#!/usr/bin/env python3
"""Benchmark of the fused quantized decode path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME]

A "step" is one batch-1 greedy decode token through the whole path (embedding
gather -> layers -> final norm -> lm_head -> argmax) with the position and the token
resident on the device: by default inside the persistent launch, which runs up to 64
such steps per launch and chooses every next token on the device (the same steps as
replays of a captured one-launch hipGraph are timed beside it).  The W warmup
steps are the W prompt positions; the K timed steps are the K decode positions
after them.  Weights are synthetic (seeded N(0, 0.02), quantized on the host by
the library's own loader) and resident in HBM before the timed region starts.

Prints ONE JSON line: the throughput of the headline configuration, the roofline of
the kernel that takes most of the step's time (HIP events around its launches inside
the step), a per-launch table, the lm_head matvec's own bandwidth (the second half of
the metric), the CPU oracle timed on this box's host cores as a baseline, and -- under
"configs" -- the same measurements for the other benchmark configurations (toy,
TinyLlama-1.1B shape, Qwen2.5-0.5B Q4_0 with a leg through the weight-streaming front end,
Llama-3-8B shape at a short context, at ~4k context with fp32 and with fp16 K/V rows, and
its 512-token batched prefill), each with its greedy tokens checked against the oracle
on a bounded sample (the ~4k-context runs against the fused launches on the same positions).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published peak

# HBM bytes per launch from rocprofv3 --pmc runs of this script (FETCH_SIZE then WRITE_SIZE,
# KiB per dispatch), each scaled by what the same counter reads for a 256 MiB device copy in
# the same run (FETCH_SIZE reads 131090-131102 KiB for the 262144 KiB copied -> x1.9995-1.9997;
# WRITE_SIZE reads 262144.0 -> x1.0).  Counts are a property of kernel and shape, so they are recorded
# here, keyed by (configuration, launch); profiles/ holds the runs they come from.  The default run
# measures the headline launch's traffic itself (live_pmc_traffic: the same two passes as children of this
# process) and reports the recorded figure beside it; where it cannot (a flag that leaves the default path,
# no rocprofv3, a pass that fails) and for the other configurations the recorded figures are reported, and
# "traffic_source" / "traffic_note" in the output say which it was.
PMC_TRAFFIC_BYTES = {
    # the launch that runs whole tokens: bytes a TOKEN (all timed launches' counters over their tokens)
    ("qwen2.5-0.5b", "token"): int(((16442513.9 + 16834705.5 + 17266254.7 + 2186297.5) * (262144.0 / 131090.0)
                                    + (168980.9 + 170548.5 + 175650.0 + 22851.3)) * 1024 / 200),
    ("tinyllama-1.1b", "token"): int((26410817.8 * (262144.0 / 131090.0) + 144870.5) * 1024 / 50),
    ("llama-3-8b", "token"): int((239270332.8 * (262144.0 / 131090.0) + 622790.0) * 1024 / 64),
    # separate launches (--no-flow-tail, --exec-mode 1): bytes a launch
    ("qwen2.5-0.5b", "lm_head"): int((67135.1 * (262144.0 / 131102.4) + 660.5 * 1.0) * 1024),
    ("qwen2.5-0.5b", "flow"): int((190867.0 * (262144.0 / 131102.4) + 952.0 * 1.0) * 1024),
    ("llama-3-8b", "lm_head"): int((257245.0 * (262144.0 / 131102.4) + 715.6 * 1.0) * 1024),
    ("llama-3-8b", "flow"): int((3510548.2 * (262144.0 / 131102.4) + 4432.0 * 1.0) * 1024),
}
PMC_SOURCE = "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script recorded in profiles/ (constants in bench.py, not measured by this run)"



def live_pmc_traffic(config, steps, warmup, timeout_s=100):
    """HBM bytes of the token launches of THIS build on THIS box: two rocprofv3 --pmc passes (FETCH_SIZE, then WRITE_SIZE --
    together they need more counters of one block than a pass holds) over `bench.py --lean --pmc-copy`, run as child
    processes before this process touches the GPU.  Returns (dict, None) or (None, reason)."""
    import csv
    import shutil
    import signal
    import subprocess
    import tempfile
    exe = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(exe):
        return None, "rocprofv3 not found"
    tmp = tempfile.mkdtemp(prefix="mg_pmc_", dir="/tmp")
    env = dict(os.environ, TMPDIR="/tmp")
    got = {}
    try:
        for ctr in ("FETCH_SIZE", "WRITE_SIZE"):
            cmd = [exe, "--pmc", ctr, "--output-format", "csv", "-d", tmp, "-o", ctr.lower(), "--",
                   sys.executable, os.path.join(ROOT, "bench.py"), "--lean", "--pmc-copy", "--config", config,
                   "--steps", str(steps), "--warmup", str(warmup)]
            print(f"bench.py: rocprofv3 --pmc {ctr} pass", file=sys.stderr, flush=True)
            proc = subprocess.Popen(cmd, cwd=ROOT, env=env, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE,
                                    start_new_session=True, text=True)
            try:
                _, err = proc.communicate(timeout=timeout_s)
            except subprocess.TimeoutExpired:
                os.killpg(proc.pid, signal.SIGKILL)
                proc.communicate()
                return None, f"rocprofv3 --pmc {ctr} pass did not end within {timeout_s} s"
            if proc.returncode != 0:
                return None, f"rocprofv3 --pmc {ctr} pass ended with status {proc.returncode}: {(err or '').strip()[-200:]}"
            path = None
            for dp, _, files in os.walk(tmp):
                for fn in files:
                    if fn == f"{ctr.lower()}_counter_collection.csv":
                        path = os.path.join(dp, fn)
            if path is None:
                return None, f"no counter file from the {ctr} pass"
            launch, copies = [], []
            for r in csv.DictReader(open(path)):
                if r.get("Counter_Name") != ctr:
                    continue
                v = float(r["Counter_Value"])
                if "flow_layers_kernel" in r["Kernel_Name"]:
                    launch.append(v)
                elif "copyBuffer" in r["Kernel_Name"] and v > 65536:
                    copies.append(v)
            if not launch or not copies:
                return None, f"{ctr} pass: no dispatch of the launch or of the 256 MiB copies in the counter file"
            got[ctr] = (launch, 262144.0 / (sum(copies) / len(copies)))
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return got, None


LAUNCH_NAMES = {0: "embed_gather", 1: "norm+qkv", 2: "rope+kvwrite+attention", 3: "wo+residual", 4: "norm+gate_up+swiglu",
                5: "down+residual", 6: "norm+lm_head+argmax_partials", 7: "argmax_finish"}
FLOW_NAME = "persistent layer launch (all layers: norm, q|k|v, RoPE, KV write, attention, Wo, gate|up, SwiGLU, down)"
TOKEN_NAME = "persistent launch, whole tokens (embedding gather, all layers, final norm, lm_head, argmax)"


def slot_shape(s, kv, idx):
    nL = s.nLayers
    if idx < nL * 12:
        return {0: (s.dim, 1), 1: (s.dim, s.dim), 2: (kv, s.dim), 3: (kv, s.dim), 4: (s.dim, 1), 5: (kv, 1),
                6: (kv, 1), 7: (s.dim, s.dim), 8: (s.dim, 1), 9: (s.ffnDim, s.dim), 10: (s.ffnDim, s.dim),
                11: (s.dim, s.ffnDim)}[idx % 12]
    return (s.dim, 1) if idx == nL * 12 else (s.vocab, s.dim)


def gen_slot(E, np, s, kv, seed, idx):
    rows, cols = slot_shape(s, kv, idx)
    a = E.synth_normal(seed, idx, 0.02, (rows, cols) if cols > 1 else (rows,))
    w = idx % 12 if idx < s.nLayers * 12 else -1
    if cols == 1 and (w in (0, 8) or idx == s.nLayers * 12):
        a = (a + np.float32(1.0)).astype(np.float32)
    return a


def slots(s):
    for idx in range(s.nLayers * 12 + 2):
        w = idx % 12 if idx < s.nLayers * 12 else -1
        if w in (4, 5, 6) and not s.bias:
            continue
        yield idx


def load_model(E, np, s, seed, maxSeq, eng, oracle=None, oracle_layers=None, kv_f16=False):
    """Build the GPU context through the library's own loader (SetWeight quantizes on the host);
    optionally mirror the same quantized bytes into the CPU oracle."""
    from mongoose_amd import configs
    kv = configs.kv_dim(s)
    f = E.NewHIPFusedInference(eng, s.dim, kv, s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab, s.nLayers,
                               maxSeq, s.theta, s.eps)
    if f is None:
        raise RuntimeError("NewHIPFusedInference failed: " + E.last_error())
    if kv_f16 and f.SetKVFormat(1) != 0:
        raise RuntimeError(E.last_error())
    if f.SetLayerRange(0, s.nLayers) != 0:
        raise RuntimeError(E.last_error())
    for idx in slots(s):
        rows, cols = slot_shape(s, kv, idx)
        data = gen_slot(E, np, s, kv, seed, idx)
        if cols == 1:
            rc = f.SetWeight(idx, data)
            if oracle is not None:
                oracle.set_f32(idx, data)
        elif s.fmt == "q8":
            q, sc = E.quantize_q8(data, 0)
            rc = f.SetWeightQ8(idx, q, sc)
            if oracle is not None:
                oracle.set_q8(idx, q, sc)
        else:
            blk = E.quantize_q4_0(data)
            rc = f.SetWeightQ4_0(idx, blk)
            if oracle is not None:
                oracle.set_q4_0(idx, blk)
        if rc != 0:
            raise RuntimeError(f"slot {idx}: " + E.last_error())
    if not s.tied:
        emb = E.synth_normal(seed, 10_000_019, 0.02, (s.vocab, s.dim)).astype(np.float16)
        if f.SetEmbeddingF16(emb) != 0:
            raise RuntimeError(E.last_error())
        if oracle is not None:
            oracle.set_embed_f16(emb)
    return f


def cpu_baseline(E, np, s, seed, prompt, first_tokens, budget_s, kv_f16=False):
    """The CPU oracle (restatement of the Go CPU engine's arithmetic, single
    thread like cpu.go) on the same model and the same positions, for a bounded
    number of tokens."""
    from mongoose_amd import configs
    from oracle import binding as ob
    kv = configs.kv_dim(s)
    nP = len(prompt)
    sample = 4
    orc = ob.Oracle(s.dim, kv, s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab, s.nLayers, nP + 64,
                    s.theta, s.eps, threads=1)
    if kv_f16:
        orc.set_kv_f16(True)
    for idx in slots(s):
        rows, cols = slot_shape(s, kv, idx)
        data = gen_slot(E, np, s, kv, seed, idx)
        if cols == 1:
            orc.set_f32(idx, data)
        elif s.fmt == "q8":
            q, sc = E.quantize_q8(data, 0)
            orc.set_q8(idx, q, sc)
        else:
            orc.set_q4_0(idx, E.quantize_q4_0(data))
    if not s.tied:
        orc.set_embed_f16(E.synth_normal(seed, 10_000_019, 0.02, (s.vocab, s.dim)).astype(np.float16))
    stream = list(prompt) + list(first_tokens)
    t0 = time.perf_counter()
    done = 0
    match = True
    for pos in range(len(stream) - 1):
        nxt, _, _ = orc.decode_token(int(stream[pos]), pos)
        done += 1
        if pos >= nP - 1 and nxt != int(stream[pos + 1]):
            match = False
        el = time.perf_counter() - t0
        if done >= sample and el + el / done > budget_s:
            break
    el = time.perf_counter() - t0
    orc.close()
    return {"value": done / el, "unit": "tok/s", "cores": 1, "host_cores": os.cpu_count(), "kind": "port",
            "sample": f"{done} tokens (positions 0..{done - 1} of the same prompt+decode stream) in {el:.1f} s, "
                      f"single thread; C restatement of the Go CPU engine, not the Go binary (no Go toolchain)",
            "tokens_match_gpu": bool(match)}


def oracle_for(ob, configs, s, maxSeq, threads):
    kv = configs.kv_dim(s)
    return ob.Oracle(s.dim, kv, s.headDim, s.nHeads, s.nKVHeads, s.ffnDim, s.vocab, s.nLayers, maxSeq, s.theta, s.eps,
                     threads=threads)


def launch_table(f, configs, s, first_tok, pos, steps, ms_per_step, kv_f16):
    """Per-launch-class averages inside eager steps at positions pos.. (HIP events on the context's stream)."""
    kv = configs.kv_dim(s)
    rc, cls_ms, cls_n = f.ProfileDecode(first_tok, pos, steps)
    assert rc == 0
    flow = f.FlowInUse()
    tail = flow and f.FlowTailInUse()

    def mat(n, k):
        return n * k + 4 * n if s.fmt == "q8" else n * (k // 32) * 18
    p_prof = pos + steps // 2
    kvb = 2 * (p_prof + 1) * kv * (2 if kv_f16 else 4)
    layer_w = mat(s.dim, s.dim) * 2 + 2 * mat(kv, s.dim) + 2 * mat(s.ffnDim, s.dim) + mat(s.dim, s.ffnDim) + 8 * s.dim
    cls_bytes = {
        1: ((layer_w + kvb) * s.nLayers + (mat(s.vocab, s.dim) + 4 * s.dim if tail else 0)) if flow
           else mat(s.dim, s.dim) + 2 * mat(kv, s.dim) + 4 * s.dim,
        2: kvb,
        3: mat(s.dim, s.dim),
        4: 2 * mat(s.ffnDim, s.dim) + 4 * s.dim,
        5: mat(s.dim, s.ffnDim),
        6: mat(s.vocab, s.dim) + 4 * s.dim,
    }
    rows = []
    total = sum(float(cls_ms[c]) * int(cls_n[c]) for c in range(8))
    for c in range(8):
        n = int(cls_n[c])
        if n == 0:
            continue
        ms = float(cls_ms[c])
        # share of the eager step's launch time (events between launches; a replayed graph runs the same kernels closer together)
        e = {"launch": (TOKEN_NAME if tail else FLOW_NAME) if (flow and c == 1) else LAUNCH_NAMES[c], "cls": c, "per_token": n, "avg_us": round(ms * 1e3, 3),
             "share_of_step": round(ms * n / total, 4) if total > 0 else None}
        if c in cls_bytes and ms > 0:
            e["bytes"] = int(cls_bytes[c])
            e["GBps"] = round(cls_bytes[c] / (ms * 1e-3) / 1e9, 1)
            e["frac_of_peak"] = round(e["GBps"] / HBM_PEAK_GBS, 4)
        rows.append(e)
    return rows


def phase_table(f, np, configs, s, first_tok, pos, kv_f16, steps=8):
    """Per-phase times inside the persistent launch from its own trace (100 MHz wall clock stamps per workgroup): for
    every matvec phase of a layer and for the lm_head, the bytes the phase reads over the time from the first workgroup
    having its input staged to the last workgroup being done (median over the layers of the last traced token)."""
    kv = configs.kv_dim(s)
    rc, _ = f.FlowTrace(True)
    if rc != 0:
        return None
    rc, _ = f.TimedDecode(first_tok, pos, steps, useGraph=True)
    assert rc == 0
    rc, tr = f.FlowTrace(True, read=True)
    assert rc == 0
    tt = None
    if f.FlowTailInUse():
        rc, tt = f.FlowTailTrace()
        assert rc == 0
    f.FlowTrace(False)

    def mat(n, k):
        return n * k + 4 * n if s.fmt == "q8" else n * (k // 32) * 18
    p_last = pos + steps - 1
    spans = [("norm+q|k|v (+bias, RoPE, KV write)", 1, 2, mat(s.dim, s.dim) + 2 * mat(kv, s.dim) + 4 * s.dim),
             ("attention", 3, 4, 2 * (p_last + 1) * kv * (2 if kv_f16 else 4)),
             ("Wo+residual", 5, 6, mat(s.dim, s.dim)),
             ("norm+gate|up+SwiGLU", 7, 8, 2 * mat(s.ffnDim, s.dim) + 4 * s.dim),
             ("down+residual", 9, 10, mat(s.dim, s.ffnDim))]
    nL = tr.shape[0]
    rows = []
    tot_phase = 0.0
    for name, a, b, nbytes in spans:
        us = []
        for l in range(1 if nL > 1 else 0, nL):
            ta, tb = tr[l, a][tr[l, a] > 0], tr[l, b][tr[l, b] > 0]
            if ta.size and tb.size:
                us.append((float(tb.max()) - float(ta.min())) / 100.0)
        if not us:
            continue
        u = float(np.median(us))
        tot_phase += u
        rows.append({"phase": name, "bytes": int(nbytes), "us": round(u, 2), "GBps": round(nbytes / u / 1e3, 1),
                     "frac_of_peak": round(nbytes / u / 1e3 / HBM_PEAK_GBS, 4)})
    layer_us = float(np.median(np.diff(np.median(tr[:, 0, :], axis=1)))) / 100.0 if nL > 1 else None
    out = {"position": p_last, "layer_us": round(layer_us, 2) if layer_us else None,
           "hand_overs_and_waits_us": round(layer_us - tot_phase, 2) if layer_us else None, "phases": rows,
           "note": "input staged by the first workgroup -> last workgroup done, per phase; a phase's weights may already be in "
                   "the L2s (read there by the prefetching workgroups during earlier phases), so a phase can exceed the HBM peak"}
    if tt is not None:
        lm = mat(s.vocab, s.dim) + 4 * s.dim
        staged, done, known = tt[1][tt[1] > 0], tt[4][tt[4] > 0], tt[3][tt[3] > 0]
        u = (float(done.max()) - float(staged.min())) / 100.0
        um = (float(np.median(done)) - float(np.median(staged))) / 100.0
        out["lm_head"] = {"phase": "final norm+lm_head+argmax partials", "bytes": int(lm), "us": round(u, 2),
                          "GBps": round(lm / u / 1e3, 1), "frac_of_peak": round(lm / u / 1e3 / HBM_PEAK_GBS, 4),
                          "us_median_workgroup": round(um, 2),
                          "frac_of_peak_median_workgroup": round(lm / um / 1e3 / HBM_PEAK_GBS, 4),
                          "token_known_after_us": round((float(known.max()) - float(done.max())) / 100.0, 2)}
    return out


def check_tokens(E, orc, prompt, toks, budget_s):
    """Greedy tokens of the GPU against the oracle's on the same stream, as far as the budget goes."""
    stream = list(prompt) + [int(t) for t in toks]
    nP = len(prompt)
    t0 = time.perf_counter()
    checked, match = 0, True
    for pos in range(len(stream) - 1):
        nxt, _, _ = orc.decode_token(int(stream[pos]), pos)
        if pos >= nP - 1:
            checked += 1
            if nxt != int(stream[pos + 1]):
                match = False
                break
        if time.perf_counter() - t0 > budget_s and checked >= 2:
            break
    return {"tokens_match": bool(match), "tokens_checked": checked, "oracle_s": round(time.perf_counter() - t0, 1)}


def measure(E, np, configs, eng, s, seed, W, K, contexts, profile_steps, use_graph=True, exec_mode=None, kv_f16=False,
            prefill=0, oracle_threads=0, check_budget_s=8.0, want_mode1_table=True, keep=False, tokens_per_launch=None,
            want_phases=True, flow_tail=True, stream_tokens=0, lean=False, flow_generic=False):
    """One configuration: load, warm up on the W prompt positions, time K decode steps at each start position of
    `contexts` (0 = right after the prompt), per-launch table, optional batched prefill, optional token check."""
    from oracle import binding as ob
    P = [max(c, W) for c in contexts]
    maxSeq = max(max(P) + K + profile_steps + 16, prefill + 8, W + 56)
    orc = oracle_for(ob, configs, s, W + 72, oracle_threads) if oracle_threads else None
    t_load = time.perf_counter()
    f = load_model(E, np, s, seed, maxSeq, eng, oracle=orc, kv_f16=kv_f16)
    if exec_mode is not None and f.SetExecMode(exec_mode) != 0:
        raise SystemExit("bench.py: " + E.last_error())
    if flow_generic:
        assert f.SetFlowGeneric(True) == 0
    if not flow_tail:
        f.SetFlowTail(False)
    t_load = time.perf_counter() - t_load
    prompt = E.synth_tokens(seed, 20_000_003, s.vocab, W)
    rc, first = f.Generate(prompt, 1, useGraph=use_graph)
    assert rc == 0, E.last_error()
    wbytes = configs.weight_bytes_per_token(s)
    assert f.WeightBytesPerToken() == wbytes
    flow = f.FlowInUse()
    tail = flow and f.FlowTailInUse()
    if tokens_per_launch is not None and f.SetTokensPerLaunch(tokens_per_launch) != 0:
        raise SystemExit("bench.py: " + E.last_error())
    tpl = f.TokensPerLaunch() if tail and use_graph else 1
    if tail:
        how = f"persistent launch running whole tokens, {tpl} tokens a launch" if tpl > 1 else \
              "persistent launch running a whole token, one launch a token" + (" (hipGraph replay)" if use_graph else " (eager)")
    else:
        how = ("persistent layer launch + lm_head + argmax" if flow else "fused launches (5 a layer)") + \
              (", hipGraph replay" if use_graph else ", eager")
    res = {"exec": how, "weight_bytes_per_token": int(wbytes), "load_s": round(t_load, 1), "runs": []}
    for P0 in P:
        rc, ms = f.TimedDecode(int(first[0]), P0, K, useGraph=use_graph)
        assert rc == 0, E.last_error()
        ms_step = ms / K
        step_bytes = wbytes + configs.kv_bytes_at(s, P0 + K // 2) // (2 if kv_f16 else 1)
        run = {"start_position": P0, "steps": K, "ms_per_step": round(ms_step, 5), "tok_per_s": round(K / (ms / 1e3), 1),
               "step_bytes": int(step_bytes), "step_GBps": round(step_bytes / (ms_step * 1e-3) / 1e9, 1),
               "step_roofline_frac": round(step_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
               "launches": (K + tpl - 1) // tpl}
        if tail and tpl > 1 and not lean:
            # the same steps as replays of the captured one-token graph (one launch a token)
            assert f.SetTokensPerLaunch(1) == 0
            rc, msg = f.TimedDecode(int(first[0]), P0, K, useGraph=use_graph)
            assert rc == 0, E.last_error()
            assert f.SetTokensPerLaunch(tpl) == 0
            run["graph_replay_one_token_a_launch_ms_per_step"] = round(msg / K, 5)
        if flow and want_phases and not lean:
            run["in_launch_phases"] = phase_table(f, np, configs, s, int(first[0]), P0 + K, kv_f16)
        table = [] if (lean and tail) else launch_table(f, configs, s, int(first[0]), P0 + K, profile_steps, ms_step, kv_f16)
        run["kernels"] = table
        if flow and want_mode1_table and not lean:
            assert f.SetExecMode(1) == 0
            rc, ms1 = f.TimedDecode(int(first[0]), P0, K, useGraph=use_graph)
            assert rc == 0, E.last_error()
            run["fused_launches_ms_per_step"] = round(ms1 / K, 5)
            run["kernels_fused_launches"] = launch_table(f, configs, s, int(first[0]), P0 + K, profile_steps, ms1 / K, kv_f16)
            assert f.SetExecMode(3 if exec_mode is None else exec_mode) == 0
            table = run["kernels_fused_launches"]
        if flow and P0 > W and not lean:
            # a long context is beyond the oracle's budget: the tokens of the launch that was timed against the fused
            # launches' (whose attention kernel the tests check against the oracle at this geometry), same positions
            seqs = {}
            for md in (3 if exec_mode is None else exec_mode, 1):
                assert f.SetExecMode(md) == 0
                tok, seq = int(first[0]), []
                for i in range(12):
                    rc, tok = f.DecodeToken(tok, P0 + i)
                    assert rc == 0, E.last_error()
                    seq.append(tok)
                seqs[md] = seq
            assert f.SetExecMode(3 if exec_mode is None else exec_mode) == 0
            a_, b_ = list(seqs.values())
            run["tokens_match_fused_launches"] = bool(a_ == b_)
            run["tokens_compared"] = len(a_)
        att = [e for e in table if e["cls"] == 2]
        if att and "GBps" in att[0]:
            run["attention_KV_GBps"] = att[0]["GBps"]
        res["runs"].append(run)
    # K/V read rate of the launches in use at a long context: the extra K/V bytes a step reads there, over the extra
    # time it takes, against the first (short) context of the same run
    for run in res["runs"][1:]:
        base = res["runs"][0]
        dms = run["ms_per_step"] - base["ms_per_step"]
        dbytes = (configs.kv_bytes_at(s, run["start_position"] + K // 2) - configs.kv_bytes_at(s, base["start_position"] + K // 2)) // (2 if kv_f16 else 1)
        if dms > 0 and dbytes > 0:
            run["KV_GBps_from_step_delta"] = round(dbytes / (dms * 1e-3) / 1e9, 1)
            run["KV_GBps_note"] = f"extra K/V bytes over extra step time against start_position {base['start_position']}"
    if prefill > 0:
        ptoks = E.synth_tokens(seed, 20_000_003, s.vocab, prefill)
        times = []
        for _ in range(4):                              # first call allocates the row buffers
            assert f.ResetKV() == 0
            rc, _, _, pms = f.Prefill(ptoks, 0)
            assert rc == 0, E.last_error()
            times.append(pms)
        pms = min(times[1:])
        kv = configs.kv_dim(s)
        macs = sum(n * k for n, k in
                   [(s.dim, s.dim), (kv, s.dim), (kv, s.dim), (s.dim, s.dim), (s.ffnDim, s.dim), (s.ffnDim, s.dim),
                    (s.dim, s.ffnDim)]) * s.nLayers
        flops = 2.0 * macs * prefill
        res["prefill"] = {"tokens": prefill, "ms": round(pms, 3), "tok_per_s": round(prefill / (pms * 1e-3), 1),
                          "model_TFLOPs": round(flops / (pms * 1e-3) / 1e12, 2),
                          "mfma_TFLOPs_issued": round(2 * flops / (pms * 1e-3) / 1e12, 2),
                          "mfma_frac_of_bf16_peak": round(2 * flops / (pms * 1e-3) / 1e12 / 2500.0, 4),
                          "note": "model flops = 2*T*weights of the layer projections; each is issued twice (bf16 hi and lo activation terms)"}
    toks = None
    if (orc is not None or keep) and not lean:
        # the token check runs on a 4-token prompt, so that the oracle's budget goes into decoded tokens
        cprompt = prompt[:4] if orc is not None else prompt
        assert f.ResetKV() == 0
        rc, toks = f.Generate(cprompt, 48, useGraph=use_graph)
        assert rc == 0, E.last_error()
    if orc is not None:
        res.update(check_tokens(E, orc, cprompt, toks, check_budget_s))
        res["tokens_checked_at"] = "positions 3.. of a 4-token prompt + 48 decode tokens (short context)"
        orc.close()
    if stream_tokens > 0 and s.fmt == "q4_0":
        res["stream"] = stream_leg(E, np, configs, f, s, seed, stream_tokens)
    if keep:
        return res, f, prompt, first, toks
    f.Close()
    return res


def stream_leg(E, np, configs, f, s, seed, n):
    """n tokens through the weight-streaming front end (every layer's Q4_0 blocks cross PCIe per token)."""
    kv = configs.kv_dim(s)
    st = f.StreamBuild()
    assert st is not None, E.last_error()
    ptrs, sizes = [], []
    for l in range(s.nLayers):
        for w in range(12):
            idx = l * 12 + w
            rows, cols = slot_shape(s, kv, idx)
            if cols == 1:
                ptrs.append(gen_slot(E, np, s, kv, seed, idx) if (w not in (4, 5, 6) or s.bias) else None)
            else:
                blk = E.quantize_q4_0(gen_slot(E, np, s, kv, seed, idx))
                ptrs.append(blk)
                sizes.append(blk.size)
    layer_bytes = sum(a.nbytes for a in ptrs if a is not None)
    assert f.ResetKV() == 0
    h0 = np.zeros(s.dim, np.float32)
    h0[:] = E.synth_normal(seed, 30_000_001, 0.02, (s.dim,))
    logits = np.empty(s.vocab, np.float32)
    for pos in range(2):                               # warm the staging buffers
        assert st.StreamForwardToken(pos, h0, s.nLayers, ptrs, sizes, logits) == 0, E.last_error()
    t0 = time.perf_counter()
    for i in range(n):
        assert st.StreamForwardToken(2 + i, h0, s.nLayers, ptrs, sizes, logits) == 0, E.last_error()
    el = time.perf_counter() - t0
    st.Close()
    return {"tokens": n, "ms_per_token": round(el / n * 1e3, 3),
            "tok_per_s": round(n / el, 1), "host_to_device_bytes_per_token": int(layer_bytes),
            "host_to_device_GBps": round(layer_bytes * n / el / 1e9, 2),
            "note": "host wall clock; every token stages all layers from pageable host memory through two pinned "
                    "buffers into two device sets (copy of layer l+1 overlaps compute of layer l); logits read back each token"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--config", default="qwen2.5-0.5b")
    ap.add_argument("--seed", type=int, default=20250)
    ap.add_argument("--cpu-budget", type=float, default=20.0, help="seconds of CPU baseline work (0 = skip)")
    ap.add_argument("--profile-steps", type=int, default=20)
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--exec-mode", type=int, default=-1, choices=[-1, 0, 1, 2, 3, 4],
                    help="-1 = the library's automatic choice (default); 1 = fused launches; 2 = the same without the L2 prefetch by "
                         "the attention launch's idle workgroups; 3 = one persistent launch for all layers wherever the model allows it")
    ap.add_argument("--context", type=int, default=0,
                    help="start the timed decode at this position (KV rows between the prompt and it are zeros): long-context timing")
    ap.add_argument("--pmc-copy", action="store_true",
                    help="also run three 256 MiB device copies (a kernel of known traffic, to scale rocprofv3 --pmc counters)")
    ap.add_argument("--kv", choices=["f32", "f16"], default="f32",
                    help="KV cache row format (f32 is the reference's; f16 is this backend's option, not the headline configuration)")
    ap.add_argument("--prefill", type=int, default=0,
                    help="also time a batched prefill of this many prompt tokens (extra 'prefill' object)")
    ap.add_argument("--stream", type=int, default=0,
                    help="also time this many tokens through the weight-streaming front end (Q4_0 configurations: "
                         "every layer's weights cross PCIe per token; extra 'stream' object)")
    ap.add_argument("--flow-trace", action="store_true",
                    help="also record the persistent layer launch's per-workgroup timeline (extra 'flow_trace' object)")
    ap.add_argument("--tokens-per-launch", type=int, default=0,
                    help="tokens the persistent launch runs per launch (0 = the library's default, 64; 1 = a launch per token)")
    ap.add_argument("--no-flow-tail", action="store_true",
                    help="lm_head and argmax as launches of their own behind the persistent layer launch (for comparisons)")
    ap.add_argument("--lean", action="store_true",
                    help="only the timed region of the configuration (no per-launch tables, no graph-replay leg, no trace, no "
                         "token check): the run to put under rocprofv3")
    ap.add_argument("--flow-generic", action="store_true",
                    help="only the persistent launch's variants whose sizes come with the launch (for comparisons with the "
                         "variants that have a known shape's sizes compiled in)")
    ap.add_argument("--no-live-pmc", action="store_true",
                    help="do not run the two rocprofv3 --pmc passes that measure the launch's HBM traffic (the figures recorded "
                         "from profiles/ are reported instead)")
    ap.add_argument("--no-configs", action="store_true",
                    help="only the configuration named by --config (no 'configs' object with the other benchmark configurations)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); "
              "the decode path is batch-1 on a single device", file=sys.stderr)
        sys.exit(2)

    # HBM traffic of the run's own launches, from counters: before anything here touches the GPU (the profiler runs
    # children of this process).  Only for the default path, whose dispatches the passes can pick out.
    pmc_live, pmc_why = None, "not the default path (flags)"
    default_path = (not args.lean and args.exec_mode < 0 and not args.no_flow_tail and args.context == 0 and args.kv == "f32"
                    and not args.tokens_per_launch and not args.no_graph and not args.pmc_copy and not args.flow_generic)
    if default_path and not args.no_live_pmc:
        pmc_live, pmc_why = live_pmc_traffic(args.config, args.steps, max(args.warmup, 1))

    import numpy as np
    from mongoose_amd import configs
    from mongoose_amd import engine as E

    s = configs.BY_NAME[args.config]
    eng = E.NewHIP(0)
    if eng is None:
        print("bench.py: no HIP device", file=sys.stderr)
        sys.exit(1)
    K, W = args.steps, max(args.warmup, 1)
    use_graph = not args.no_graph
    kv_f16 = args.kv == "f16"
    mode = None if args.exec_mode < 0 else args.exec_mode
    res, f, prompt, first, toks = measure(E, np, configs, eng, s, args.seed, W, K, [args.context], args.profile_steps,
                                          use_graph=use_graph, exec_mode=mode, kv_f16=kv_f16, prefill=args.prefill,
                                          oracle_threads=0, keep=not args.lean or True, tokens_per_launch=args.tokens_per_launch or None,
                                          flow_tail=not args.no_flow_tail, lean=args.lean, flow_generic=args.flow_generic)
    run = res["runs"][0]
    P0 = run["start_position"]
    ms_per_step = run["ms_per_step"]
    toks_per_s = K / (ms_per_step * K / 1e3)
    flow = f.FlowInUse()

    tail = flow and f.FlowTailInUse()
    table = run["kernels"]

    def roof(entry, ms, key):
        sec = ms * 1e-3
        b = entry["bytes"]
        return {"bound": "hbm", "kernel": entry["launch"], "achieved": round(b / sec / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(b / sec / 1e9 / HBM_PEAK_GBS, 4), "bytes_per_launch": int(b), "avg_launch_us": round(sec * 1e6, 2),
                "launches_per_step": entry["per_token"], "share_of_step": entry["share_of_step"],
                "launches_timed": int(args.profile_steps) * entry["per_token"],
                "traffic": PMC_TRAFFIC_BYTES.get((s.name, key)),
                "traffic_source": PMC_SOURCE if (s.name, key) in PMC_TRAFFIC_BYTES else None}
    if tail:
        # The step is one kernel: the launch that runs whole tokens.  Its average duration is the timed region itself (HIP
        # events on the context's stream around the K steps), divided by the launches it took.
        launches = run["launches"]
        sec = ms_per_step * 1e-3 * K / launches
        b = run["step_bytes"] * K / launches
        tr_b = PMC_TRAFFIC_BYTES.get((s.name, "token"))
        roofline = {"bound": "hbm", "kernel": TOKEN_NAME, "achieved": round(b / sec / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(b / sec / 1e9 / HBM_PEAK_GBS, 4), "bytes_per_launch": int(b), "avg_launch_us": round(sec * 1e6, 2),
                    "tokens_per_launch": round(K / launches, 2), "launches_timed": launches, "share_of_step": 1.0,
                    "traffic": int(tr_b * K / launches) if tr_b else None,
                    "traffic_source": PMC_SOURCE if tr_b else None,
                    "traffic_note": None if tr_b else "not collected for this kernel"}
        if pmc_live and all(len(pmc_live[c][0]) >= launches for c in pmc_live):
            # the timed launches are the last `launches` dispatches of the kernel in each pass (the same command line)
            fe, ff = pmc_live["FETCH_SIZE"]
            wr, wf = pmc_live["WRITE_SIZE"]
            tb = (sum(fe[-launches:]) * ff + sum(wr[-launches:]) * wf) * 1024.0 / launches
            roofline["traffic_recorded"] = roofline["traffic"]
            roofline["traffic"] = int(tb)
            roofline["traffic_over_algorithmic"] = round(tb / b, 4)
            roofline["traffic_source"] = ("measured by this run: rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE passes over `bench.py --lean "
                                          "--pmc-copy` with this configuration, made before the timing (same build, same box); KiB per dispatch of "
                                          f"the timed launches, scaled by what the same counters read for 256 MiB device copies (x{ff:.4f} / x{wf:.4f})")
            roofline["traffic_note"] = None
        elif not args.lean:
            roofline["traffic_note"] = ((roofline["traffic_note"] + "; ") if roofline["traffic_note"] else "") + \
                f"no live counter passes: {pmc_why or 'fewer dispatches in the counter files than timed launches'}"
        ph = run.get("in_launch_phases") or {}
        lmh = ph.get("lm_head")
        sep = [e for e in (run.get("kernels_fused_launches") or []) if e["cls"] == 6]
        matvec = None
        if lmh:
            matvec = {"bound": "hbm", "kernel": "final norm + lm_head + argmax partials, a phase of the persistent launch",
                      "achieved": lmh["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": lmh["frac_of_peak"],
                      "bytes": lmh["bytes"], "us": lmh["us"],
                      "timed_by": "the launch's own 100 MHz wall-clock stamps: first workgroup's input staged -> last workgroup's last wave done",
                      "median_workgroup": {"us": lmh["us_median_workgroup"], "frac": lmh["frac_of_peak_median_workgroup"]},
                      "as_a_launch_of_its_own_event_timed": sep[0] if sep else None}
    else:
        # the launch that takes most of the step, and the lm_head matvec, once more with events around them alone
        # (less event overhead inside their intervals)
        dom = max(table, key=lambda e: e["avg_us"] * e["per_token"])
        rc, only, _ = f.ProfileDecode(int(first[0]), P0 + K, args.profile_steps, classMask=(1 << dom["cls"]) | (1 << 6))
        assert rc == 0, E.last_error()
        roofline = roof(dom, float(only[dom["cls"]]), "flow" if (flow and dom["cls"] == 1) else LAUNCH_NAMES[dom["cls"]])
        lm = [e for e in table if e["cls"] == 6][0]
        matvec = roof(lm, float(only[6]), "lm_head")

    flow_trace = None
    if args.flow_trace and flow:
        rc, _ = f.FlowTrace(True)
        assert rc == 0, E.last_error()
        rc, _ = f.TimedDecode(int(first[0]), P0 + K, 8, useGraph=use_graph)
        assert rc == 0, E.last_error()
        rc, tr = f.FlowTrace(True, read=True)
        assert rc == 0, E.last_error()
        f.FlowTrace(False)
        L = s.nLayers // 2
        base = float(np.median(tr[L, 0]))
        pts = []
        for b, name in enumerate(f.FLOW_TRACE_POINTS):
            v = (tr[L, b][tr[L, b] > 0] - base) / 100.0
            pts.append({"point": name, "workgroups": int(v.size), "min_us": round(float(v.min()), 2),
                        "median_us": round(float(np.median(v)), 2), "max_us": round(float(v.max()), 2)})
        flow_trace = {"position": P0 + K + 7, "layer": L, "zero": "median workgroup entering the layer",
                      "points": pts, "layer_us": round((float(np.median(tr[L + 1, 0])) - base) / 100.0, 2),
                      "all_layers_us": round((float(tr[-1, -1].max()) - float(np.median(tr[0, 0]))) / 100.0, 1)}

    if args.pmc_copy:
        n = 256 << 20
        a, b = eng.UploadRawBytes(np.zeros(n, np.uint8)), eng.UploadRawBytes(np.zeros(n, np.uint8))
        for _ in range(3):
            E.KCopy(b, a, n)
        E.KSync()
        a.Release()
        b.Release()

    stream = None
    if args.stream > 0:
        if s.fmt != "q4_0":
            print("bench.py: --stream needs a Q4_0 configuration (the streaming front end takes GGUF block_q4_0 layers)",
                  file=sys.stderr)
            sys.exit(2)
        stream = stream_leg(E, np, configs, f, s, args.seed, args.stream)
    f.Close()

    cpu = None
    if args.cpu_budget > 0 and not args.lean:
        cpu = cpu_baseline(E, np, s, args.seed, prompt, toks, args.cpu_budget, kv_f16=kv_f16)

    others = None
    if not args.no_configs and not args.lean and args.config == "qwen2.5-0.5b":
        others = {}
        plan = [("toy", dict(K=200, contexts=[0], threads=8)),
                ("tinyllama-1.1b", dict(K=50, contexts=[0], threads=16)),
                ("qwen2.5-0.5b-q4_0", dict(K=200, contexts=[0], threads=16, stream=20)),
                ("llama-3-8b", dict(K=64, contexts=[0, 4000], threads=16, prefill=512))]
        for name, o in plan:
            print(f"bench.py: configuration {name}", file=sys.stderr, flush=True)
            others[name] = measure(E, np, configs, eng, configs.BY_NAME[name], args.seed + 1, 16, o["K"], o["contexts"],
                                   10, use_graph=True, prefill=o.get("prefill", 0), oracle_threads=o["threads"],
                                   check_budget_s=10.0, stream_tokens=o.get("stream", 0))
        # the 8B shape's long-context leg once more with fp16 K/V rows (this backend's option, mg_set_kv_format)
        print("bench.py: configuration llama-3-8b, fp16 K/V rows", file=sys.stderr, flush=True)
        others["llama-3-8b-kv-f16"] = measure(E, np, configs, eng, configs.BY_NAME["llama-3-8b"], args.seed + 1, 16, 64, [4000],
                                              10, use_graph=True, kv_f16=True, oracle_threads=0, want_mode1_table=False)

    out = {
        "metric": "Q8 decode tok/s (bs=1, Qwen2.5-0.5B shape) + matvec HBM GB/s % of peak" if s.name == "qwen2.5-0.5b"
                  else f"decode tok/s (bs=1, {s.name} shape)",
        "value": round(toks_per_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "weight_dtype": "int8 per-row scale" if s.fmt == "q8" else "q4_0 (fp16 block scale)",
        "data": "synthetic",
        "config": {"workload": f"{s.name} shape, random-init {s.fmt.upper()} weights, greedy decode: {W}-token prompt, {K} decode "
                               f"tokens from position {P0}, batch 1, {'fp16' if kv_f16 else 'fp32'} KV cache; {res['exec']}"},
        "step_bytes": run["step_bytes"], "step_GBps": run["step_GBps"], "step_roofline_frac": run["step_roofline_frac"],
        "roofline": roofline, "matvec": matvec, "kernels": run["kernels"],
        "kernels_fused_launches": run.get("kernels_fused_launches"),
        "fused_launches_ms_per_step": run.get("fused_launches_ms_per_step"),
        "graph_replay_one_token_a_launch_ms_per_step": run.get("graph_replay_one_token_a_launch_ms_per_step"),
        "in_launch_phases": run.get("in_launch_phases"),
        "cpu_baseline": cpu, "prefill": res.get("prefill"), "stream": stream, "flow_trace": flow_trace, "configs": others,
        "load_s": res["load_s"], "device": eng.Name(),
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the fused quantized decode path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME]

A "step" is one batch-1 greedy decode token through the whole path (embedding
gather -> layers -> final norm -> lm_head -> argmax), replayed from a captured
hipGraph with the position and the token resident on the device.  The W warmup
steps are the W prompt positions; the K timed steps are the K decode positions
after them.  Weights are synthetic (seeded N(0, 0.02), quantized on the host by
the library's own loader) and resident in HBM before the timed region starts.

Prints ONE JSON line with the throughput, the roofline of the dominant kernel
(the lm_head matvec) measured inside the replayed token, a per-launch-class
table, and the CPU oracle timed on this box's host cores as a baseline.
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

# HBM bytes per launch of the lm_head kernel from rocprofv3 --pmc runs of this script
# (FETCH_SIZE then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter
# reads for a 256 MiB device copy in the same run (FETCH_SIZE reads 131106.2 KiB for the
# 262144 KiB copied -> x1.9995; WRITE_SIZE reads 262144.0 -> x1.0).  Counts are a property
# of kernel and shape, so they are recorded here; profiles/ holds the run they come from.
PMC_TRAFFIC_BYTES = {
    "qwen2.5-0.5b": int((67136.6 * (262144.0 / 131106.2) + 661.7 * 1.0) * 1024),
}


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
    return {"value": done / el, "unit": "tok/s", "cores": 1, "kind": "port",
            "sample": f"{done} tokens (positions 0..{done - 1} of the same prompt+decode stream) in {el:.1f} s, "
                      f"single thread; C restatement of the Go CPU engine, not the Go binary (no Go toolchain)",
            "tokens_match_gpu": bool(match)}


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
    ap.add_argument("--exec-mode", type=int, default=1, choices=[1, 2],
                    help="1 = fused launches (default); 2 = the same without the L2 prefetch by the attention launch's idle workgroups")
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
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); "
              "the decode path is batch-1 on a single device", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    from mongoose_amd import configs
    from mongoose_amd import engine as E

    s = configs.BY_NAME[args.config]
    eng = E.NewHIP(0)
    if eng is None:
        print("bench.py: no HIP device", file=sys.stderr)
        sys.exit(1)
    K, W = args.steps, max(args.warmup, 1)
    P0 = max(args.context, W)                      # position of the first timed step
    maxSeq = max(P0 + K + args.profile_steps + 8, args.prefill, args.stream + 2)
    t_load = time.perf_counter()
    kv_f16 = args.kv == "f16"
    f = load_model(E, np, s, args.seed, maxSeq, eng, kv_f16=kv_f16)
    if args.exec_mode != 1 and f.SetExecMode(args.exec_mode) != 0:
        raise SystemExit("bench.py: " + E.last_error())
    t_load = time.perf_counter() - t_load
    prompt = E.synth_tokens(args.seed, 20_000_003, s.vocab, W)
    use_graph = not args.no_graph

    # warmup = the W prompt positions (+ graph capture), then the first decoded token
    rc, first = f.Generate(prompt, 1, useGraph=use_graph)
    assert rc == 0, E.last_error()
    # timed region: K decode steps at positions W .. W+K-1, token and position stay on the device
    rc, ms = f.TimedDecode(int(first[0]), P0, K, useGraph=use_graph)
    assert rc == 0, E.last_error()
    toks_per_s = K / (ms / 1e3)
    ms_per_step = ms / K

    # the same K tokens again to read them back (for the CPU baseline's comparison)
    assert f.ResetKV() == 0
    rc, toks = f.Generate(prompt, min(K, 48), useGraph=use_graph)
    assert rc == 0, E.last_error()

    # per-launch-class timing inside a replayed token
    kv = configs.kv_dim(s)
    rc, cls_ms, cls_n = f.ProfileDecode(int(first[0]), P0 + K, args.profile_steps)
    assert rc == 0, E.last_error()
    cls_ms = [float(x) for x in cls_ms]
    cls_n = [int(x) for x in cls_n]
    # the dominant kernel once more with events around it alone (less event overhead in its interval)
    rc, lm_only, _ = f.ProfileDecode(int(first[0]), P0 + K, args.profile_steps, classMask=1 << 6)
    assert rc == 0, E.last_error()
    lm_only_ms = float(lm_only[6])

    def mat(n, k):
        return n * k + 4 * n if s.fmt == "q8" else n * (k // 32) * 18
    p_mid = P0 + K // 2
    p_prof = P0 + K + args.profile_steps // 2
    cls_bytes = {
        1: mat(s.dim, s.dim) + 2 * mat(kv, s.dim) + 4 * s.dim,
        2: 2 * (p_prof + 1) * kv * (2 if kv_f16 else 4),
        3: mat(s.dim, s.dim),
        4: 2 * mat(s.ffnDim, s.dim) + 4 * s.dim,
        5: mat(s.dim, s.ffnDim),
        6: mat(s.vocab, s.dim) + 4 * s.dim,
    }
    names = {0: "embed_gather", 1: "norm+qkv", 2: "rope+kvwrite+attention", 3: "wo+residual", 4: "norm+gate_up+swiglu",
             5: "down+residual", 6: "norm+lm_head+argmax_partials", 7: "argmax_finish"}
    kernels = []
    for c in range(8):
        if cls_n[c] == 0:
            continue
        e = {"launch": names[c], "per_token": int(cls_n[c]), "avg_us": round(float(cls_ms[c]) * 1e3, 3)}
        if c in cls_bytes and cls_ms[c] > 0:
            e["bytes"] = int(cls_bytes[c])
            e["GBps"] = round(cls_bytes[c] / (cls_ms[c] * 1e-3) / 1e9, 1)
            e["frac_of_peak"] = round(e["GBps"] / HBM_PEAK_GBS, 4)
        kernels.append(e)

    wbytes = configs.weight_bytes_per_token(s)
    assert f.WeightBytesPerToken() == wbytes
    step_bytes = wbytes + configs.kv_bytes_at(s, p_mid) // (2 if kv_f16 else 1)
    lm_bytes = cls_bytes[6]
    lm_s = lm_only_ms * 1e-3
    roofline = {"bound": "hbm", "kernel": "matvec lm_head (final norm + Q8 matvec + argmax partials)",
                "achieved": round(lm_bytes / lm_s / 1e9, 1) if lm_s > 0 else None, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(lm_bytes / lm_s / 1e9 / HBM_PEAK_GBS, 4) if lm_s > 0 else None,
                "bytes_per_launch": int(lm_bytes), "avg_launch_us": round(lm_s * 1e6, 2),
                "launches_timed": int(args.profile_steps), "traffic": PMC_TRAFFIC_BYTES.get(s.name)}

    if args.pmc_copy:
        n = 256 << 20
        a, b = eng.UploadRawBytes(np.zeros(n, np.uint8)), eng.UploadRawBytes(np.zeros(n, np.uint8))
        for _ in range(3):
            E.KCopy(b, a, n)
        E.KSync()
        a.Release()
        b.Release()

    prefill = None
    if args.prefill > 0:
        ptoks = E.synth_tokens(args.seed, 20_000_003, s.vocab, args.prefill)
        times = []
        for _ in range(4):                              # first call allocates the row buffers
            assert f.ResetKV() == 0
            rc, _, _, pms = f.Prefill(ptoks, 0)
            assert rc == 0, E.last_error()
            times.append(pms)
        pms = min(times[1:])
        macs = sum(n * k for n, k in
                   [(s.dim, s.dim), (kv, s.dim), (kv, s.dim), (s.dim, s.dim), (s.ffnDim, s.dim), (s.ffnDim, s.dim),
                    (s.dim, s.ffnDim)]) * s.nLayers
        flops = 2.0 * macs * args.prefill
        prefill = {"tokens": args.prefill, "ms": round(pms, 3), "tok_per_s": round(args.prefill / (pms * 1e-3), 1),
                   "model_TFLOPs": round(flops / (pms * 1e-3) / 1e12, 2),
                   "mfma_TFLOPs_issued": round(2 * flops / (pms * 1e-3) / 1e12, 2),
                   "note": "model flops = 2*T*weights of the layer projections; each is issued twice (bf16 hi and lo activation terms)"}

    stream = None
    if args.stream > 0:
        if s.fmt != "q4_0":
            print("bench.py: --stream needs a Q4_0 configuration (the streaming front end takes GGUF block_q4_0 layers)",
                  file=sys.stderr)
            sys.exit(2)
        st = f.StreamBuild()
        assert st is not None, E.last_error()
        ptrs, sizes = [], []
        for l in range(s.nLayers):
            for w in range(12):
                idx = l * 12 + w
                rows, cols = slot_shape(s, kv, idx)
                if cols == 1:
                    ptrs.append(gen_slot(E, np, s, kv, args.seed, idx) if (w not in (4, 5, 6) or s.bias) else None)
                else:
                    blk = E.quantize_q4_0(gen_slot(E, np, s, kv, args.seed, idx))
                    ptrs.append(blk)
                    sizes.append(blk.size)
        layer_bytes = sum(a.nbytes for a in ptrs if a is not None)
        assert f.ResetKV() == 0
        h0 = np.zeros(s.dim, np.float32)
        h0[:] = E.synth_normal(args.seed, 30_000_001, 0.02, (s.dim,))
        logits = np.empty(s.vocab, np.float32)
        for pos in range(2):                               # warm the staging buffers
            assert st.StreamForwardToken(pos, h0, s.nLayers, ptrs, sizes, logits) == 0, E.last_error()
        t0 = time.perf_counter()
        for i in range(args.stream):
            assert st.StreamForwardToken(2 + i, h0, s.nLayers, ptrs, sizes, logits) == 0, E.last_error()
        el = time.perf_counter() - t0
        st.Close()
        stream = {"tokens": args.stream, "ms_per_token": round(el / args.stream * 1e3, 3),
                  "tok_per_s": round(args.stream / el, 1), "host_to_device_bytes_per_token": int(layer_bytes),
                  "host_to_device_GBps": round(layer_bytes * args.stream / el / 1e9, 2),
                  "note": "host wall clock; every token stages all layers from pageable host memory through two pinned "
                          "buffers into two device sets (copy of layer l+1 overlaps compute of layer l); logits read back each token"}

    cpu = None
    if args.cpu_budget > 0:
        cpu = cpu_baseline(E, np, s, args.seed, prompt, toks, args.cpu_budget, kv_f16=kv_f16)

    out = {
        "metric": "Q8 decode tok/s (bs=1, Qwen2.5-0.5B shape) + matvec HBM GB/s % of peak" if s.name == "qwen2.5-0.5b"
                  else f"decode tok/s (bs=1, {s.name} shape)",
        "value": round(toks_per_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "weight_dtype": "int8 per-row scale" if s.fmt == "q8" else "q4_0 (fp16 block scale)",
        "data": "synthetic",
        "config": {"workload": f"{s.name} random-init {s.fmt.upper()} greedy decode, {W}-token prompt, {K} decode tokens, "
                               f"batch 1, {'fp16' if kv_f16 else 'fp32'} KV cache", "layers": s.nLayers, "hidden": s.dim, "heads": s.nHeads,
                   "kv_heads": s.nKVHeads, "ffn": s.ffnDim, "vocab": s.vocab, "graph_replay": use_graph},
        "step_bytes": int(step_bytes), "step_GBps": round(step_bytes * toks_per_s / 1e9, 1),
        "step_roofline_frac": round(step_bytes * toks_per_s / 1e9 / HBM_PEAK_GBS, 4),
        "roofline": roofline, "kernels": kernels, "cpu_baseline": cpu, "prefill": prefill, "stream": stream,
        "load_s": round(t_load, 1), "device": eng.Name(),
    }
    f.Close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()

"""CPU-side checks of the product: the C ABI library loads and exports every
symbol the header declares, and its host-side quantizers / fp16 conversion /
synthetic generator agree bit for bit with the oracle (no GPU needed)."""
import os
import re
import subprocess

import numpy as np

from mongoose_amd import engine as E
from mongoose_amd.lib import LIB_PATH, lib
from oracle import binding as ob

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
rng = np.random.default_rng(99)


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "mongoose_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b((?:mg|tw|mongoose)_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) > 50
    out = subprocess.check_output(["nm", "-D", "--defined-only", LIB_PATH], text=True)
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l}
    missing = sorted(declared - exported)
    assert not missing, missing
    for name in declared:
        assert getattr(lib, name) is not None


def test_host_q8_quantizer_matches_oracle_bit_for_bit():
    w = (rng.standard_normal((64, 896)) * 0.02).astype(np.float32)
    w[0] = 0
    w[1, 5] = 9.0
    for mode in (0, 1):
        q, s = E.quantize_q8(w, mode)
        qo, so = ob.quantize_q8(w, mode)
        assert (q == qo).all() and (s.view(np.uint32) == so.view(np.uint32)).all()


def test_host_q4_0_quantizer_matches_oracle_bit_for_bit():
    w = (rng.standard_normal((32, 4864)) * 0.02).astype(np.float32)
    w[0, :32] = 0
    assert (E.quantize_q4_0(w) == ob.quantize_q4_0(w)).all()


def test_host_fp16_matches_oracle():
    xs = np.concatenate([(rng.standard_normal(5000) * 10.0 ** rng.uniform(-9, 5, 5000)).astype(np.float32),
                         np.array([0, -0.0, 65504, 65520, 1e9, 2.0 ** -24, 2.0 ** -25, 6e-8], np.float32)])
    for x in xs:
        assert lib.mg_f32_to_f16(float(x)) == ob.lib.orc_f32_to_f16(float(x))
    for b in range(0, 65536, 7):
        a, o = lib.mg_f16_to_f32(b), ob.lib.orc_f16_to_f32(b)
        assert (np.isnan(a) and np.isnan(o)) or a == o


def test_synthetic_generator_is_deterministic_and_normal():
    a = E.synth_normal(1, 2, 0.02, (1000, 333))
    b = E.synth_normal(1, 2, 0.02, (1000, 333))
    assert (a == b).all()
    assert not (a == E.synth_normal(1, 3, 0.02, (1000, 333))).all()
    assert abs(float(a.mean())) < 2e-4 and abs(float(a.std()) - 0.02) < 2e-4
    # fraction beyond 2 sigma ~ 4.55 %
    assert abs(float((np.abs(a) > 0.04).mean()) - 0.0455) < 0.003
    # pinned values: the stream must be the same on every machine
    c = E.synth_normal(42, 7, 1.0, (8,))
    assert c.view(np.uint32).tolist() == PINNED_42_7
    t = E.synth_tokens(42, 7, 151936, 6)
    assert t.tolist() == PINNED_TOK_42_7 and t.min() >= 0 and t.max() < 151936


PINNED_42_7 = [3211424173, 1066722117, 1057553308, 3206656046, 3224072043, 3213916856, 1036707676, 1063582405]
PINNED_TOK_42_7 = [27601, 53205, 31491, 35801, 36736, 81368]


def test_context_requires_device_or_fails_cleanly():
    # Without a GPU, NewHIP() is None and so is the context (nil constructor
    # convention, cuda.go:213-217); with one, both exist.
    eng = E.NewHIP()
    f = E.NewHIPFusedInference(eng, 512, 512, 64, 8, 8, 1376, 256, 1, 16, 1e4, 1e-5)
    if eng is None:
        assert f is None
    else:
        assert f is not None and f.NumWeights() == 14
        f.Close()


def test_host_worker_pool_is_safe_under_concurrent_callers():
    """The library's host loops share one set of worker threads, one parallel region at a time.
    Several Python threads (ctypes drops the GIL) quantizing matrices of very different sizes at
    once must each get exactly what a lone caller gets."""
    import threading
    mats = [(rng.standard_normal((r, 256)) * 0.02).astype(np.float32) for r in (1, 3, 17, 64, 300, 1000)]
    want = [(E.quantize_q8(m, 0), E.quantize_q4_0(m)) for m in mats]
    bad = []

    def worker(seed):
        for it in range(60):
            i = (seed + it) % len(mats)
            q, s = E.quantize_q8(mats[i], 0)
            b = E.quantize_q4_0(mats[i])
            if not (np.array_equal(q, want[i][0][0]) and np.array_equal(s, want[i][0][1]) and np.array_equal(b, want[i][1])):
                bad.append((seed, it))

    ths = [threading.Thread(target=worker, args=(k,)) for k in range(6)]
    for t in ths:
        t.start()
    for t in ths:
        t.join()
    assert not bad, bad[:5]

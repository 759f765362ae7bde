"""Writes tests/golden/toy_q8.npz from the CPU oracle: the toy configuration's
full workload (8-token prompt, 64 greedy tokens) with logits and final hidden
states at a few positions.  The reference holds no vectors for this path (its
fused inference has no tests), so these are produced by the oracle, which is
itself pinned by tests/test_oracle_*.py.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from mongoose_amd import configs  # noqa: E402
from tests import helpers as H  # noqa: E402

SEED = 1
POSITIONS = [0, 7, 40, 70]


def main():
    s = configs.TOY
    m = H.Model(s, seed=SEED, maxSeq=72, eng=None, oracle=True, threads=4)
    prompt = m.prompt(8)
    toks, rec = H.oracle_generate(m, prompt, 64, want=set(POSITIONS))
    toks64, _ = H.oracle_generate(m, prompt, 64, shadow=True)
    assert (toks == toks64).all(), "float and double oracle paths disagree; choose another seed"
    logits = np.stack([rec[p][0] for p in POSITIONS])
    hidden_last = np.stack([rec[p][1][-1] for p in POSITIONS])
    layer_hidden = np.stack([rec[p][1] for p in POSITIONS])
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "toy_q8.npz")
    np.savez_compressed(out, seed=np.int64(SEED), prompt=prompt, tokens=toks, positions=np.array(POSITIONS, np.int32),
                        logits=logits, hidden_last=hidden_last, layer_hidden=layer_hidden)
    print(out, os.path.getsize(out), "bytes; tokens:", toks.tolist())


if __name__ == "__main__":
    main()

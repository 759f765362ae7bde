"""The committed toy fixture against a fresh oracle run: guards the oracle and
the synthetic-weight generator against drifting between machines."""
import os

import numpy as np

from mongoose_amd import configs
from tests import helpers as H


def test_oracle_reproduces_toy_fixture():
    fx = np.load(os.path.join(os.path.dirname(__file__), "golden", "toy_q8.npz"))
    m = H.Model(configs.TOY, seed=int(fx["seed"]), maxSeq=72, eng=None, oracle=True, threads=4)
    prompt = m.prompt(8)
    assert (prompt == fx["prompt"]).all()
    want = set(int(p) for p in fx["positions"])
    toks, rec = H.oracle_generate(m, prompt, 64, want=want)
    assert (toks == fx["tokens"]).all()
    for i, p in enumerate(fx["positions"]):
        lg, ly = rec[int(p)]
        assert (lg.view(np.uint32) == fx["logits"][i].view(np.uint32)).all()
        assert (ly.view(np.uint32) == fx["layer_hidden"][i].view(np.uint32)).all()
    m.close()

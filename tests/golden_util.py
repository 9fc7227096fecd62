"""Loader of the golden logits under tests/golden (written by tests/golden/make_hf_fp64_logits.py)."""
import hashlib
import json
import os

import numpy as np

from lumen_amd import synth

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = ("llama", "qwen3")


def load_case(name):
    """-> (cfg, params, ids, fp64 logits [n, V]) with the weights regenerated from the stored seed and
    checked against the stored digest."""
    with np.load(os.path.join(GOLDEN_DIR, f"hf_fp64_{name}.npz")) as z:
        cfg = json.loads(str(z["config"]))
        seed = int(z["seed"])
        ids = z["ids"].astype(np.int32)
        digest = str(z["params_sha256"])
        logits = z["logits"].astype(np.float64)
    params = synth.make_params(cfg, seed=seed, std=0.1, gains_one=False)
    h = hashlib.sha256()
    for pname in sorted(params):
        h.update(pname.encode())
        h.update(np.ascontiguousarray(params[pname], np.float32).tobytes())
    assert h.hexdigest() == digest, "the weight generator no longer reproduces the fixture's weights: regenerate it"
    return cfg, params, ids, logits

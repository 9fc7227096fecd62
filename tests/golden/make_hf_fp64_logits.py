"""Writes the golden logits of tests/golden/hf_fp64_*.npz.

The reference ships no tests, fixtures or golden vectors for its Llama forward, so the vectors here come
from an independent implementation of the same textbook model: a config-only (random-init, nothing
downloaded) Hugging Face LlamaForCausalLM / Qwen3ForCausalLM evaluated in fp64 on seeded weights and
token ids.  Each file holds the configuration (JSON), the seeds, the token ids, a SHA-256 of the
generated weights (so that a drift of the generator is told apart from a numerical regression) and the
fp64 logits of every position of one causal pass.

Run from the repository root:  python tests/golden/make_hf_fp64_logits.py
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
from lumen_amd import synth  # noqa: E402
from tests.test_oracle_model import TINY, TINY_QWEN, hf_model  # noqa: E402

# head_dim 16 and 32: sizes both the CPU checker and the GPU attention kernels take
LLAMA = dict(TINY, hidden_size=128)
CASES = {"llama": (LLAMA, 3, 20), "qwen3": (TINY_QWEN, 5, 24)}


def params_digest(params):
    h = hashlib.sha256()
    for name in sorted(params):
        h.update(name.encode())
        h.update(np.ascontiguousarray(params[name], np.float32).tobytes())
    return h.hexdigest()


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    for name, (cfg, seed, n) in CASES.items():
        params = synth.make_params(cfg, seed=seed, std=0.1, gains_one=False)
        ids = synth.make_tokens(n, cfg["vocab_size"], seed=seed)
        with torch.no_grad():
            logits = hf_model(cfg, params)(torch.from_numpy(ids.astype(np.int64))[None]).logits[0].numpy()
        np.savez_compressed(os.path.join(here, f"hf_fp64_{name}.npz"), config=json.dumps(cfg), seed=seed,
                            ids=ids.astype(np.int32), params_sha256=params_digest(params),
                            logits=logits.astype(np.float64))
        print(name, logits.shape, params_digest(params)[:16])


if __name__ == "__main__":
    main()

"""Writes sampler.npz by calling the reference's PIPELINE.sample_logits (CPU branch) in the build
container:   python tests/golden/make_sampler_goldens.py

For a list of seeded logit vectors and (temperature, top_p, top_k) settings it stores the token the
reference draws with numpy's global generator seeded per case; only seeds, settings and the
reference's outputs are stored.  The logits are drawn here with numpy PCG64 so the test can rebuild them.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF_SRC = "/root/reference/rwkv_pip_package/src"
sys.path.insert(0, REF_SRC)
from rwkv.utils import PIPELINE  # noqa: E402

CASES = [  # (vocab, logit scale, temperature, top_p, top_k)
    (211, 3.0, 1.0, 0.85, 0), (211, 3.0, 1.0, 0.5, 0), (211, 3.0, 0.7, 0.85, 0), (211, 3.0, 1.5, 0.3, 10),
    (211, 3.0, 0.0, 0.85, 0), (211, 3.0, 1.0, 0.0, 0), (211, 3.0, 1.0, 0.9999, 0), (211, 3.0, 1.0, 0.999, 5),
    (1000, 6.0, 1.0, 0.85, 0), (1000, 6.0, 1.2, 0.9, 50), (50277, 4.0, 1.0, 0.85, 0), (50277, 4.0, 0.8, 0.7, 100),
    (65536, 5.0, 1.0, 0.95, 0), (65536, 1.0, 1.0, 0.2, 0),
]
DRAWS = 8


def logits_for(case_index, vocab, scale):
    rng = np.random.Generator(np.random.PCG64([case_index, 0x5A11]))
    return (rng.standard_normal(vocab) * scale).astype(np.float32)


def main():
    tokens = np.zeros((len(CASES), DRAWS), dtype=np.int64)
    for ci, (V, scale, temp, top_p, top_k) in enumerate(CASES):
        x = torch.from_numpy(logits_for(ci, V, scale))
        for d in range(DRAWS):
            np.random.seed(1000 * ci + d)
            tokens[ci, d] = PIPELINE.sample_logits(None, x.clone(), temperature=temp, top_p=top_p, top_k=top_k)
    np.savez(os.path.join(HERE, "sampler.npz"), cases=np.array(CASES, dtype=np.float64), tokens=tokens, draws=DRAWS)
    print("wrote sampler.npz", tokens[:, :4])


if __name__ == "__main__":
    main()

"""Writes the RWKV-7 golden fixtures by running the reference's ``RWKV_x070`` on CPU.

Run in the build container only (the reference lives at /root/reference and never travels):
    python tests/golden/make_goldens_v7.py
    python tests/golden/make_goldens_v7.py --deep-embed

It imports ``rwkv.model`` from /root/reference/rwkv_pip_package/src with RWKV_V7_ON=1 and
RWKV_CUDA_ON=0 (pure-torch recurrence, no native build), feeds it a tiny synthetic checkpoint from
``chatrwkv_amd.synth.make_checkpoint_v7`` and stores the seeds plus the reference's outputs:

  e2e_v7_cpu_fp32.npz   'cpu fp32': logits with full_output over a 9-token prompt, logits of chunked
                        calls (sequence and one-token calls interleaved) and both final states
  e2e_v7_cpu_fp16.npz   the same under 'cpu fp16' (every tensor in half precision on the CPU), which
                        shows where the reference rounds to fp16
  e2e_v7_de_cpu_fp32.npz, e2e_v7_de_cpu_fp16.npz   (--deep-embed) the same for the DeepEmbed variant: the
                        reference is imported with RWKV_DE_VERSION=1 (it picks its forward functions when the class
                        is defined, model.py:304, 365, 424, 576), the checkpoint carries the ffn.s_* tensors
Only outputs and seeds are stored; no reference source is copied.
"""
import os
import sys
import tempfile

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
REF_SRC = "/root/reference/rwkv_pip_package/src"

from chatrwkv_amd import synth  # noqa: E402

TINY7 = dict(n_layer=3, n_embd=128, n_ffn=512, vocab=211, lora=(32, 32, 32, 64))
CKPT_SEED = 270
PROMPT_SEED = 11
CHUNKS = ((0, 2), (2, 3), (3, 7), (7, 8), (8, 9))


def main():
    de = "--deep-embed" in sys.argv[1:]
    if de:
        os.environ["RWKV_DE_VERSION"] = "1"
    os.environ["RWKV_V7_ON"] = "1"
    os.environ["RWKV_CUDA_ON"] = "0"
    os.environ["RWKV_JIT_ON"] = "1"
    sys.path.insert(0, REF_SRC)
    from rwkv.model import RWKV  # RWKV_x070 under RWKV_V7_ON=1 (model.py:1679-1680)

    ck = synth.make_checkpoint_v7(seed=CKPT_SEED + (1 if de else 0), deep_embed=de, **TINY7)
    toks = synth.random_tokens(9, TINY7["vocab"], seed=PROMPT_SEED)
    with tempfile.TemporaryDirectory() as tmp:
        stem = os.path.join(tmp, "tiny7")
        torch.save({k: v.clone() for k, v in ck.items()}, stem + ".pth")
        for strat in ("cpu fp32", "cpu fp16"):
            m = RWKV(stem, strat)
            full, st_full = m.forward(toks, None, full_output=True)
            outs, st = [], None
            for a, b in CHUNKS:
                o, st = m.forward(toks[a:b], st)
                outs.append(o.detach().float().cpu().numpy())
            d = {"tokens": np.array(toks), "full_logits": full.detach().float().cpu().numpy(),
                 "chunk_logits": np.stack(outs)}
            for tag, s in (("full", st_full), ("chunk", st)):
                for i, t in enumerate(s):
                    d[f"{tag}_state_{i}"] = t.detach().float().cpu().contiguous().numpy()
            name = f"e2e_v7_{'de_' if de else ''}{strat.replace(' ', '_')}.npz"
            np.savez_compressed(os.path.join(HERE, name), **d)
            print("wrote", name)


if __name__ == "__main__":
    main()

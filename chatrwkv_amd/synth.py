"""Synthetic RWKV checkpoints in the reference's on-disk layout.

The reference loads a flat ``{name: tensor}`` dict with ``torch.load``
(rwkv_pip_package/src/rwkv/model.py:642) and detects the architecture from
key names and shapes (model.py:658-680).  This module writes such dicts with
random-initialised weights so that every box (CPU container, GPU box) can
rebuild the same model from a seed instead of shipping weights.

Distributions: 2-D matrices (emb, head, key/value/receptance/gate/output)
N(0, 0.02); time_decay U[-6,-1]; time_first / time_faaaa U[-1,1];
time_mix_* / time_maa_* U[0,1]; LayerNorm / GroupNorm weight 1, bias 0;
RWKV-6 LoRA matrices N(0, 0.01).  ``make_checkpoint_v7`` writes RWKV-7 checkpoints (its own key set,
non-trivial LayerNorm / GroupNorm affines and LoRA matrices large enough to matter).

Two generators:
  * ``numpy`` (default): PCG64 streams keyed by (seed, crc32(tensor name)).
    Bit-stable across machines with the same numpy; used wherever the CPU
    oracle and the GPU path must see the same model.
  * ``torch`` on a device: ``torch.randn`` with a seeded device generator, for
    the 7B/14B shapes where the fp32 checkpoint is produced directly in HBM.
"""
import zlib
from collections import OrderedDict

import numpy as np
import torch

SHAPES = {
    # name: (version, n_layer, n_embd, n_ffn, vocab)
    "v4-169m": (4, 12, 768, 3072, 50277),
    "v4-7b": (4, 32, 4096, 16384, 50277),
    "v4-14b": (4, 40, 5120, 20480, 50277),
    "v6-7b": (6, 32, 4096, 14336, 65536),
    "v7-7b": (7, 32, 4096, 16384, 65536),
}


class _NumpyGen:
    def __init__(self, seed):
        self.seed = int(seed)

    def _rng(self, name):
        return np.random.Generator(np.random.PCG64([self.seed, zlib.crc32(name.encode())]))

    def normal(self, name, shape, std):
        a = self._rng(name).standard_normal(size=shape, dtype=np.float32) * np.float32(std)
        return torch.from_numpy(a)

    def uniform(self, name, shape, lo, hi):
        a = self._rng(name).random(size=shape, dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)
        return torch.from_numpy(a)

    def const(self, shape, v):
        return torch.full(shape, float(v), dtype=torch.float32)


class _TorchGen:
    def __init__(self, seed, device):
        self.device = torch.device(device)
        self.g = torch.Generator(device=self.device)
        self.g.manual_seed(int(seed))

    def normal(self, name, shape, std):
        return torch.randn(shape, generator=self.g, device=self.device, dtype=torch.float32) * std

    def uniform(self, name, shape, lo, hi):
        return torch.rand(shape, generator=self.g, device=self.device, dtype=torch.float32) * (hi - lo) + lo

    def const(self, shape, v):
        return torch.full(shape, float(v), dtype=torch.float32, device=self.device)


def make_checkpoint(version=4, n_layer=2, n_embd=64, n_ffn=None, vocab=97, seed=0,
                    head_size=64, lora_maa=32, lora_decay=64, device=None, n_att=None, affine=False,
                    time_state=False):
    """Return an OrderedDict checkpoint in the reference's raw (pre-conversion) layout.

    version: 4, 5 (v5.0), 5.1, 5.2 or 6.
    affine: LayerNorm / GroupNorm weights U[0.8, 1.2] and biases N(0, 0.05) instead of 1 / 0, so that
    every affine vector is told apart from every other one (parity tests); the benchmark shapes keep 1 / 0.
    time_state: RWKV-5/6 only, adds a trained initial state ``att.time_state`` [H, N, N] per block
    (model.py:1467-1468).
    Key order follows real checkpoints; for v6, ``time_maa_*`` precede
    ``time_faaaa`` inside a block because the reference's head-count
    detection depends on it (model.py:676-679).
    """
    C = int(n_embd)
    F = int(n_ffn) if n_ffn is not None else 4 * C
    V = int(vocab)
    A = int(n_att) if n_att is not None else C
    g = _NumpyGen(seed) if device is None else _TorchGen(seed, device)

    def ln(name, n):
        if affine:
            w[name + ".weight"] = g.uniform(name + ".weight", (n,), 0.8, 1.2)
            w[name + ".bias"] = g.normal(name + ".bias", (n,), 0.05)
        else:
            w[name + ".weight"] = g.const((n,), 1.0)
            w[name + ".bias"] = g.const((n,), 0.0)

    w = OrderedDict()
    w["emb.weight"] = g.normal("emb.weight", (V, C), 0.02)
    v5 = int(version) == 5
    v6 = int(version) == 6
    if v5 or v6:
        assert A % head_size == 0
        H = A // head_size
    for i in range(n_layer):
        b = f"blocks.{i}."
        for name in (("ln1", "ln2", "ln0") if i == 0 else ("ln1", "ln2")):
            ln(b + name, C)
        a = b + "att."
        if version == 4:
            w[a + "time_decay"] = g.uniform(a + "time_decay", (A,), -6.0, -1.0)
            w[a + "time_first"] = g.uniform(a + "time_first", (A,), -1.0, 1.0)
            for m in "kvr":
                w[a + "time_mix_" + m] = g.uniform(a + "time_mix_" + m, (1, 1, C), 0.0, 1.0)
        elif v5:
            for m in ("kvr" if version == 5 else "kvrg"):
                w[a + "time_mix_" + m] = g.uniform(a + "time_mix_" + m, (1, 1, C), 0.0, 1.0)
            if version == 5.2:
                w[a + "time_decay"] = g.uniform(a + "time_decay", (H, head_size), -6.0, -1.0)
                w[a + "time_faaaa"] = g.uniform(a + "time_faaaa", (H, head_size), -1.0, 1.0)
            else:
                w[a + "time_decay"] = g.uniform(a + "time_decay", (H,), -6.0, -1.0)
                w[a + "time_first"] = g.uniform(a + "time_first", (H,), -1.0, 1.0)
        else:
            for m in "xwkvrg":
                w[a + "time_maa_" + m] = g.uniform(a + "time_maa_" + m, (1, 1, C), 0.0, 1.0)
            w[a + "time_maa_w1"] = g.normal(a + "time_maa_w1", (C, 5 * lora_maa), 0.01)
            w[a + "time_maa_w2"] = g.normal(a + "time_maa_w2", (5, lora_maa, C), 0.01)
            w[a + "time_decay"] = g.uniform(a + "time_decay", (1, 1, A), -6.0, -1.0)
            w[a + "time_decay_w1"] = g.normal(a + "time_decay_w1", (C, lora_decay), 0.01)
            w[a + "time_decay_w2"] = g.normal(a + "time_decay_w2", (lora_decay, A), 0.01)
            w[a + "time_faaaa"] = g.uniform(a + "time_faaaa", (H, head_size), -1.0, 1.0)
        w[a + "key.weight"] = g.normal(a + "key.weight", (A, C), 0.02)
        w[a + "value.weight"] = g.normal(a + "value.weight", (A, C), 0.02)
        w[a + "receptance.weight"] = g.normal(a + "receptance.weight", (A, C), 0.02)
        if version in (5.1, 5.2) or v6:
            w[a + "gate.weight"] = g.normal(a + "gate.weight", (A, C), 0.02)
        w[a + "output.weight"] = g.normal(a + "output.weight", (C, A), 0.02)
        if v5 or v6:
            ln(a + "ln_x", A)
            if time_state:
                w[a + "time_state"] = g.normal(a + "time_state", (H, head_size, head_size), 0.3)
        f = b + "ffn."
        mixname = "time_maa_" if v6 else "time_mix_"
        for m in "kr":
            w[f + mixname + m] = g.uniform(f + mixname + m, (1, 1, C), 0.0, 1.0)
        w[f + "key.weight"] = g.normal(f + "key.weight", (F, C), 0.02)
        w[f + "receptance.weight"] = g.normal(f + "receptance.weight", (C, C), 0.02)
        w[f + "value.weight"] = g.normal(f + "value.weight", (C, F), 0.02)
    ln("ln_out", C)
    w["head.weight"] = g.normal("head.weight", (V, C), 0.02)
    return w


def v7_lora_dims(n_embd):
    """LoRA ranks (decay, in-context rate, value residual, gate) that released RWKV-7 checkpoints of
    width ``n_embd`` use: multiples of 32 growing with the width."""
    c = float(n_embd)
    r32 = lambda v: max(32, int(round(v / 32.0)) * 32)
    return r32(1.8 * c ** 0.5), r32(1.8 * c ** 0.5), r32(1.3 * c ** 0.5), r32(0.6 * c ** 0.8)


def make_checkpoint_v7(n_layer=2, n_embd=128, n_ffn=None, vocab=97, seed=0, head_size=64, lora=None, device=None,
                       deep_embed=False):
    """RWKV-7 checkpoint with the keys ``RWKV_x070.__init__`` reads (model.py:245-282) and the forward
    passes use (model.py:349-358): per block ``att.x_{r,w,k,v,a,g}``, ``att.{w,a,v}{0,1,2}``,
    ``att.g{1,2}``, ``att.k_k``, ``att.k_a``, ``att.r_k`` [H, N], the four square matrices, ``att.ln_x``,
    ``ffn.x_k`` and the two channel-mix matrices.  LoRA matrices are stored [in, rank] / [rank, out]
    and are not transposed by the loader.  ``lora`` = (decay, a, v, gate) ranks.
    ``deep_embed``: also the tensors of the DeepEmbed variant (RWKV_DE_VERSION=1, model.py:274-277, 578-594): per
    block ``ffn.s_emb.weight`` [V, 1024], ``ffn.s_emb_x.weight`` [1024, C], ``ffn.s1`` [C, 32], ``ffn.s2``
    [32, F] and ``ffn.s0`` [1, 1, F]."""
    C = int(n_embd)
    F = int(n_ffn) if n_ffn is not None else 4 * C
    V = int(vocab)
    H = C // head_size
    assert H * head_size == C
    dw, da, dv, dg = lora if lora is not None else v7_lora_dims(C)
    g = _NumpyGen(seed) if device is None else _TorchGen(seed, device)
    w = OrderedDict()
    w["emb.weight"] = g.normal("emb.weight", (V, C), 0.02)
    for i in range(n_layer):
        b = f"blocks.{i}."
        for ln in (("ln1", "ln2", "ln0") if i == 0 else ("ln1", "ln2")):
            w[b + ln + ".weight"] = g.uniform(b + ln + ".weight", (C,), 0.8, 1.2)
            w[b + ln + ".bias"] = g.normal(b + ln + ".bias", (C,), 0.05)
        a = b + "att."
        for m in "rwkvag":
            w[a + "x_" + m] = g.uniform(a + "x_" + m, (1, 1, C), 0.0, 1.0)
        w[a + "w0"] = g.uniform(a + "w0", (1, 1, C), -3.0, 2.0)
        w[a + "w1"] = g.normal(a + "w1", (C, dw), 0.1)
        w[a + "w2"] = g.normal(a + "w2", (dw, C), 0.2)
        w[a + "a0"] = g.uniform(a + "a0", (1, 1, C), -1.0, 1.0)
        w[a + "a1"] = g.normal(a + "a1", (C, da), 0.1)
        w[a + "a2"] = g.normal(a + "a2", (da, C), 0.2)
        w[a + "v0"] = g.uniform(a + "v0", (1, 1, C), -1.0, 1.0)
        w[a + "v1"] = g.normal(a + "v1", (C, dv), 0.1)
        w[a + "v2"] = g.normal(a + "v2", (dv, C), 0.2)
        w[a + "g1"] = g.normal(a + "g1", (C, dg), 0.1)
        w[a + "g2"] = g.normal(a + "g2", (dg, C), 0.2)
        w[a + "k_k"] = g.uniform(a + "k_k", (1, 1, C), 0.5, 1.5)
        w[a + "k_a"] = g.uniform(a + "k_a", (1, 1, C), 0.0, 1.0)
        w[a + "r_k"] = g.normal(a + "r_k", (H, head_size), 0.3)
        for name in ("receptance", "key", "value", "output"):
            w[a + name + ".weight"] = g.normal(a + name + ".weight", (C, C), 0.05)
        w[a + "ln_x.weight"] = g.uniform(a + "ln_x.weight", (C,), 0.8, 1.2)
        w[a + "ln_x.bias"] = g.normal(a + "ln_x.bias", (C,), 0.05)
        f = b + "ffn."
        w[f + "x_k"] = g.uniform(f + "x_k", (1, 1, C), 0.0, 1.0)
        w[f + "key.weight"] = g.normal(f + "key.weight", (F, C), 0.05)
        w[f + "value.weight"] = g.normal(f + "value.weight", (C, F), 0.05)
        if deep_embed:
            w[f + "s_emb.weight"] = g.normal(f + "s_emb.weight", (V, 1024), 0.3)
            w[f + "s_emb_x.weight"] = g.normal(f + "s_emb_x.weight", (1024, C), 0.03)
            w[f + "s1"] = g.normal(f + "s1", (C, 32), 0.1)
            w[f + "s2"] = g.normal(f + "s2", (32, F), 0.2)
            w[f + "s0"] = g.uniform(f + "s0", (1, 1, F), 0.5, 1.5)
    w["ln_out.weight"] = g.uniform("ln_out.weight", (C,), 0.8, 1.2)
    w["ln_out.bias"] = g.normal("ln_out.bias", (C,), 0.05)
    w["head.weight"] = g.normal("head.weight", (V, C), 0.05)
    return w


def make_named(name, seed=0, device=None, n_layer=None):
    """Checkpoint for one of the named shapes in ``SHAPES`` (optionally fewer layers)."""
    version, L, C, F, V = SHAPES[name]
    if version == 7:
        return make_checkpoint_v7(n_layer=L if n_layer is None else n_layer, n_embd=C, n_ffn=F, vocab=V,
                                  seed=seed, device=device)
    return make_checkpoint(version=version, n_layer=L if n_layer is None else n_layer, n_embd=C,
                           n_ffn=F, vocab=V, seed=seed, device=device)


def random_tokens(n, vocab, seed=0):
    """Uniform random token ids in [0, vocab) as a Python list of ints."""
    rng = np.random.Generator(np.random.PCG64([int(seed), 0x70C3]))
    return [int(t) for t in rng.integers(0, vocab, size=n)]

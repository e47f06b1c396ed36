"""Writes the golden fixtures in this folder by running the reference on CPU.

Run in the build container only (the reference lives at /root/reference and never
travels):   python tests/golden/make_goldens.py

It imports ``rwkv.model`` from /root/reference/rwkv_pip_package/src with
RWKV_CUDA_ON=0 (no native build), feeds it synthetic checkpoints from
``chatrwkv_amd.synth`` and stores inputs' seeds plus the reference's outputs:

  quant_v4_cpu_fp32i8.npz   converted weight dict of a tiny RWKV-4 under 'cpu fp32i8'
                            (uint8 matrices + fp32 mx/rx/my/ry; both quantizer branches)
  quant_v4_cuda_fp16i8.npz  dict saved by convert_and_save_and_exit under 'cuda fp16i8'
                            (fp16 scales, RESCALE_LAYER = 6, 8 layers so the rescale shows)
  e2e_<ver>_<strategy>.npz  logits (full_output over a 9-token prompt, then chunked calls
                            and one-token calls) and the final state, tiny models of
                            RWKV-4 / 5.0 / 5.1 / 5.2 / 6.0 under 'cpu fp32i8' and 'cpu fp32'
  e2e_<ver>_cpu_fp16.npz    the same runs under 'cpu fp16' (the reference's pure-torch functions on half
                            tensors, RESCALE_LAYER = 6): pins where the fp16 path rounds; and
  e2e_<ver>_l8_cpu_fp16.npz 8-layer RWKV-4 / RWKV-6 models (n_embd 64) under 'cpu fp16', deep enough for
                            the rescale (x / 2 after layer 6, matrices of layers >= 6 halved) to act
  e2e_<ver>_mixed_cpu.npz   RWKV-4 / RWKV-6 under 'cpu fp32i8 *2 -> cpu fp32': uint8 weights for two layers, float
                            weights for the third and the head
  e2e_<ver>_state_<strategy>.npz  RWKV-5.2 / RWKV-6 checkpoints that carry a trained initial state
                            (att.time_state, model.py:765-768, 1467-1468) under 'cpu fp32' and 'cpu fp16'
  planner.json              the per-slot plan the reference prints for a list of strategy strings
  e2e_v4_169m_cpu_fp32i8.npz  the 169M-shape model: 128-token prefill + 32 greedy steps;
                            argmax per position, 256 fixed logits per position, state sums
Only outputs and seeds are stored; no reference source is copied.
"""
import os
import subprocess
import sys
import tempfile

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
REF_SRC = "/root/reference/rwkv_pip_package/src"

from chatrwkv_amd import synth  # noqa: E402

# affine=True: random LayerNorm / GroupNorm weights and biases, so a swapped, dropped or mis-indexed affine
# vector shows in every fixture below
TINY = dict(n_layer=3, n_embd=128, n_ffn=512, vocab=211, affine=True)
TINY8 = dict(n_layer=8, n_embd=64, n_ffn=256, vocab=100, affine=True)
PROMPT_SEED = 11


def _ref():
    os.environ["RWKV_CUDA_ON"] = "0"
    sys.path.insert(0, REF_SRC)
    from rwkv.model import RWKV
    return RWKV


def _save_ckpt(ck, path):
    torch.save({k: v.clone() for k, v in ck.items()}, path)


def _dump_w(w):
    out = {}
    for k, v in w.items():
        if isinstance(v, torch.Tensor):
            v = v.detach().cpu()
            out[k] = v.contiguous().numpy()
    return out


def quant_cpu(tmp):
    RWKV = _ref()
    ck = synth.make_checkpoint(version=4, seed=101, **TINY)
    p = os.path.join(tmp, "tiny4.pth")
    _save_ckpt(ck, p)
    m = RWKV(p, "cpu fp32i8", verbose=False)
    np.savez_compressed(os.path.join(HERE, "quant_v4_cpu_fp32i8.npz"), **_dump_w(m.w))


def quant_cuda_convert(tmp):
    ck = synth.make_checkpoint(version=4, seed=102, **TINY8)
    p = os.path.join(tmp, "tiny8.pth")
    outp = os.path.join(tmp, "tiny8_conv.pth")
    _save_ckpt(ck, p)
    code = (
        "import os, sys\n"
        "os.environ['RWKV_CUDA_ON']='0'\n"
        f"sys.path.insert(0, {REF_SRC!r})\n"
        "from rwkv.model import RWKV\n"
        f"RWKV({p!r}, 'cuda fp16i8', verbose=False, convert_and_save_and_exit={outp!r})\n"
    )
    subprocess.run([sys.executable, "-c", code], check=True)
    w = torch.load(outp, map_location="cpu", weights_only=True)
    meta = {k: w[k] for k in ("_strategy", "_version", "_rescale_layer")}
    d = _dump_w(w)
    d["meta_strategy"] = np.array(str(meta["_strategy"]))
    d["meta_version"] = np.array(str(meta["_version"]))
    d["meta_rescale_layer"] = np.array(int(meta["_rescale_layer"]))
    np.savez_compressed(os.path.join(HERE, "quant_v4_cuda_fp16i8.npz"), **d)


def _state_np(state):
    return {f"state_{i}": s.detach().float().cpu().contiguous().numpy() for i, s in enumerate(state)}


MIXED = "cpu fp32i8 *2 -> cpu fp32"


def e2e_mixed(tmp):
    """A chain of weight types on one device: uint8 for the first two layers, float for the third and the head."""
    RWKV = _ref()
    for ver, tag in ((4, "v4"), (6, "v6_0")):
        ck = synth.make_checkpoint(version=ver, seed=200 + int(ver * 10), **TINY)
        p = os.path.join(tmp, f"mixed_{tag}.pth")
        _save_ckpt(ck, p)
        toks = synth.random_tokens(9, TINY["vocab"], seed=PROMPT_SEED)
        m = RWKV(p, MIXED, verbose=False)
        kinds = [str(m.w[f"blocks.{i}.att.key.weight"].dtype) for i in range(TINY["n_layer"])] + [str(m.w["head.weight"].dtype)]
        full, st_full = m.forward(toks, None, full_output=True)
        outs, st = [], None
        for a, b in ((0, 2), (2, 3), (3, 7), (7, 8), (8, 9)):
            o, st = m.forward(toks[a:b], st)
            outs.append(o.detach().float().cpu().numpy())
        d = {"tokens": np.array(toks), "full_logits": full.detach().float().cpu().numpy(), "chunk_logits": np.stack(outs),
             "weight_kinds": np.array(kinds)}
        d.update({"chunk_" + k: v for k, v in _state_np(st).items()})
        name = f"e2e_{tag}_mixed_cpu.npz"
        np.savez_compressed(os.path.join(HERE, name), **d)
        print("wrote", name, kinds)


def e2e_deep_fp16(tmp):
    RWKV = _ref()
    for ver, tag in ((4, "v4"), (6, "v6_0")):
        ck = synth.make_checkpoint(version=ver, seed=300 + int(ver * 10), **TINY8)
        p = os.path.join(tmp, f"deep_{tag}.pth")
        _save_ckpt(ck, p)
        toks = synth.random_tokens(9, TINY8["vocab"], seed=PROMPT_SEED)
        m = RWKV(p, "cpu fp16", verbose=False)
        assert m.RESCALE_LAYER == 6
        full, st_full = m.forward(toks, None, full_output=True)
        outs, st = [], None
        for a, b in ((0, 2), (2, 3), (3, 7), (7, 8), (8, 9)):
            o, st = m.forward(toks[a:b], st)
            outs.append(o.detach().float().cpu().numpy())
        d = {"tokens": np.array(toks), "full_logits": full.detach().float().cpu().numpy(), "chunk_logits": np.stack(outs)}
        d.update({"full_" + k: v for k, v in _state_np(st_full).items()})
        d.update({"chunk_" + k: v for k, v in _state_np(st).items()})
        name = f"e2e_{tag}_l8_cpu_fp16.npz"
        np.savez_compressed(os.path.join(HERE, name), **d)
        print("wrote", name)


def e2e_tiny(tmp, which_strats=None):
    RWKV = _ref()
    for ver, tag in ((4, "v4"), (5, "v5_0"), (5.1, "v5_1"), (5.2, "v5_2"), (6, "v6_0")):
        ck = synth.make_checkpoint(version=ver, seed=200 + int(ver * 10), **TINY)
        p = os.path.join(tmp, f"tiny_{tag}.pth")
        _save_ckpt(ck, p)
        toks = synth.random_tokens(9, TINY["vocab"], seed=PROMPT_SEED)
        for strat in ("cpu fp32i8", "cpu fp32", "cpu fp16"):
            if which_strats and strat not in which_strats:
                continue
            m = RWKV(p, strat, verbose=False)
            full, st_full = m.forward(toks, None, full_output=True)
            # chunked: [0:2] seq, [2:3] one, [3:7] seq, [7:8] one, [8:9] one
            outs = []
            st = None
            for a, b in ((0, 2), (2, 3), (3, 7), (7, 8), (8, 9)):
                o, st = m.forward(toks[a:b], st)
                outs.append(o.detach().float().cpu().numpy())
            d = {"tokens": np.array(toks), "full_logits": full.detach().float().cpu().numpy(),
                 "chunk_logits": np.stack(outs)}
            d.update({"full_" + k: v for k, v in _state_np(st_full).items()})
            d.update({"chunk_" + k: v for k, v in _state_np(st).items()})
            name = f"e2e_{tag}_{strat.replace(' ', '_')}.npz"
            np.savez_compressed(os.path.join(HERE, name), **d)
            print("wrote", name, "version", m.version)


def e2e_time_state(tmp):
    """Checkpoints with att.time_state: forward(tokens, None) starts from it (transposed) instead of zeros."""
    RWKV = _ref()
    for ver, tag in ((5.2, "v5_2"), (6, "v6_0")):
        ck = synth.make_checkpoint(version=ver, seed=500 + int(ver * 10), time_state=True, **TINY)
        p = os.path.join(tmp, f"ts_{tag}.pth")
        _save_ckpt(ck, p)
        toks = synth.random_tokens(9, TINY["vocab"], seed=PROMPT_SEED)
        for strat in ("cpu fp32", "cpu fp16"):
            m = RWKV(p, strat, verbose=False)
            assert m.args.time_state
            full, st_full = m.forward(toks, None, full_output=True)
            outs, st = [], None
            for a, b in ((0, 1), (1, 4), (4, 5), (5, 9)):
                o, st = m.forward(toks[a:b], st)
                outs.append(o.detach().float().cpu().numpy())
            d = {"tokens": np.array(toks), "full_logits": full.detach().float().cpu().numpy(),
                 "chunk_logits": np.stack(outs)}
            d.update({"full_" + k: v for k, v in _state_np(st_full).items()})
            d.update({"chunk_" + k: v for k, v in _state_np(st).items()})
            name = f"e2e_{tag}_state_{strat.replace(' ', '_')}.npz"
            np.savez_compressed(os.path.join(HERE, name), **d)
            print("wrote", name)


def e2e_169m(tmp):
    RWKV = _ref()
    ck = synth.make_named("v4-169m", seed=0)
    p = os.path.join(tmp, "v4_169m.pth")
    _save_ckpt(ck, p)
    del ck
    V = synth.SHAPES["v4-169m"][4]
    toks = synth.random_tokens(128, V, seed=0)
    m = RWKV(p, "cpu fp32i8", verbose=False)
    idx = np.sort(np.random.Generator(np.random.PCG64(7)).choice(V, size=256, replace=False))
    full, st = m.forward(toks, None, full_output=True)
    full = full.detach().cpu().numpy()
    argmax = list(full.argmax(axis=-1))
    subset = [full[:, idx]]
    top2gap = [np.sort(full, axis=-1)[:, -1] - np.sort(full, axis=-1)[:, -2]]
    nxt = int(argmax[-1])
    gen = []
    for _ in range(32):
        gen.append(nxt)
        o, st = m.forward([nxt], st)
        o = o.detach().cpu().numpy()
        argmax.append(int(o.argmax()))
        subset.append(o[None, idx])
        so = np.sort(o)
        top2gap.append(np.array([so[-1] - so[-2]]))
        nxt = int(o.argmax())
    d = {"tokens": np.array(toks), "generated": np.array(gen), "argmax": np.array(argmax),
         "logit_index": idx, "logit_subset": np.concatenate(subset).astype(np.float32),
         "top2gap": np.concatenate(top2gap).astype(np.float32)}
    for i, s in enumerate(st):
        s = s.detach().cpu().numpy().astype(np.float64)
        d[f"state_sum_{i}"] = np.array([s.sum(), np.abs(s).sum()])
        d[f"state_head_{i}"] = s[:8].astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "e2e_v4_169m_cpu_fp32i8.npz"), **d)
    print("wrote e2e_v4_169m_cpu_fp32i8.npz")


PLAN_STRATEGIES = [
    "cuda fp16i8", "cuda fp16", "cpu fp32i8", "cpu fp32", "cuda:0 fp16i8", "cuda fp16i8 *10 -> cuda fp16",
    "cuda fp16 *10+", "cuda:0 fp16 *20 -> cuda:1 fp16", "cuda fp16i8 *1 -> cuda fp16", "cuda fp16i8 -> cpu fp32 *1",
    "cuda fp16 *0+ -> cpu fp32 *1", "cuda fp16i8 *4 -> cuda fp16 *3 -> cpu fp32", "cuda fp16 *6+",
    "cuda fp16i8 *2 -> cuda fp16 *2+ -> cpu fp32 *1", "cuda fp16 -> cuda:1 fp16", "cpu bf16", "cuda fp16i8 *100",
    "cuda fp16 *3 -> cuda:1 fp16 *3 -> cpu fp32",
    "cuda fp16 *3 -> cuda fp16i8", "cuda fp16i8 *2 -> cuda fp16 *3 -> cuda fp16i8", "cuda fp16i8 -> cuda fp16",
    "cuda fp16i8 *2 -> cuda fp16 -> cuda fp16i8 *1", "cuda fp16i8 *9 -> cuda fp16", "cuda:0 fp16i8 *5 -> cuda fp16",
]


def planner(tmp):
    """The per-slot plan the reference prints (model.py:726-750) for a list of strategy strings,
    on an 8-layer model.  The loader later fails where it moves tensors to a GPU that is not there;
    the plan is printed before that."""
    ck = synth.make_checkpoint(version=4, seed=102, **TINY8)
    p = os.path.join(tmp, "tiny8p.pth")
    _save_ckpt(ck, p)
    out = {}
    for strat in PLAN_STRATEGIES:
        code = (
            "import os, sys\n"
            "os.environ['RWKV_CUDA_ON']='0'\n"
            f"sys.path.insert(0, {REF_SRC!r})\n"
            "from rwkv.model import RWKV\n"
            f"RWKV({p!r}, {strat!r}, verbose=True)\n"
        )
        r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
        line = [l for l in r.stdout.splitlines() if l.startswith("0-")]
        out[strat] = line[0].strip() if line else "ERROR"
    import json
    with open(os.path.join(HERE, "planner.json"), "w") as f:
        json.dump({"n_layer": TINY8["n_layer"], "plans": out}, f, indent=1)
    print("wrote planner.json")


if __name__ == "__main__":
    torch.manual_seed(0)
    with tempfile.TemporaryDirectory() as tmp:
        which = sys.argv[1:] or ["quant_cpu", "quant_cuda", "tiny", "fp16", "mixed", "state", "169m", "planner"]
        if "planner" in which:
            planner(tmp)
        if "fp16" in which and "tiny" not in which:
            e2e_tiny(tmp, which_strats=("cpu fp16",))   # only the half-precision files
        if "fp16" in which:
            e2e_deep_fp16(tmp)
        if "mixed" in which:
            e2e_mixed(tmp)
        if "quant_cpu" in which:
            quant_cpu(tmp)
        if "quant_cuda" in which:
            quant_cuda_convert(tmp)
        if "tiny" in which:
            e2e_tiny(tmp)
        if "state" in which:
            e2e_time_state(tmp)
        if "169m" in which:
            e2e_169m(tmp)

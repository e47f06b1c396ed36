"""Strategy strings: validation and the per-layer plan.

Restates the planner of RWKV.__init__ (rwkv_pip_package/src/rwkv/model.py:620-750): a
strategy is a chain of segments ``device dtype[i8] [*N | *N+]`` joined by ``->``; the
n_layer + 1 slots (the last one holds ln_out + head, model.py:776-778) are dealt to the
segments in order.  This package then runs only plans that put every slot on one ROCm
GPU with fp16 activations and uint8 or fp16 weights: 'cuda fp16i8', 'cuda fp16', chains of the
two on the same GPU such as 'cuda fp16i8 *20 -> cuda fp16' (uint8 weights for the first 20 layers,
fp16 for the rest and the head), and streamed segments ('cuda fp16i8 *10+': the big matrices of the layers
after the first 10 stay in pinned host memory and are copied to the GPU for every call, model.py:854-858,
1526-1530).  Any other valid strategy raises NotImplementedError, an invalid string raises ValueError as the
reference does (model.py:621-622).
"""
import re
import types

import torch

# same language as model.py:620
STRATEGY_REGEX = re.compile(
    r"^(?:(?:^|->) *(?:cuda(?::[\d]+)?|cpu|mps|dml) (?:fp(?:16|32)|bf16)(?:i8|i4|i3)?(?: \*[\d]+\+?)? *)+$")

_DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


def normalize(strategy):
    """Canonical spelling stored in args.strategy_string and in converted checkpoints (model.py:624)."""
    if not STRATEGY_REGEX.match(strategy):
        raise ValueError("Invalid strategy. Please read https://pypi.org/project/rwkv/")
    return " -> ".join(seg.strip() for seg in strategy.split("->"))


def plan(strategy, n_layer):
    """Return the list of n_layer + 1 slot descriptors (device, atype, wtype, stream)."""
    strategy = normalize(strategy)
    segs = []
    for seg in strategy.split("->"):
        parts = seg.strip().split(" ")
        dt = parts[1]
        atype = _DTYPES[dt[:4]]
        wtype = torch.uint8 if dt.endswith("i8") else atype
        segs.append(dict(device=parts[0], atype=atype, wtype=wtype, spec=parts[2] if len(parts) > 2 else None))

    slots = n_layer + 1
    counts = [0] * len(segs)
    stream_seg, dealt, open_segs = -1, 0, 0
    for i, s in enumerate(segs):
        if s["spec"] is None:
            open_segs += 1
            continue
        spec = s["spec"]
        if spec.endswith("+"):
            counts[i] = int(spec[1:-1])
            stream_seg = i
        else:
            counts[i] = int(spec[1:])
        dealt += counts[i]
        if dealt >= slots:  # this segment takes what is left; later segments get nothing
            counts[i] += slots - dealt
            break
    streamed = 0
    if stream_seg < 0:
        if open_segs > 0 and slots > dealt:
            for i in range(len(segs)):
                if counts[i] == 0:
                    counts[i] = (slots - dealt) // open_segs
                    dealt += counts[i]
                    open_segs -= 1
        if slots > dealt:
            counts[-1] += slots - dealt
    elif slots > dealt:
        streamed = slots - dealt
        counts[stream_seg] += streamed

    ends, run = [], 0
    for c in counts:
        run += c
        ends.append(run)
    out = []
    for n in range(slots):
        for i, s in enumerate(segs):
            if n < ends[i]:
                out.append(types.SimpleNamespace(
                    device=s["device"], atype=s["atype"], wtype=s["wtype"],
                    stream=(i == stream_seg and n >= ends[i] - streamed)))
                break
        else:
            out.append(None)
    return out


def require_single_gpu(slots):
    """Check that a plan is one this package runs; return the weight type: 'u8', 'f16', or 'mixed' when
    the slots differ (then each layer, and the head, has the type of its own slot)."""
    kinds = set()
    for s in slots:
        if s is None:
            raise NotImplementedError("strategy leaves layers unassigned")
        if not str(s.device).startswith("cuda"):
            raise NotImplementedError(
                "chatrwkv_amd runs single-GPU strategies only ('cuda fp16i8', 'cuda fp16', chains of the two, "
                f"streamed or not); got device {s.device!r}")
        if s.device not in ("cuda", "cuda:0"):
            raise NotImplementedError("chatrwkv_amd uses GPU 0 only")
        if s.atype != torch.float16 or s.wtype not in (torch.uint8, torch.float16):
            raise NotImplementedError("supported strategies: 'cuda fp16i8', 'cuda fp16' and chains of the two")
        kinds.add("u8" if s.wtype == torch.uint8 else "f16")
    return kinds.pop() if len(kinds) == 1 else "mixed"

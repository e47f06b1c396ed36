"""Strategy planner against the plans the reference prints (tests/golden/planner.json)."""
import json
import os

import pytest

from chatrwkv_amd import strategy

G = os.path.join(os.path.dirname(__file__), "golden")


def _fmt(slots):
    return " ".join(
        f"{n}-{s.device}-{str(s.atype).replace('torch.', '')}-{str(s.wtype).replace('torch.', '')}"
        f"{'-stream' if s.stream else ''}" for n, s in enumerate(slots))


def test_plans_match_reference():
    gold = json.load(open(os.path.join(G, "planner.json")))
    assert len(gold["plans"]) >= 15
    for strat, line in gold["plans"].items():
        assert line != "ERROR", strat
        assert _fmt(strategy.plan(strat, gold["n_layer"])) == line, strat


@pytest.mark.parametrize("bad", ["", "gpu fp16", "cuda fp8", "cuda fp16i8 ->", "cuda  fp16", "cuda fp16 * 3", "fp16 cuda"])
def test_invalid_strategy_raises_value_error(bad):
    with pytest.raises(ValueError):
        strategy.plan(bad, 4)


def test_only_single_gpu_plans_are_accepted():
    assert strategy.require_single_gpu(strategy.plan("cuda fp16i8", 4)) == "u8"
    assert strategy.require_single_gpu(strategy.plan("cuda:0 fp16", 4)) == "f16"
    assert strategy.require_single_gpu(strategy.plan("cuda fp16i8 *100", 4)) == "u8"
    # chains of the two weight types on the one GPU
    assert strategy.require_single_gpu(strategy.plan("cuda fp16i8 *1 -> cuda fp16", 4)) == "mixed"
    assert strategy.require_single_gpu(strategy.plan("cuda:0 fp16 *2 -> cuda fp16i8", 4)) == "mixed"
    assert strategy.require_single_gpu(strategy.plan("cuda fp16i8 *9 -> cuda fp16", 4)) == "u8"   # the first segment takes all
    # streamed segments on the one GPU: the slots after the first two stream (the head slot among them)
    slots = strategy.plan("cuda fp16 *2+", 4)
    assert strategy.require_single_gpu(slots) == "f16" and [s.stream for s in slots] == [False, False, True, True, True]
    assert strategy.require_single_gpu(strategy.plan("cuda fp16i8 *1 -> cuda fp16 *1+", 4)) == "mixed"
    for s in ("cpu fp32", "cpu fp32i8", "cuda fp32", "cuda bf16", "cuda fp16i8 -> cpu fp32 *1", "cuda fp16 *2+ -> cpu fp32 *1",
              "cuda fp16 -> cuda:1 fp16", "cuda:1 fp16", "cuda fp16i8 *1 -> cuda fp32"):
        with pytest.raises(NotImplementedError):
            strategy.require_single_gpu(strategy.plan(s, 4))


def test_normalize_spelling():
    assert strategy.normalize("cuda fp16i8 *2->cpu fp32") == "cuda fp16i8 *2 -> cpu fp32"


def test_oracle_planner_matches_reference():
    """The oracle's own restatement of the slot allocation (used for chains of weight types on one device)
    against the same golden plans."""
    from oracle.model import plan_wtypes
    gold = json.load(open(os.path.join(G, "planner.json")))
    n = 0
    for strat, line in gold["plans"].items():
        try:
            dev, at, kinds = plan_wtypes(strat, gold["n_layer"])
        except ValueError:
            continue                      # second device, streaming, bf16: not emulated
        ref = [tok.split("-") for tok in line.split()]
        assert [r[3] == "uint8" for r in ref] == kinds, strat
        assert all(r[1].replace(":0", "") == dev for r in ref), strat
        n += 1
    assert n >= 14

"""The C-ABI library loads without a GPU and exports every symbol include/rwkv_hip.h declares;
the ctypes table covers them all; the product path refuses to run without a GPU."""
import os
import re

import pytest

from chatrwkv_amd import lib, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(headers=("rwkv_hip.h", "rwkv_hip_bench.h")):
    names = set()
    for h in headers:
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(rwkv_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_measurement_aids_are_not_in_the_product_header():
    product = _declared(("rwkv_hip.h",))
    assert not [n for n in product if "profile" in n or "time_" in n]
    assert set(_declared(("rwkv_hip_bench.h",))) == {"rwkv_v4_profile_one", "rwkv_v4_time_phase", "rwkv_mm8_seq_time_kernel"}


def test_header_symbols_exported_and_bound():
    if not os.path.exists(lib.LIB_PATH):
        from chatrwkv_amd import build
        build.build(verbose=False)
    L = lib.load()
    names = _declared()
    assert len(names) >= 15
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/rwkv_hip.h but not exported"
        assert n in lib.SIGNATURES, f"{n} has no ctypes signature in chatrwkv_amd/lib.py"
    for n in lib.SIGNATURES:
        assert n in names, f"{n} bound in lib.py but not declared in the header"
    assert L.rwkv_abi_version() == 3


def test_argument_validation_without_gpu():
    """Rejected arguments return negative codes before anything is launched."""
    L = lib.load()
    assert L.rwkv_mm8_one_f16(4096, 4096, None, None, 1, 4096, None, None, None, None, None, 0, None) == -3
    assert L.rwkv_mm8_seq_workspace(0, 4096) == 0
    assert L.rwkv_mm8_seq_workspace(4, 64) >= 4 * 64 * 2 + 32
    with pytest.raises(lib.RwkvHipError):
        lib.check(-2, "x")


def test_product_fails_loudly_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from chatrwkv_amd.model import RWKV
    ck = synth.make_checkpoint(version=4, n_layer=1, n_embd=64, n_ffn=256, vocab=50, seed=0)
    with pytest.raises(lib.RwkvHipError):
        RWKV(ck, "cuda fp16i8", verbose=False)
    from chatrwkv_amd import ops
    with pytest.raises(lib.RwkvHipError):
        ops.cuda_mm8_one(64, 64, torch.zeros(64, dtype=torch.float16), torch.zeros((64, 64), dtype=torch.uint8),
                         *(torch.zeros(s, dtype=torch.float16) for s in ((64,), (64,), (64, 1), (64, 1))))


def test_product_does_not_import_oracle():
    pkg = os.path.join(ROOT, "chatrwkv_amd")
    for fn in os.listdir(pkg):
        if fn.endswith(".py"):
            src = open(os.path.join(pkg, fn)).read()
            assert not re.search(r"^\s*(from|import)\s+oracle\b", src, flags=re.M), fn

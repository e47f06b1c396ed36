"""The reference-side binding printed in the integration guide at the repository root, executed as it stands: the python block that replaces the
reference's JIT-loaded ops (model.py:29-86) is taken out of the document, pointed at the built library, and its
three wrappers are checked against the fp64 / oracle results the operator tests use.  A signature in the document
that drifts from include/rwkv_hip.h fails here."""
import os
import re

import numpy as np
import pytest
import torch

from chatrwkv_amd import lib as _lib
from oracle import ops as oops
from oracle import quant as oquant

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"


def _binding():
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    src = next(b for b in blocks if "def cuda_mm8_one" in b and "def cuda_wkv" in b)
    assert "ctypes.CDLL('librwkv_hip.so')" in src
    src = src.replace("ctypes.CDLL('librwkv_hip.so')", f"ctypes.CDLL({_lib.LIB_PATH!r})")
    ns = {}
    exec(compile(src, "<documented binding>", "exec"), ns)
    return ns


def test_documented_binding_runs_and_agrees():
    ns = _binding()
    rng = np.random.default_rng(17)
    N, M, B = 768, 3072, 37
    w = (rng.standard_normal((N, M)) * 0.02).astype(np.float32)
    q, mx, rx, my, ry = oquant.quantize_u8(w, atype=np.float16)
    x = rng.standard_normal((B, N)).astype(np.float16)
    ref = x.astype(np.float64) @ oquant.dequant_f64(q, mx, rx, my, ry)
    # the document's load-time note: matrices input-contiguous, shape [in, out], strides (1, in)
    qd = torch.from_numpy(np.ascontiguousarray(q.T)).to(DEV).t()
    assert qd.shape == (N, M) and qd.stride() == (1, N)
    dmx, drx, dmy, dry = (torch.from_numpy(a).to(DEV) for a in (mx, rx, my, ry))
    xt = torch.from_numpy(x).to(DEV)
    scale = np.sqrt(np.mean(ref ** 2))
    tol = 1e-3 * scale + np.abs(ref).max() * 2 ** -10
    y1 = ns["cuda_mm8_one"](N, M, xt[0].contiguous(), qd, dmx, drx, dmy, dry)
    assert y1.dtype == torch.float16 and tuple(y1.shape) == (M,)
    assert np.abs(y1.cpu().numpy().astype(np.float64) - ref[0]).max() <= tol
    ys = ns["cuda_mm8_seq"](B, N, M, xt, qd, dmx, drx, dmy, dry)
    assert ys.dtype == torch.float16 and tuple(ys.shape) == (B, M)
    assert np.abs(ys.cpu().numpy().astype(np.float64) - ref).max() <= tol
    # the reference's own device layout (model.py:860: contiguous [in, out]): the binding repacks it once per tensor
    q_ref = torch.from_numpy(q).to(DEV)
    assert q_ref.stride() == (M, 1)
    assert torch.equal(ns["cuda_mm8_seq"](B, N, M, xt, q_ref, dmx, drx, dmy, dry), ys)
    assert torch.equal(ns["cuda_mm8_one"](N, M, xt[0].contiguous(), q_ref, dmx, drx, dmy, dry), y1)
    assert len(ns["_kept"]) == 1
    T, C = 19, 256
    k = rng.standard_normal((T, C)).astype(np.float32)
    v = rng.standard_normal((T, C)).astype(np.float32)
    wd = -np.exp(rng.uniform(-6, -1, C)).astype(np.float32)
    u = rng.uniform(-1, 1, C).astype(np.float32)
    a0, b0, p0 = np.zeros(C, np.float32), np.zeros(C, np.float32), np.full(C, -1e30, np.float32)
    y_ref, a_ref, b_ref, p_ref = oops.wkv4(k, v, u, wd, a0, b0, p0)
    ta, tb, tp = (torch.from_numpy(t.copy()).to(DEV) for t in (a0, b0, p0))
    y, _, _, _ = ns["cuda_wkv"](T, C, torch.from_numpy(wd).to(DEV), torch.from_numpy(u).to(DEV),
                                torch.from_numpy(k).to(DEV), torch.from_numpy(v).to(DEV), ta, tb, tp)
    torch.cuda.synchronize()
    np.testing.assert_allclose(y.cpu().numpy(), y_ref, rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(ta.cpu().numpy(), a_ref, rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(tp.cpu().numpy(), p_ref, rtol=1e-5, atol=1e-5)

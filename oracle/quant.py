"""Oracle: the reference's uint8 weight quantizer and its dequantisation.

Test infrastructure only (see oracle/__init__.py).

Follows rwkv_pip_package/src/rwkv/model.py:818-847 (quantizer) and
model.py:91-97 (dequantisation used by torch_mm8_seq / torch_mm8_one).
All arithmetic is IEEE fp32 in the reference's order, so the result is
bit-determined; tests/golden/quant_*.npz (written by the reference's own
loader) pin it.
"""
import numpy as np

f32 = np.float32


def quantize_u8(w, atype=np.float32):
    """Quantize the logical [N(in), M(out)] fp32 matrix ``w``.

    Returns (u8 [N,M], mx [M], rx [M], my [N,1], ry [N,1]); the four vectors are
    cast to ``atype`` and rx, ry are the stored ones (already divided by 16).

    model.py:824-832 (N > M): row minimum first, then column minimum;
    model.py:833-841 (N <= M): column minimum first, then row minimum;
    both then divide by the column maximum and by the row maximum.
    model.py:843: u8 = clip(floor(w * 256), 0, 255).  model.py:844-847: casts.
    """
    w = np.array(w, dtype=f32, copy=True)
    assert w.ndim == 2
    N, M = w.shape
    if N > M:
        my = w.min(axis=1, keepdims=True)
        w = w - my
        mx = w.min(axis=0)
        w = w - mx
    else:
        mx = w.min(axis=0)
        w = w - mx
        my = w.min(axis=1, keepdims=True)
        w = w - my
    rx = w.max(axis=0)
    w = w / rx
    ry = w.max(axis=1, keepdims=True)
    w = w / ry
    assert w.dtype == f32
    q = np.clip(np.floor(w * f32(256)), 0, 255).astype(np.uint8)
    return (q,
            mx.astype(atype),
            (rx / f32(16)).astype(atype),
            my.astype(atype),
            (ry / f32(16)).astype(atype))


def dequant(q, mx, rx, my, ry, dtype=np.float32):
    """W' = (q + 0.5) * ry * rx + my + mx evaluated in ``dtype`` left to right (model.py:93)."""
    d = dtype
    return (q.astype(d) + d(0.5)) * ry.astype(d) * rx.astype(d) + my.astype(d) + mx.astype(d)


def dequant_f64(q, mx, rx, my, ry):
    """Exact value of the stored representation, in fp64 (for error analysis)."""
    return dequant(q, mx, rx, my, ry, dtype=np.float64)

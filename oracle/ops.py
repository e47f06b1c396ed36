"""Oracle: per-op arithmetic of the RWKV inference path, in numpy.

Test infrastructure only (see oracle/__init__.py).

Every function takes and returns numpy arrays.  Activations are 2-D ``[T, C]``
(one-token mode is T == 1).  ``atype`` is the activation dtype of the strategy
(np.float32 for 'cpu fp32i8' / 'cpu fp32', np.float16 for the emulation of
'cuda fp16i8' / 'cuda fp16').  Where the reference's GPU path rounds to fp16 the
same rounding is applied here (rounding points: model.py:86 and
cuda/operators.cu:138 for mm8; model.py:1041-1042, 1048, 1359 for WKV-4;
model.py:1281-1298, 1379-1390 for RWKV-5/6; cuda/gemm_fp16_cublas.cpp:31-33 for
the fp16 GEMM whose fp32 output is not rounded through fp16).
"""
import numpy as np

from . import quant

f16, f32, f64 = np.float16, np.float32, np.float64


# ----------------------------------------------------------------------------- norms / gates

def layer_norm(x, w, b, eps=1e-5):
    """F.layer_norm over the last axis (model.py:985, 1035, 1668).  Statistics in
    high precision, affine applied before the single rounding to x.dtype."""
    if x.ndim == 2 and x.shape[0] > 4096:             # a whole embedding table: row blocks that stay in cache
        out = np.empty_like(x)
        for r in range(0, x.shape[0], 2048):
            out[r:r + 2048] = layer_norm(x[r:r + 2048], w, b, eps)
        return out
    x64 = x.astype(f64)
    mu = x64.mean(axis=-1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(axis=-1, keepdims=True)
    y = (x64 - mu) / np.sqrt(var + eps) * w.astype(f64) + b.astype(f64)
    return y.astype(x.dtype)


def group_norm(x, groups, w, b, eps=64e-5):
    """F.group_norm on [T, H*N] with H groups (model.py:1109, 1294, 1386); biased variance."""
    T, C = x.shape
    x64 = x.astype(f64).reshape(T, groups, C // groups)
    mu = x64.mean(axis=-1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(axis=-1, keepdims=True)
    y = ((x64 - mu) / np.sqrt(var + eps)).reshape(T, C) * w.astype(f64) + b.astype(f64)
    return y.astype(x.dtype)


def sigmoid(x):
    return (1.0 / (1.0 + np.exp(-x.astype(f64)))).astype(x.dtype)


def silu(x):
    x64 = x.astype(f64)
    return (x64 / (1.0 + np.exp(-x64))).astype(x.dtype)


def relu_sq(x):
    """torch.relu(k) ** 2 in the activation dtype (model.py:990): squared and rounded in x.dtype."""
    r = np.maximum(x, x.dtype.type(0))
    return (r * r).astype(x.dtype)


# ----------------------------------------------------------------------------- matmuls

class Mat:
    """One matrix of the model in the layout the reference keeps after loading:
    logical shape [N(in), M(out)]; either float (fp32 / fp16) or uint8 with mx, rx [M]
    and my, ry [N,1] (model.py:818-847)."""

    def __init__(self, w, mx=None, rx=None, my=None, ry=None):
        self.w, self.mx, self.rx, self.my, self.ry = w, mx, rx, my, ry
        self._deq = None

    @property
    def quantized(self):
        return self.w.dtype == np.uint8

    def dense_f32(self, cache, dtype=f32):
        """fp32 matrix used by the contraction.  For uint8 weights this is the dequantised
        matrix evaluated in fp32 (model.py:93 order; cuda/operators.cu:130-134 is the same
        expression with the factors commuted).  dtype=f64: the same stored values (uint8 matrix and
        its stored scale vectors) expanded without rounding, for the exact evaluation."""
        if self._deq is not None and self._deq.dtype == dtype:
            return self._deq
        if self.quantized:
            d = quant.dequant(self.w, self.mx, self.rx, self.my, self.ry, dtype=dtype)
        else:
            d = self.w.astype(dtype)
        if cache:
            self._deq = d
        return d


def matmul(a, m, atype, output_dtype=None, cache=False, via_atype=False):
    """The reference's ``matmul`` (model.py:127-140).

    uint8 weights: contraction with fp32 accumulation, result rounded to the activation
    dtype (fp16 on the GPU path: model.py:86, operators.cu:138), then cast to
    ``output_dtype`` (model.py:138).
    float weights: fp32 accumulation, result written directly in ``output_dtype``
    (model.py:150-161, gemm_fp16_cublas.cpp:31-33).  ``via_atype``: the plain-torch form
    ``(a @ b).to(output_dtype)`` (model.py:163, 167) that runs without the native library, whose
    product is first rounded to the activation dtype.
    """
    if output_dtype is None:
        output_dtype = atype
    if atype == f64:                                  # exact evaluation: no rounding anywhere
        return a @ m.dense_f32(cache, f64)
    acc = a.astype(f32) @ m.dense_f32(cache)
    if m.quantized or via_atype:
        return acc.astype(atype).astype(output_dtype)
    return acc.astype(output_dtype)


def small_matmul(a, b, out_dtype):
    """Plain ``a @ b`` / ``torch.bmm`` on float operands with fp32 accumulation (RWKV-6 LoRA,
    model.py:1268-1269, 1286)."""
    if out_dtype == f64:
        return a.astype(f64) @ b.astype(f64)
    return (a.astype(f32) @ b.astype(f32)).astype(out_dtype)


# ----------------------------------------------------------------------------- WKV-4

def wkv4(k, v, t_first, t_decay, aa, bb, pp):
    """RWKV-4 WKV recurrence with running-maximum tracking, fp32.

    model.py:1070-1084 (att_seq loop), model.py:1044-1055 (att_one) and
    cuda/operators.cu:30-46 state the same steps.  k, v: [T, C] fp32; t_first = u,
    t_decay = w = -exp(raw) (model.py:798); state (aa, bb, pp) fp32 [C].
    Returns y [T, C] fp32 and the new state.
    """
    T, C = k.shape
    ft = f64 if k.dtype == f64 else f32               # f64 only in the exact evaluation
    aa, bb, pp = aa.astype(ft), bb.astype(ft), pp.astype(ft)
    y = np.empty((T, C), dtype=ft)
    for t in range(T):
        kk, vv = k[t], v[t]
        ww = t_first + kk
        p = np.maximum(pp, ww)
        e1, e2 = np.exp(pp - p), np.exp(ww - p)
        y[t] = (e1 * aa + e2 * vv) / (e1 * bb + e2)
        ww = t_decay + pp
        p = np.maximum(ww, kk)
        e1, e2 = np.exp(ww - p), np.exp(kk - p)
        aa = e1 * aa + e2 * vv
        bb = e1 * bb + e2
        pp = p
    return y, aa, bb, pp


# ----------------------------------------------------------------------------- WKV-5 / WKV-6

def wkv56(r, k, v, w, u, S):
    """RWKV-5/6 recurrence on a per-head N x N state, fp32.

    r, k, v: [T, H, N] fp32.  w: decay already mapped to (0,1): [H, N] (v5.2), [H, 1]
    (v5.0/5.1, one decay per head) or [T, H, N] (v6, per token; model.py:1287, 1325).
    u: [H, N] or [H, 1].  S: [H, N(key j), N(value i)] -- the layout of the state list
    (model.py:1470); w and u scale the *key* index.
    Per step (model.py:1289-1291, 1331-1333; cuda/rwkv6.cu:42-66 with S transposed):
        a = k_t^T v_t ; out_t = r_t (u * a + S) ; S = a + w_t * S
    Returns out [T, H, N] fp32 and the new S.
    """
    T, H, N = r.shape
    ft = f64 if r.dtype == f64 else f32               # f64 only in the exact evaluation
    S = S.astype(ft).copy()
    out = np.empty((T, H, N), dtype=ft)
    u3 = np.broadcast_to(u.astype(ft).reshape(H, -1), (H, N))[:, :, None]
    for t in range(T):
        wt = w[t] if w.ndim == 3 else w
        w3 = np.broadcast_to(wt.astype(ft).reshape(H, -1), (H, N))[:, :, None]
        a = k[t][:, :, None] * v[t][:, None, :]
        out[t] = np.einsum('hj,hji->hi', r[t], u3 * a + S, dtype=ft)
        S = a + w3 * S
    return out, S

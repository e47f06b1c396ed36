"""Operator-level Python interface: the functions the reference's block code calls
(rwkv_pip_package/src/rwkv/model.py:51-167, 910-969), with the same names, argument
order and return values, dispatching to librwkv_hip.so through ctypes.

Weight tensors keep the reference's logical shape [N(in), M(out)].  The kernels read the
input-contiguous layout, i.e. a tensor whose strides are (1, N): ``store.t()`` of the
[M, N] array a checkpoint holds.  ``to_input_contiguous`` converts a tensor in the
reference's device layout (strides (M, 1)) once, with the repack kernel.

Every function requires tensors on a ROCm device and raises if the native library is
missing or rejects the call; nothing here computes with PyTorch.
"""
import weakref

import torch

from . import lib as _lib

F16, F32 = _lib.RWKV_DT_F16, _lib.RWKV_DT_F32


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _need_cuda(*ts):
    for t in ts:
        if not t.is_cuda:
            raise _lib.RwkvHipError("chatrwkv_amd.ops needs tensors on the GPU; there is no CPU path")


def _ptr(t):
    return t.data_ptr()


def to_input_contiguous(w):
    """Return a tensor with the same shape/values as ``w`` [N, M] and strides (1, N)."""
    N, M = w.shape
    if w.stride(0) == 1 and w.stride(1) >= N:
        return w
    _need_cuda(w)
    store = torch.empty((M, N), dtype=w.dtype, device=w.device)
    L = _lib.load()
    fn = {torch.uint8: L.rwkv_repack_u8, torch.float16: L.rwkv_repack_f16}[w.dtype]
    if not (w.stride(1) == 1 or w.stride(0) == 1):
        w = w.contiguous()
    _lib.check(fn(N, M, _ptr(w), w.stride(0), w.stride(1), _ptr(store), 1, N, _stream()), "repack")
    return store.t()


# Weight matrices that arrive in the reference's own device layout (output index contiguous: what
# ``w[x].contiguous()`` of model.py:860 leaves, asserted at cuda/wrapper.cpp:56) are repacked once per tensor and the
# copy is kept for as long as the tensor lives, so that a binding written against the reference's converted checkpoint
# works unchanged; an in-place change of the tensor (its version counter) repacks it again.
_repacked = {}


def _kernel_layout(w):
    """``w`` [N, M] as the kernels read it (strides (1, ld)): itself, or its cached repacked copy."""
    N = w.shape[0]
    if w.stride(0) == 1 and w.stride(1) >= N:
        return w
    key = id(w)
    hit = _repacked.get(key)
    if hit is not None and hit[0]() is w and hit[1] == w._version and hit[2] == w.data_ptr():
        return hit[3]
    ic = to_input_contiguous(w)
    _repacked[key] = (weakref.ref(w, lambda _, k=key: _repacked.pop(k, None)), w._version, w.data_ptr(), ic)
    return ic


def quantize_u8(w, scale_dtype=torch.float16, input_contiguous=True):
    """The reference's uint8 quantizer (model.py:818-847) on the GPU, bit-identical.

    w: fp32 [N, M] on the GPU (any of the two dense layouts).  Returns
    (q uint8 [N, M], mx [M], rx [M], my [N, 1], ry [N, 1]) with scales in ``scale_dtype``;
    q has strides (1, N) when ``input_contiguous`` else (M, 1).
    """
    _need_cuda(w)
    assert w.dtype == torch.float32 and w.dim() == 2
    N, M = w.shape
    if not ((w.stride(0) == 1 and w.stride(1) >= N) or (w.stride(1) == 1 and w.stride(0) >= M)):
        w = w.contiguous()
    dev = w.device
    if input_contiguous:
        q = torch.empty((M, N), dtype=torch.uint8, device=dev).t()
    else:
        q = torch.empty((N, M), dtype=torch.uint8, device=dev)
    mx = torch.empty(M, dtype=scale_dtype, device=dev)
    rx = torch.empty(M, dtype=scale_dtype, device=dev)
    my = torch.empty((N, 1), dtype=scale_dtype, device=dev)
    ry = torch.empty((N, 1), dtype=scale_dtype, device=dev)
    ws = torch.empty(2 * (N + M), dtype=torch.float32, device=dev)
    dt = F16 if scale_dtype == torch.float16 else F32
    rc = _lib.load().rwkv_quantize_u8(N, M, _ptr(w), w.stride(0), w.stride(1), _ptr(q), q.stride(0), q.stride(1),
                                      _ptr(mx), _ptr(rx), _ptr(my), _ptr(ry), dt, _ptr(ws), ws.numel() * 4, _stream())
    _lib.check(rc, "rwkv_quantize_u8")
    return q, mx, rx, my, ry


def cuda_mm8_one(N, M, x, w, mx, rx, my, ry):
    """model.py:75-86: y[M] = x[N] @ dequant(w), returned in x.dtype (fp16)."""
    _need_cuda(x, w)
    assert x.dtype == mx.dtype == rx.dtype == my.dtype == ry.dtype == torch.float16
    assert w.dtype == torch.uint8
    assert x.shape == (N,) and w.shape == (N, M)
    assert rx.shape == mx.shape == (M,) and ry.shape == my.shape == (N, 1)
    w = _kernel_layout(w)
    y = torch.empty((M,), device=w.device, dtype=torch.float16)
    rc = _lib.load().rwkv_mm8_one_f16(N, M, _ptr(x.contiguous()), _ptr(w), w.stride(0), w.stride(1), _ptr(mx), _ptr(rx),
                                      _ptr(my), _ptr(ry), _ptr(y), F16, _stream())
    _lib.check(rc, "rwkv_mm8_one_f16")
    return y


def mm8_one_f32(N, M, x, w, mx, rx, my, ry):
    """The raw fp32 sums of torch.ops.rwkv.mm8_one (cuda/wrapper.cpp:84) before model.py:86 rounds them."""
    _need_cuda(x, w)
    w = _kernel_layout(w)
    y = torch.empty((M,), device=w.device, dtype=torch.float32)
    rc = _lib.load().rwkv_mm8_one_f16(N, M, _ptr(x.contiguous()), _ptr(w), w.stride(0), w.stride(1), _ptr(mx), _ptr(rx),
                                      _ptr(my), _ptr(ry), _ptr(y), F32, _stream())
    _lib.check(rc, "rwkv_mm8_one_f16")
    return y


def cuda_mm8_seq(B, N, M, x, w, mx, rx, my, ry):
    """model.py:63-74: y[B, M] = x[B, N] @ dequant(w), fp16."""
    _need_cuda(x, w)
    assert x.dtype == mx.dtype == rx.dtype == my.dtype == ry.dtype == torch.float16
    assert w.dtype == torch.uint8
    assert x.shape == (B, N) and w.shape == (N, M)
    assert rx.shape == mx.shape == (M,) and ry.shape == my.shape == (N, 1)
    if x.stride(1) != 1:
        x = x.contiguous()
    w = _kernel_layout(w)
    L = _lib.load()
    y = torch.empty((B, M), device=w.device, dtype=torch.float16)
    nbytes = L.rwkv_mm8_seq_workspace(B, N)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    rc = L.rwkv_mm8_seq_f16(B, N, M, _ptr(x), x.stride(0), _ptr(w), w.stride(0), w.stride(1), _ptr(mx), _ptr(rx),
                            _ptr(my), _ptr(ry), _ptr(y), y.stride(0), _ptr(ws), nbytes, _stream())
    _lib.check(rc, "rwkv_mm8_seq_f16")
    return y


def mm8(x, w, mx, rx, my, ry):
    """model.py:122-125."""
    if len(x.shape) == 1:
        return cuda_mm8_one(w.shape[0], w.shape[1], x, w, mx, rx, my, ry)
    return cuda_mm8_seq(x.shape[0], w.shape[0], w.shape[1], x, w, mx, rx, my, ry)


def _input_contiguous_f16(b):
    """A fp16 matrix [N, M], or a batch of them [batch, N, M], in the layout the kernels stream (strides (1, N) within a
    matrix); copies only if it is not."""
    if b.stride(-2) == 1 and b.stride(-1) >= b.shape[-2] and b.stride(-1) % 8 == 0 and (b.dim() == 2 or b.stride(0) % 8 == 0):
        return b
    return b.transpose(-1, -2).contiguous().transpose(-1, -2)


def matmul_float(a, b, output_dtype=None):
    """model.py:144-161 (gemm_fp16_cublas): fp16 x fp16, fp32 accumulation, output written
    directly in ``output_dtype`` (fp16 or fp32).  1-D ``a`` gives a 1-D result; 3-D ``a`` and ``b`` are a
    batch of products (cuda/gemm_fp16_cublas.cpp:61-75): one call of rwkv_gemm_f16_batched."""
    _need_cuda(a, b)
    if output_dtype is None:
        output_dtype = a.dtype
    assert a.dtype == b.dtype == torch.float16
    assert output_dtype in (torch.float16, torch.float32)
    if a.dim() == 3:
        assert b.dim() == 3 and a.shape[0] == b.shape[0] and a.shape[2] == b.shape[1]
        step = 8 if a.shape[1] == 1 else 64          # the contraction kernel's K step (8 for one-row products)
        if a.shape[2] % step:
            pad = step - a.shape[2] % step
            a = torch.nn.functional.pad(a, (0, pad))
            b = torch.nn.functional.pad(b, (0, 0, 0, pad))
        if a.stride(2) != 1 or a.stride(1) % 8 or a.stride(0) % 8:
            a = a.contiguous()
        b = _input_contiguous_f16(b)
        nb, B, N = a.shape
        M = b.shape[2]
        c = torch.empty((nb, B, M), dtype=output_dtype, device=a.device)
        rc = _lib.load().rwkv_gemm_f16_batched(nb, B, N, M, _ptr(a), a.stride(1), a.stride(0), _ptr(b), b.stride(1),
                                               b.stride(2), b.stride(0), _ptr(c), c.stride(1), c.stride(0),
                                               F16 if output_dtype == torch.float16 else F32, _stream())
        _lib.check(rc, "rwkv_gemm_f16_batched")
        return c
    one = a.dim() == 1
    a2 = a.unsqueeze(0) if one else a
    assert a2.dim() == 2 and b.dim() == 2
    # the contraction kernel steps K by 64 (8 for a one-row product): pad the inner dimension with zeros
    step = 8 if a2.shape[0] == 1 else 64
    if a2.shape[1] % step:
        pad = step - a2.shape[1] % step
        a2 = torch.nn.functional.pad(a2, (0, pad))
        b = torch.nn.functional.pad(b, (0, 0, 0, pad))
    if a2.stride(1) != 1 or a2.stride(0) % 8 != 0:
        a2 = a2.contiguous()
    b = _input_contiguous_f16(b)
    B, N = a2.shape
    M = b.shape[1]
    c = torch.empty((B, M), dtype=output_dtype, device=a.device)
    rc = _lib.load().rwkv_gemm_f16(B, N, M, _ptr(a2), a2.stride(0), _ptr(b), b.stride(0), b.stride(1), _ptr(c),
                                   c.stride(0), F16 if output_dtype == torch.float16 else F32, _stream())
    _lib.check(rc, "rwkv_gemm_f16")
    return c[0] if one else c


def matmul(a, b, mx=None, rx=None, my=None, ry=None, output_dtype=None):
    """model.py:127-140."""
    if output_dtype is None:
        output_dtype = a.dtype
    if b.dtype == torch.float16:
        assert a.dtype == b.dtype
        return matmul_float(a, b, output_dtype=output_dtype)
    elif b.dtype == torch.uint8:
        assert mx is not None and rx is not None and my is not None and ry is not None
        return mm8(a, b, mx, rx, my, ry).to(output_dtype)
    raise ValueError("Unsupported dtype")


def cuda_wkv(T, C, w, u, k, v, aa, bb, pp):
    """model.py:52-62: RWKV-4 WKV over T tokens; aa, bb, pp are updated in place."""
    _need_cuda(k, v)
    assert k.dtype == v.dtype == torch.float32
    assert w.dtype == u.dtype == aa.dtype == bb.dtype == pp.dtype == torch.float32
    w, u, k, v = w.contiguous(), u.contiguous(), k.contiguous(), v.contiguous()
    y = torch.empty((T, C), device=w.device, dtype=k.dtype)
    rc = _lib.load().rwkv_wkv4_forward(1, T, C, _ptr(w), _ptr(u), _ptr(k), _ptr(v), _ptr(y), F32, _ptr(aa), _ptr(bb),
                                       _ptr(pp), _stream())
    _lib.check(rc, "rwkv_wkv4_forward")
    return y, aa, bb, pp


def _wkv56(fn_name, B, T, C, H, state, r, k, v, w, u, state_layout):
    _need_cuda(state, r)
    assert state.dtype == w.dtype == r.dtype == k.dtype == v.dtype == torch.float32
    for t in (r, k, v, w, state):
        assert t.is_contiguous()
    u = u.to(torch.float32).contiguous()
    y = torch.empty((B, T, C), device=w.device, dtype=torch.float32)
    fn = getattr(_lib.load(), fn_name)
    rc = fn(B, T, C, H, _ptr(state), state_layout, _ptr(r), _ptr(k), _ptr(v), _ptr(w), _ptr(u), _ptr(y), _stream())
    _lib.check(rc, fn_name)
    return y, state


def RUN_RWKV_5(B, T, C, H, state, r, k, v, w, u, state_layout=0):
    """model.py:910-935 + rwkv5.forward_fp32: w is the per-channel decay in (0,1), [C] elements."""
    return _wkv56("rwkv_wkv5_forward", B, T, C, H, state, r, k, v, w.reshape(-1).contiguous(), u, state_layout)


def RUN_RWKV_6(B, T, C, H, state, r, k, v, w, u, state_layout=0):
    """model.py:943-968 + rwkv6.forward_fp32: ``w`` is the raw per-token decay logit
    [T, C]; exp(-exp(w)) is applied here as the reference's wrapper does (model.py:959)."""
    eew = torch.exp(-torch.exp(w.float())).contiguous()
    return _wkv56("rwkv_wkv6_forward", B, T, C, H, state, r, k, v, eew, u, state_layout)


def RWKV7_OP(state, r, w, k, v, a, b):
    """model.py:198-219 (WKV_7 / torch.ops.wkv7s.forward_bf16 | _fp16 | _fp32): the RWKV-7 state recurrence over T
    tokens.  r, w, k, v, a, b: [T, C] fp16, bf16 or fp32 (one dtype), ``w`` the log-decay of model.py:537; state fp32
    [H, 64, 64] laid out [head][value][key], updated in place.  Returns y [T, C] in the input dtype."""
    _need_cuda(state, r, w, k, v, a, b)
    assert all(t.dtype == r.dtype for t in (w, k, v, a, b)) and r.dtype in (torch.float16, torch.bfloat16, torch.float32)
    assert all(t.is_contiguous() for t in (r, w, k, v, a, b))      # as the reference asserts (model.py:207)
    assert state.dtype == torch.float32 and state.is_contiguous()
    T, C = r.shape
    H = state.shape[0]
    y = torch.empty((T, C), device=r.device, dtype=r.dtype)
    rc = _lib.load().rwkv_wkv7_forward(1, T, C, H, _ptr(state), _ptr(r), _ptr(w), _ptr(k), _ptr(v), _ptr(a), _ptr(b),
                                       _ptr(y), {torch.float16: F16, torch.float32: F32, torch.bfloat16: _lib.RWKV_DT_BF16}[r.dtype],
                                       _stream())
    _lib.check(rc, "rwkv_wkv7_forward")
    return y

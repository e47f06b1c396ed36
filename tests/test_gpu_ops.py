"""GPU parity tests of the operator-level entry points (through the C ABI via ctypes)
against the numpy oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

from oracle import ops as oops
from oracle import quant as oquant

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _ops():
    from chatrwkv_amd import ops
    return ops


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _quantized(N, M, seed, atype=np.float16):
    w = (_rng(seed).standard_normal((N, M)) * 0.02).astype(np.float32)
    return w, oquant.quantize_u8(w, atype=atype)


def _to_dev_ic(q):
    """uint8/fp16 [N, M] numpy -> GPU tensor of the same shape in the input-contiguous layout."""
    return torch.from_numpy(np.ascontiguousarray(q.T)).to(DEV).t()


# ------------------------------------------------------------------------------ quantizer
@pytest.mark.parametrize("N,M", [(96, 200), (200, 96), (128, 128), (768, 3072), (3072, 768), (333, 77),
                                 (4096, 4096), (4096, 16384), (16384, 4096)])
@pytest.mark.parametrize("scale_dtype", [torch.float16, torch.float32])
def test_quantize_bit_exact(N, M, scale_dtype):
    """uint8 weights and mx/rx/my/ry equal the oracle's (which is pinned bit-exact to the
    reference's routine) for both branches, both input layouts and both output layouts."""
    ops = _ops()
    w = (_rng(N * 7 + M).standard_normal((N, M)) * 0.02).astype(np.float32)
    nat = np.float16 if scale_dtype == torch.float16 else np.float32
    q, mx, rx, my, ry = oquant.quantize_u8(w, atype=nat)
    big = N * M > 4_000_000
    for in_ic in ((True,) if big else (True, False)):
        wt = torch.from_numpy(np.ascontiguousarray(w.T)).to(DEV).t() if in_ic else torch.from_numpy(w).to(DEV)
        for out_ic in ((True,) if big else (True, False)):
            gq, gmx, grx, gmy, gry = ops.quantize_u8(wt, scale_dtype=scale_dtype, input_contiguous=out_ic)
            assert gq.shape == (N, M) and gmy.shape == (N, 1) and gmx.shape == (M,)
            assert gq.stride() == ((1, N) if out_ic else (M, 1))
            assert np.array_equal(gq.cpu().numpy(), q)
            for a, b in ((gmx, mx), (grx, rx), (gmy, my), (gry, ry)):
                assert np.array_equal(a.cpu().numpy().view(np.uint8), b.view(np.uint8))


def test_repack_round_trip():
    ops = _ops()
    q = _rng(5).integers(0, 256, size=(200, 333), dtype=np.uint8)
    t = torch.from_numpy(q).to(DEV)
    ic = ops.to_input_contiguous(t)
    assert ic.stride() == (1, 200) and np.array_equal(ic.cpu().numpy(), q)
    h = torch.from_numpy(_rng(6).standard_normal((130, 70)).astype(np.float16)).to(DEV)
    hic = ops.to_input_contiguous(h)
    assert hic.stride() == (1, 130) and torch.equal(hic, h)


# ------------------------------------------------------------------------------ mm8_one / mm8_seq
MM8_SHAPES = [(768, 768), (768, 3072), (3072, 768), (768, 50277), (2560, 2560), (4096, 4096), (4096, 16384),
              (16384, 4096), (5120, 20480), (4096, 65536)]


def _mm8_case(N, M, B, seed):
    w, (q, mx, rx, my, ry) = _quantized(N, M, seed)
    x = _rng(seed + 1).standard_normal((B, N)).astype(np.float16)
    ref = x.astype(np.float64) @ oquant.dequant_f64(q, mx, rx, my, ry)
    dev = [_to_dev_ic(q)] + [torch.from_numpy(a).to(DEV) for a in (mx, rx, my, ry)]
    return x, ref, dev


@pytest.mark.parametrize("N,M", MM8_SHAPES)
def test_mm8_one(N, M):
    """fp32 result against the fp64 evaluation of x @ W'; tolerance: 1e-3 of the output scale
    (fp16 rounding of x * ry is ~2.4e-4 relative per term), and the fp16 result within one
    fp16 ulp of the rounded fp64 value."""
    ops = _ops()
    x, ref, (q, mx, rx, my, ry) = _mm8_case(N, M, 1, N + M)
    xt = torch.from_numpy(x[0]).to(DEV)
    y32 = ops.mm8_one_f32(N, M, xt, q, mx, rx, my, ry).cpu().numpy().astype(np.float64)
    scale = np.sqrt(np.mean(ref ** 2))
    err = np.abs(y32 - ref[0]).max()
    assert err <= 1e-3 * scale, (err, scale)
    y16 = ops.cuda_mm8_one(N, M, xt, q, mx, rx, my, ry)
    assert y16.dtype == torch.float16 and y16.shape == (M,)
    d = np.abs(y16.cpu().numpy().astype(np.float64) - ref[0])
    assert d.max() <= 1e-3 * scale + np.abs(ref).max() * 2 ** -10


@pytest.mark.parametrize("N,M,B", [(768, 768, 2), (768, 3072, 5), (3072, 768, 128), (768, 50277, 3),
                                   (2560, 2560, 200), (4096, 4096, 1024), (4096, 16384, 256), (16384, 4096, 130), (4096, 16384, 1024),
                                   # long calls: 256 x 256 tiles loaded straight into LDS; whole, ragged and split-K
                                   (4096, 8192, 1000), (16384, 4096, 520), (2560, 10240, 768),
                                   # ragged tiles of the direct-to-LDS kernel: widths and row counts that end inside a tile
                                   (128, 200, 37), (192, 1000, 300), (64, 8, 2), (1024, 136, 129),
                                   # 2 .. 16 rows: every weight row streamed once, K split over the 16 waves of a workgroup
                                   (768, 768, 3), (768, 50277, 9), (4096, 4096, 2), (4096, 16384, 16), (16384, 4096, 7),
                                   (2560, 2560, 13), (5120, 20480, 16), (128, 211, 4), (64, 24, 16), (2048, 512, 6)])
def test_mm8_seq(N, M, B):
    ops = _ops()
    x, ref, (q, mx, rx, my, ry) = _mm8_case(N, M, B, N + M + B)
    xt = torch.from_numpy(x).to(DEV)
    y = ops.cuda_mm8_seq(B, N, M, xt, q, mx, rx, my, ry)
    assert y.dtype == torch.float16 and y.shape == (B, M)
    scale = np.sqrt(np.mean(ref ** 2))
    d = np.abs(y.cpu().numpy().astype(np.float64) - ref)
    assert d.max() <= 1e-3 * scale + np.abs(ref).max() * 2 ** -10, (d.max(), scale)
    # one-token mode and sequence mode agree on the same row (up to fp16 rounding)
    y1 = ops.cuda_mm8_one(N, M, xt[B - 1].contiguous(), q, mx, rx, my, ry)
    assert np.abs(y1.cpu().numpy().astype(np.float64) - y[B - 1].cpu().numpy()).max() <= np.abs(ref).max() * 2 ** -9


@pytest.mark.parametrize("N,M", [(5120, 20480), (20480, 5120), (5120, 5120)])
def test_mm8_seq_14b_call_length(N, M):
    """The launches of the 14B configuration at its own call length (1024 rows; BASELINE.json configs[4]): 320 large
    tiles = 1.25 rounds over the chip for the wide product, K split for the deep one.  Checked against the fp64
    evaluation on 40 rows that include both ends of every 128- and 256-row tile boundary, all columns."""
    ops = _ops()
    B = 1024
    w, (q, mx, rx, my, ry) = _quantized(N, M, N + M + B)
    x = _rng(N + M + B + 1).standard_normal((B, N)).astype(np.float16)
    rows = sorted({0, 1, 63, 64, 127, 128, 129, 255, 256, 257, 383, 384, 511, 512, 513, 639, 640, 767, 768, 769, 895,
                   896, 1000, 1022, 1023} | {int(r) for r in _rng(7).integers(0, B, 15)})
    ref = x[rows].astype(np.float64) @ oquant.dequant_f64(q, mx, rx, my, ry)
    dev = [_to_dev_ic(q)] + [torch.from_numpy(a).to(DEV) for a in (mx, rx, my, ry)]
    y = ops.cuda_mm8_seq(B, N, M, torch.from_numpy(x).to(DEV), *dev)
    assert y.dtype == torch.float16 and y.shape == (B, M)
    scale = np.sqrt(np.mean(ref ** 2))
    d = np.abs(y[rows].cpu().numpy().astype(np.float64) - ref)
    assert d.max() <= 1e-3 * scale + np.abs(ref).max() * 2 ** -10, (d.max(), scale)


def test_mm8_seq_timing_aid_leaves_the_product():
    """rwkv_mm8_seq_time_kernel (the kernel-only timer of the bench) runs the same two launches as
    rwkv_mm8_seq_f16: the output is bit-equal and the mean launch time is positive; whole, ragged and split-K."""
    import ctypes
    from chatrwkv_amd import lib
    ops = _ops()
    L = lib.load()
    for N, M, B in ((4096, 4096, 256), (1024, 136, 129), (16384, 4096, 520)):
        x, ref, (q, mx, rx, my, ry) = _mm8_case(N, M, B, N + M + B)
        xt = torch.from_numpy(x).to(DEV)
        want = ops.cuda_mm8_seq(B, N, M, xt, q, mx, rx, my, ry)
        y = torch.zeros((B, M), device=DEV, dtype=torch.float16)
        nbytes = L.rwkv_mm8_seq_workspace(B, N)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
        ms = ctypes.c_float(-1.0)
        rc = L.rwkv_mm8_seq_time_kernel(B, N, M, xt.data_ptr(), N, q.data_ptr(), q.stride(0), q.stride(1),
                                        mx.data_ptr(), rx.data_ptr(), my.data_ptr(), ry.data_ptr(), y.data_ptr(), M,
                                        ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream, 3,
                                        ctypes.byref(ms))
        lib.check(rc, "rwkv_mm8_seq_time_kernel")
        assert torch.equal(y, want) and 0.0 < ms.value < 100.0
        assert L.rwkv_mm8_seq_time_kernel(B, N, M, xt.data_ptr(), N, q.data_ptr(), q.stride(0), q.stride(1),
                                          mx.data_ptr(), rx.data_ptr(), my.data_ptr(), ry.data_ptr(), y.data_ptr(),
                                          M, ws.data_ptr(), nbytes, None, 0, ctypes.byref(ms)) == -1  # RWKV_E_SHAPE


def test_mm8_linearity_full_size():
    """Size-independent property at the 7B shape: mm8(a + b) == mm8(a) + mm8(b) in fp32 up to rounding."""
    ops = _ops()
    N, M = 4096, 16384
    x, ref, (q, mx, rx, my, ry) = _mm8_case(N, M, 2, 99)
    a, b = torch.from_numpy(x[0]).to(DEV), torch.from_numpy(x[1]).to(DEV)
    s = (a.float() + b.float()).half()
    ya, yb, ys = (ops.mm8_one_f32(N, M, t, q, mx, rx, my, ry) for t in (a, b, s))
    exact_s = s.float().cpu().numpy().astype(np.float64) @ oquant.dequant_f64(
        q.cpu().numpy(), *(t.cpu().numpy() for t in (mx, rx, my, ry)))
    assert np.abs(ys.cpu().numpy() - exact_s).max() <= 1e-3 * np.sqrt(np.mean(exact_s ** 2))
    lin = (ya + yb - ys).abs().max().item()
    assert lin <= 2e-2 * float(np.sqrt(np.mean(exact_s ** 2)))  # s is rounded to fp16


# ------------------------------------------------------------------------------ fp16 gemm / gemv
@pytest.mark.parametrize("N,M,B", [(768, 768, 1), (768, 3072, 1), (4096, 4096, 1), (16384, 4096, 1), (768, 50277, 1),
                                   (768, 768, 7), (3072, 768, 128), (4096, 4096, 300), (768, 50277, 4),
                                   # long calls (256 x 256 tiles loaded straight into LDS): split-K, ragged, shallow
                                   (4096, 4096, 1024), (4096, 8192, 520), (128, 4096, 1024),
                                   (128, 200, 37), (192, 1000, 300), (64, 8, 2),
                                   # 2 .. 16 rows: the streaming kernel
                                   (768, 768, 3), (4096, 4096, 16), (16384, 4096, 5), (2560, 10240, 11), (128, 211, 2), (2048, 512, 6),
                                   # narrow outputs of a LoRA's first stage (17 .. 512 rows, up to 192 outputs, fp16 out):
                                   # ragged rows, an output count that is no multiple of 16, a row length that is no
                                   # multiple of the 512 values one round of the eight waves covers, the row limit
                                   (4096, 160, 256), (4096, 64, 37), (5120, 100, 300), (1056, 192, 512), (4096, 128, 17)])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_gemm_f16(N, M, B, out_dtype):
    ops = _ops()
    w = (_rng(N + 3 * M).standard_normal((N, M)) * 0.02).astype(np.float16)
    x = _rng(B).standard_normal((B, N)).astype(np.float16)
    ref = x.astype(np.float64) @ w.astype(np.float64)
    wt = _to_dev_ic(w)
    xt = torch.from_numpy(x).to(DEV)
    y = ops.matmul_float(xt[0] if B == 1 else xt, wt, output_dtype=out_dtype)
    assert y.dtype == out_dtype and tuple(y.shape) == ((M,) if B == 1 else (B, M))
    d = np.abs(y.cpu().numpy().astype(np.float64).reshape(B, M) - ref).max()
    tol = 1e-4 * np.sqrt(np.mean(ref ** 2)) + (np.abs(ref).max() * 2 ** -10 if out_dtype == torch.float16 else 0)
    assert d <= tol, (d, tol)


def test_gemm_f16_batched_and_row_major():
    """3-D operands are a batch of products (the RWKV-6 LoRA use, model.py:1269: [5, T, 32] x [5, 32, C]), and a
    plain row-major weight tensor is accepted (converted to the streamed layout)."""
    ops = _ops()
    r = _rng(99)
    a = (r.standard_normal((5, 9, 32))).astype(np.float16)
    b = (r.standard_normal((5, 32, 256)) * 0.1).astype(np.float16)
    ref = np.einsum("bij,bjk->bik", a.astype(np.float64), b.astype(np.float64))
    y = ops.matmul_float(torch.from_numpy(a).to(DEV), torch.from_numpy(b).to(DEV))
    assert y.dtype == torch.float16 and tuple(y.shape) == (5, 9, 256)
    assert np.abs(y.cpu().numpy().astype(np.float64) - ref).max() <= np.abs(ref).max() * 2 ** -10 + 1e-4
    y32 = ops.matmul_float(torch.from_numpy(a[0]).to(DEV), torch.from_numpy(b[0]).to(DEV), output_dtype=torch.float32)
    assert y32.dtype == torch.float32
    assert np.abs(y32.cpu().numpy().astype(np.float64) - ref[0]).max() <= 1e-4 * max(np.abs(ref[0]).max(), 1.0)


def test_gemm_f16_batched_entry_strides():
    """rwkv_gemm_f16_batched through the C ABI with batch strides that are not the dense ones: operands and results
    of the five products lie in larger buffers; long enough (300 rows, K = 64) for the MFMA kernel, and one-row
    products for the streaming one."""
    from chatrwkv_amd import lib
    L = lib.load()
    r = _rng(17)
    nb, N, M = 5, 64, 136
    for B in (300, 1):
        a = torch.from_numpy(r.standard_normal((nb, B + 3, N)).astype(np.float16)).to(DEV)      # 3 unused rows per item
        bt = torch.from_numpy((r.standard_normal((nb, M + 2, N)) * 0.1).astype(np.float16)).to(DEV)  # [batch, M + 2, N]
        c = torch.full((nb, B + 1, M), float("nan"), dtype=torch.float32, device=DEV)
        rc = L.rwkv_gemm_f16_batched(nb, B, N, M, a.data_ptr(), a.stride(1), a.stride(0), bt.data_ptr(), 1, bt.stride(1),
                                     bt.stride(0), c.data_ptr(), c.stride(1), c.stride(0), lib.RWKV_DT_F32,
                                     torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        ref = np.einsum("bij,bkj->bik", a[:, :B].cpu().numpy().astype(np.float64), bt[:, :M].cpu().numpy().astype(np.float64))
        got = c[:, :B].cpu().numpy().astype(np.float64)
        assert np.abs(got - ref).max() <= 1e-4 * max(np.abs(ref).max(), 1.0)
        assert bool(torch.isnan(c[:, B]).all())                                               # the spare row is untouched
    assert L.rwkv_gemm_f16_batched(0, 4, 64, 8, a.data_ptr(), 64, 0, bt.data_ptr(), 1, 64, 0, c.data_ptr(), 8, 0, 0, None) == -1
    assert L.rwkv_gemm_f16_batched(2, 4, 64, 8, a.data_ptr(), 64, 4, bt.data_ptr(), 1, 64, 0, c.data_ptr(), 8, 0, 0, None) == -2


def test_mm8_accepts_the_reference_device_layout():
    """A uint8 matrix as the reference's loader leaves it on the GPU (``.contiguous()`` [N, M], output index
    contiguous; model.py:860): the operator functions repack it once per tensor and reuse the copy; results equal the
    ones from the kernel layout bit for bit, and an in-place change of the tensor is seen."""
    ops = _ops()
    N, M, B = 768, 3072, 37
    x, ref, (q_ic, mx, rx, my, ry) = _mm8_case(N, M, B, 4321)
    q_ref = q_ic.contiguous()                                  # strides (M, 1): the reference's layout
    assert q_ref.stride() == (M, 1) and q_ic.stride() == (1, N)
    xt = torch.from_numpy(x).to(DEV)
    y_ic = ops.cuda_mm8_seq(B, N, M, xt, q_ic, mx, rx, my, ry)
    y_ref = ops.cuda_mm8_seq(B, N, M, xt, q_ref, mx, rx, my, ry)
    assert torch.equal(y_ic, y_ref)
    n_cached = len(ops._repacked)
    y1 = ops.cuda_mm8_one(N, M, xt[0].contiguous(), q_ref, mx, rx, my, ry)
    assert len(ops._repacked) == n_cached                      # the second call reused the repacked copy
    assert torch.equal(y1, ops.cuda_mm8_one(N, M, xt[0].contiguous(), q_ic, mx, rx, my, ry))
    q_ref[5].add_(1)                                           # in place: the version counter moves, the copy is redone
    q_ic2 = q_ic.clone()
    q_ic2[5].add_(1)
    assert torch.equal(ops.cuda_mm8_seq(B, N, M, xt, q_ref, mx, rx, my, ry), ops.cuda_mm8_seq(B, N, M, xt, q_ic2, mx, rx, my, ry))
    del q_ref
    import gc
    gc.collect()
    assert len(ops._repacked) == n_cached - 1                  # the copy goes with the tensor


# ------------------------------------------------------------------------------ WKV
@pytest.mark.parametrize("T,C", [(1, 768), (7, 768), (64, 1000), (300, 768), (1024, 4096)])
def test_wkv4(T, C):
    ops = _ops()
    r = _rng(T * C)
    k = r.standard_normal((T, C)).astype(np.float32)
    v = r.standard_normal((T, C)).astype(np.float32)
    w = -np.exp(r.uniform(-6, -1, C)).astype(np.float32)
    u = r.uniform(-1, 1, C).astype(np.float32)
    aa = r.standard_normal(C).astype(np.float32)
    bb = np.abs(r.standard_normal(C)).astype(np.float32) + 0.1
    pp = r.standard_normal(C).astype(np.float32)
    for zero_state in (True, False):
        if zero_state:
            a0, b0, p0 = np.zeros(C, np.float32), np.zeros(C, np.float32), np.full(C, -1e30, np.float32)
        else:
            a0, b0, p0 = aa, bb, pp
        y_ref, a_ref, b_ref, p_ref = oops.wkv4(k, v, u, w, a0, b0, p0)
        ta, tb, tp = (torch.from_numpy(t.copy()).to(DEV) for t in (a0, b0, p0))
        y, ta2, tb2, tp2 = ops.cuda_wkv(T, C, torch.from_numpy(w).to(DEV), torch.from_numpy(u).to(DEV),
                                        torch.from_numpy(k).to(DEV), torch.from_numpy(v).to(DEV), ta, tb, tp)
        assert ta2 is ta  # state is updated in place, as the reference's kernel does
        np.testing.assert_allclose(y.cpu().numpy(), y_ref, rtol=2e-4, atol=2e-4)
        np.testing.assert_allclose(ta.cpu().numpy(), a_ref, rtol=2e-4, atol=2e-4)
        np.testing.assert_allclose(tb.cpu().numpy(), b_ref, rtol=2e-4, atol=2e-4)
        np.testing.assert_allclose(tp.cpu().numpy(), p_ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("T,H", [(1, 2), (5, 3), (16, 2), (17, 2), (50, 4), (256, 64)])
@pytest.mark.parametrize("v6", [False, True])
@pytest.mark.parametrize("layout", [0, 1])
def test_wkv56(T, H, v6, layout):
    ops = _ops()
    N = 64
    C = H * N
    g = _rng(T * H + 10 * layout + int(v6))
    r, k, v = (g.standard_normal((T, H, N)).astype(np.float32) * 0.5 for _ in range(3))
    u = g.uniform(-1, 1, (H, N)).astype(np.float32)
    S0 = g.standard_normal((H, N, N)).astype(np.float32)  # [h][key j][value i], deliberately non-symmetric
    if v6:
        wlogit = g.uniform(-6, 1, (T, H, N)).astype(np.float32)
        dec = np.exp(-np.exp(wlogit)).astype(np.float32)
    else:
        dec = np.exp(-np.exp(g.uniform(-6, 1, (H, N)))).astype(np.float32)
    out_ref, S_ref = oops.wkv56(r, k, v, dec, u, S0)
    st = S0 if layout == 1 else np.ascontiguousarray(S0.transpose(0, 2, 1))
    st_t = torch.from_numpy(st.copy()).to(DEV)
    args = [torch.from_numpy(a.reshape(1, T, C).copy()).to(DEV) for a in (r, k, v)]
    ut = torch.from_numpy(u.reshape(-1)).to(DEV)
    if v6:
        y, st2 = ops.RUN_RWKV_6(1, T, C, H, st_t, *args, torch.from_numpy(wlogit.reshape(1, T, C)).to(DEV), ut,
                                state_layout=layout)
    else:
        y, st2 = ops.RUN_RWKV_5(1, T, C, H, st_t, *args, torch.from_numpy(dec.reshape(-1)).to(DEV), ut,
                                state_layout=layout)
    assert st2 is st_t and y.shape == (1, T, C)
    np.testing.assert_allclose(y.cpu().numpy().reshape(T, H, N), out_ref, rtol=1e-4, atol=1e-4)
    got = st_t.cpu().numpy()
    if layout == 0:
        got = got.transpose(0, 2, 1)
    np.testing.assert_allclose(got, S_ref, rtol=1e-4, atol=1e-4)

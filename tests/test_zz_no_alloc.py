"""rwkv_mm8_seq_f16_static: the dequant-matmul for callers that cannot allocate device memory.

Called through the C ABI with outputs that exist before the call, and compared with rwkv_mm8_seq_f16 (the entry
point that takes a workspace) on the same inputs: two calls in a row, the second with a smaller input, so that
whatever the first call left in the library's built-in scratch does not leak into the second.  Then shapes whose
K split differs between the two entry points, the size limit, and a check that the call allocates nothing."""
import numpy as np
import pytest
import torch

from oracle import quant as oquant

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _case(N, M, B, seed):
    g = np.random.Generator(np.random.PCG64(seed))
    w = (g.standard_normal((N, M)) * 0.02).astype(np.float32)
    q, mx, rx, my, ry = oquant.quantize_u8(w, atype=np.float16)
    x = g.standard_normal((B, N)).astype(np.float16)
    ref = x.astype(np.float64) @ oquant.dequant_f64(q, mx, rx, my, ry)
    qd = torch.from_numpy(np.ascontiguousarray(q.T)).to(DEV).t()        # input-contiguous
    vec = [torch.from_numpy(a).to(DEV) for a in (mx, rx, my, ry)]
    return torch.from_numpy(x).to(DEV), qd, vec, ref


def _both(L, x, q, vec, y_static, y_ws, ws):
    """Both entry points on the same operands; outputs and workspace are allocated by the caller beforehand."""
    B, N = x.shape
    M = q.shape[1]
    mx, rx, my, ry = vec
    st = torch.cuda.current_stream().cuda_stream
    before = torch.cuda.memory_allocated()
    rc = L.rwkv_mm8_seq_f16_static(B, N, M, x.data_ptr(), x.stride(0), q.data_ptr(), q.stride(0), q.stride(1),
                                   mx.data_ptr(), rx.data_ptr(), my.data_ptr(), ry.data_ptr(), y_static.data_ptr(),
                                   y_static.stride(0), st)
    assert rc == 0, rc
    assert torch.cuda.memory_allocated() == before                      # nothing allocated through torch either
    rc = L.rwkv_mm8_seq_f16(B, N, M, x.data_ptr(), x.stride(0), q.data_ptr(), q.stride(0), q.stride(1),
                            mx.data_ptr(), rx.data_ptr(), my.data_ptr(), ry.data_ptr(), y_ws.data_ptr(),
                            y_ws.stride(0), ws.data_ptr(), ws.numel(), st)
    assert rc == 0, rc
    torch.cuda.synchronize()


def _check(y_static, y_ws, ref, exact):
    a, b = y_static.float().cpu().numpy(), y_ws.float().cpu().numpy()
    scale = np.sqrt(np.mean(ref ** 2))
    tol = 1e-3 * scale + np.abs(ref).max() * 2 ** -10                  # the bound test_mm8_seq uses against fp64
    assert np.abs(a - ref).max() <= tol, (np.abs(a - ref).max(), tol)
    if exact:
        assert np.array_equal(a, b)                                     # same kernels, same split: same bits
    else:
        assert np.abs(a - b).max() <= np.abs(ref).max() * 2 ** -10      # one fp16 rounding step of the largest output


def test_static_scratch_entry_matches_workspace_entry():
    from chatrwkv_amd import lib
    L = lib.load()
    assert L.rwkv_mm8_seq_static_max_elems() == 4 << 20 and L.rwkv_mm8_seq_static_max_rows() == 8192
    big = _case(4096, 4096, 300, 1)        # first call: 300 rows, fills 2.4 MB of the scratch, K split
    small = _case(768, 3072, 37, 2)        # second call: smaller in every dimension, ragged row tile
    ws = torch.empty(L.rwkv_mm8_seq_workspace(300, 4096), dtype=torch.uint8, device=DEV)
    outs = []
    for x, q, vec, ref in (big, small):
        B, M = x.shape[0], q.shape[1]
        y_static = torch.full((B, M), float("nan"), dtype=torch.float16, device=DEV)
        y_ws = torch.full((B, M), float("nan"), dtype=torch.float16, device=DEV)
        outs.append((y_static, y_ws, ref))
    torch.cuda.synchronize()
    for (x, q, vec, ref), (y_static, y_ws, _) in zip((big, small), outs):
        _both(L, x, q, vec, y_static, y_ws, ws)
    for y_static, y_ws, ref in outs:
        _check(y_static, y_ws, ref, exact=True)
    # the first shape again after the small one: what the small call left behind does not matter either
    x, q, vec, ref = big
    y_static, y_ws = torch.empty_like(outs[0][0]), torch.empty_like(outs[0][1])
    _both(L, x, q, vec, y_static, y_ws, ws)
    _check(y_static, y_ws, ref, exact=True)
    assert torch.equal(y_static, outs[0][0])


@pytest.mark.parametrize("N,M,B", [(4096, 16384, 256), (16384, 4096, 130), (64, 8, 2), (4096, 4096, 1024)])
def test_static_scratch_entry_other_shapes(N, M, B):
    """Shapes whose split-K slabs may not fit the built-in 16 MiB: the product is then split less (or not at all),
    which changes the order of the fp32 sums only."""
    from chatrwkv_amd import lib
    L = lib.load()
    x, q, vec, ref = _case(N, M, B, N + M + B)
    ws = torch.empty(L.rwkv_mm8_seq_workspace(B, N), dtype=torch.uint8, device=DEV)
    y_static = torch.empty((B, M), dtype=torch.float16, device=DEV)
    y_ws = torch.empty((B, M), dtype=torch.float16, device=DEV)
    _both(L, x, q, vec, y_static, y_ws, ws)
    _check(y_static, y_ws, ref, exact=False)


def test_static_scratch_entry_rejects_oversize():
    from chatrwkv_amd import lib
    L = lib.load()
    x, q, vec, _ = _case(64, 8, 2, 5)
    mx, rx, my, ry = vec
    y = torch.zeros((2, 8), dtype=torch.float16, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    args = lambda B, N, M: (B, N, M, x.data_ptr(), N, q.data_ptr(), 1, N, mx.data_ptr(), rx.data_ptr(), my.data_ptr(),
                            ry.data_ptr(), y.data_ptr(), M, st)
    # nothing is launched for a rejected size, so the (too small) operands are never touched
    assert L.rwkv_mm8_seq_f16_static(*args(1025, 4096, 8)) == -6        # B * N beyond 4 Mi elements
    assert L.rwkv_mm8_seq_f16_static(*args(8193, 64, 8)) == -6          # more rows than the sums hold
    with pytest.raises(lib.RwkvHipError, match="RWKV_E_SCRATCH"):
        lib.check(-6, "rwkv_mm8_seq_f16_static")
    torch.cuda.synchronize()
    assert float(y.abs().max()) == 0.0


def test_static_scratch_entry_under_graph_capture():
    """The entry point is meant for callers under HIP graph capture: after one call outside capture (the first call on
    a device does host-side set-up), the call is captured into a graph; three replays, with eager work and
    synchronisations between them and the input changed before the last one, each equal to rwkv_mm8_seq_f16 on the
    same input bit for bit."""
    from chatrwkv_amd import lib
    L = lib.load()
    x, q, vec, ref = _case(4096, 4096, 300, 11)
    B, N, M = 300, 4096, 4096
    mx, rx, my, ry = vec
    ws = torch.empty(L.rwkv_mm8_seq_workspace(B, N), dtype=torch.uint8, device=DEV)
    y_static = torch.empty((B, M), dtype=torch.float16, device=DEV)
    y_ws = torch.empty((B, M), dtype=torch.float16, device=DEV)
    _both(L, x, q, vec, y_static, y_ws, ws)                     # warm call outside capture
    assert torch.equal(y_static, y_ws)
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            rc = L.rwkv_mm8_seq_f16_static(B, N, M, x.data_ptr(), x.stride(0), q.data_ptr(), q.stride(0), q.stride(1),
                                           mx.data_ptr(), rx.data_ptr(), my.data_ptr(), ry.data_ptr(), y_static.data_ptr(),
                                           y_static.stride(0), torch.cuda.current_stream().cuda_stream)
            assert rc == 0, rc
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        if rep == 2:
            x.mul_(0.5)                                        # new input in the same buffer
        y_static.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        rc = L.rwkv_mm8_seq_f16(B, N, M, x.data_ptr(), x.stride(0), q.data_ptr(), q.stride(0), q.stride(1), mx.data_ptr(),
                                rx.data_ptr(), my.data_ptr(), ry.data_ptr(), y_ws.data_ptr(), y_ws.stride(0), ws.data_ptr(),
                                ws.numel(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        assert torch.equal(y_static, y_ws), rep

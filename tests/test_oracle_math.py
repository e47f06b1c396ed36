"""What the mathematics fixes about the oracle, independent of any golden vector: closed forms,
invariants and library routines chosen so that a dropped term, a wrong sign or a transposed
operand fails."""
import numpy as np
import pytest
import torch

from chatrwkv_amd import synth
from oracle import ops as oops
from oracle import quant as oquant
from oracle.model import OracleRWKV


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


# ------------------------------------------------------------------------------ quantizer
@pytest.mark.parametrize("N,M", [(96, 200), (200, 96), (64, 64), (33, 7)])
def test_quantizer_invariants(N, M):
    w = (rng(N + M).standard_normal((N, M)) * 0.02).astype(np.float32)
    q, mx, rx, my, ry = oquant.quantize_u8(w)
    assert q.dtype == np.uint8 and q.shape == (N, M) and my.shape == (N, 1) and mx.shape == (M,)
    # the last two steps divide by the column max, then by the row max: every row attains 255
    # and (subtracted minima) every row and every column contains a 0
    assert (q.max(axis=1) == 255).all()
    assert (q.min(axis=1) == 0).all() and (q.min(axis=0) == 0).all()
    rec = oquant.dequant_f64(q, mx, rx, my, ry)
    step = rx[None, :].astype(np.float64) * ry.astype(np.float64)
    assert (np.abs(rec - w) <= 0.5 * step * (1 + 1e-4) + 1e-9).all()
    # scaling the matrix by a power of two changes only the scales
    q2, mx2, rx2, my2, ry2 = oquant.quantize_u8(w / 4)
    assert np.array_equal(q, q2)
    np.testing.assert_array_equal(mx2, mx / 4)
    np.testing.assert_array_equal(my2, my / 4)
    np.testing.assert_array_equal(rx2 * ry2, (rx * ry) / 4)


def test_quantizer_branch_order_matters():
    """N > M subtracts the row minimum first, N <= M the column minimum first."""
    w = np.array([[0.0, 1.0], [2.0, 5.0], [4.0, 4.5]], dtype=np.float32)   # N=3 > M=2
    np.seterr(invalid="ignore")   # a 3x2 toy leaves a constant column: 0/0 as in the reference
    _, mx, _, my, _ = oquant.quantize_u8(w)
    np.testing.assert_array_equal(my[:, 0], [0.0, 2.0, 4.0])
    np.testing.assert_array_equal(mx, [0.0, 0.5])
    _, mx, _, my, _ = oquant.quantize_u8(w.T.copy())                        # N=2 <= M=3
    np.testing.assert_array_equal(mx, [0.0, 2.0, 4.0])
    np.testing.assert_array_equal(my[:, 0], [0.0, 0.5])


def test_mm8_equals_dense_matmul_and_factorised_form():
    N, M, B = 80, 48, 5
    w = (rng(1).standard_normal((N, M)) * 0.02).astype(np.float32)
    q, mx, rx, my, ry = oquant.quantize_u8(w)
    x = rng(2).standard_normal((B, N)).astype(np.float32)
    dense = x.astype(np.float64) @ oquant.dequant_f64(q, mx, rx, my, ry)
    got = oops.matmul(x, oops.Mat(q, mx, rx, my, ry), np.float32)
    np.testing.assert_allclose(got, dense, rtol=1e-5, atol=1e-5)
    x64 = x.astype(np.float64)
    fact = ((x64 * ry[:, 0]) @ (q + 0.5)) * rx + np.outer(x64.sum(1), mx) + (x64 @ my[:, 0])[:, None]
    np.testing.assert_allclose(fact, dense, rtol=1e-12, atol=1e-12)
    # against the original weights: the error of one row is bounded by the quantisation step
    exact = x64 @ w
    assert np.abs(dense - exact).max() <= np.abs(x64).sum(1).max() * 0.5 * (rx.max() * ry.max())


# ------------------------------------------------------------------------------ norms
def test_norms_match_torch():
    x = rng(3).standard_normal((4, 128)).astype(np.float32)
    w = rng(4).standard_normal(128).astype(np.float32)
    b = rng(5).standard_normal(128).astype(np.float32)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x), (128,), torch.from_numpy(w), torch.from_numpy(b)).numpy()
    np.testing.assert_allclose(oops.layer_norm(x, w, b), ref, rtol=1e-5, atol=1e-5)
    ref = torch.nn.functional.group_norm(torch.from_numpy(x), 2, torch.from_numpy(w), torch.from_numpy(b), eps=64e-5).numpy()
    np.testing.assert_allclose(oops.group_norm(x, 2, w, b), ref, rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------------------ WKV-4
def _wkv4_closed_form(k, v, u, w, T):
    """wkv_t = (sum_{i<t} e^{(t-1-i) w + k_i} v_i + e^{u + k_t} v_t) / (sum_{i<t} e^{(t-1-i) w + k_i} + e^{u + k_t})."""
    k, v, u, w = (a.astype(np.float64) for a in (k, v, u, w))
    out = np.zeros_like(k)
    for t in range(T):
        num = np.exp(u + k[t]) * v[t]
        den = np.exp(u + k[t])
        for i in range(t):
            e = np.exp((t - 1 - i) * w + k[i])
            num += e * v[i]
            den += e
        out[t] = num / den
    return out


def test_wkv4_closed_form_and_special_cases():
    T, C = 9, 6
    g = rng(6)
    k, v = g.standard_normal((T, C)).astype(np.float32), g.standard_normal((T, C)).astype(np.float32)
    w = -np.exp(g.uniform(-6, -1, C)).astype(np.float32)
    u = g.uniform(-1, 1, C).astype(np.float32)
    z, m = np.zeros(C, np.float32), np.full(C, -1e30, np.float32)
    y, aa, bb, pp = oops.wkv4(k, v, u, w, z, z, m)
    np.testing.assert_allclose(y, _wkv4_closed_form(k, v, u, w, T), rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(y[0], v[0], rtol=1e-6)            # empty history: wkv = v
    # state carries: processing [0:4] then [4:9] equals one pass; one-token mode == sequence of length 1
    y1, a1, b1, p1 = oops.wkv4(k[:4], v[:4], u, w, z, z, m)
    y2, a2, b2, p2 = oops.wkv4(k[4:], v[4:], u, w, a1, b1, p1)
    np.testing.assert_allclose(np.concatenate([y1, y2]), y, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(a2 * np.exp(p2 - pp), aa, rtol=1e-4, atol=1e-6)
    # large k must not overflow (running maximum)
    yb, *_ = oops.wkv4(k + 80, v, u, w, z, z, m)
    assert np.isfinite(yb).all()
    np.testing.assert_allclose(yb, y, rtol=1e-4, atol=1e-5)       # wkv is invariant to a common shift of k


# ------------------------------------------------------------------------------ WKV-5 / 6
def _wkv56_closed_form(r, k, v, w, u, S0):
    """out_t = r_t (diag(u) k_t^T v_t + sum_{i<t} diag(prod_{i<s<t} w_s) k_i^T v_i + diag(prod_{s<t} w_s) S0)."""
    T, H, N = r.shape
    r, k, v, u, S0 = (a.astype(np.float64) for a in (r, k, v, u, S0))
    w = w.astype(np.float64)
    wt = (lambda t: w[t]) if w.ndim == 3 else (lambda t: w)
    out = np.zeros((T, H, N))
    for t in range(T):
        for h in range(H):
            M = np.diag(u[h]) @ np.outer(k[t, h], v[t, h])
            for i in range(t):
                d = np.ones(N)
                for s in range(i + 1, t):
                    d = d * wt(s)[h]
                M += np.diag(d) @ np.outer(k[i, h], v[i, h])
            d = np.ones(N)
            for s in range(t):
                d = d * wt(s)[h]
            M += np.diag(d) @ S0[h]
            out[t, h] = r[t, h] @ M
    return out


@pytest.mark.parametrize("per_token", [False, True])
def test_wkv56_closed_form(per_token):
    T, H, N = 6, 2, 5
    g = rng(7 + per_token)
    r, k, v = (g.standard_normal((T, H, N)).astype(np.float32) for _ in range(3))
    u = g.uniform(-1, 1, (H, N)).astype(np.float32)
    w = np.exp(-np.exp(g.uniform(-3, 1, (T, H, N) if per_token else (H, N)))).astype(np.float32)
    S0 = g.standard_normal((H, N, N)).astype(np.float32)        # non-symmetric: [h][key][value]
    out, S = oops.wkv56(r, k, v, w, u, S0)
    np.testing.assert_allclose(out, _wkv56_closed_form(r, k, v, w, u, S0), rtol=2e-4, atol=2e-5)
    # a transposed state must NOT give the same answer (guards the key/value index convention)
    out_t, _ = oops.wkv56(r, k, v, w, u, S0.transpose(0, 2, 1).copy())
    assert np.abs(out_t - out).max() > 1e-2
    # chunking carries the state
    o1, S1 = oops.wkv56(r[:2], k[:2], v[:2], w[:2] if per_token else w, u, S0)
    o2, S2 = oops.wkv56(r[2:], k[2:], v[2:], w[2:] if per_token else w, u, S1)
    np.testing.assert_allclose(np.concatenate([o1, o2]), out, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(S2, S, rtol=1e-5, atol=1e-6)


def test_wkv5_parallel_form_equals_recurrence():
    """The T x T decay-matrix form used for RWKV-5.0 / 5.1 sequences equals the recurrent form."""
    T, H, N = 7, 2, 4
    g = rng(9)
    r, k, v = (g.standard_normal((T, H, N)) for _ in range(3))
    wh = np.exp(-np.exp(g.uniform(-3, 0, H)))                    # one decay per head
    uh = g.uniform(-1, 1, H)
    S0 = g.standard_normal((H, N, N))
    out, S = oops.wkv56(r.astype(np.float32), k.astype(np.float32), v.astype(np.float32),
                        wh.reshape(H, 1).astype(np.float32), uh.reshape(H, 1).astype(np.float32), S0.astype(np.float32))
    par = np.zeros((T, H, N))
    for h in range(H):
        A = r[:, h] @ k[:, h].T                                  # [t, i]
        D = np.zeros((T, T))
        for t in range(T):
            for i in range(T):
                D[t, i] = wh[h] ** (t - 1 - i) if i < t else (uh[h] if i == t else 0.0)
        par[:, h] = (A * D) @ v[:, h] + (r[:, h] @ S0[h]) * (wh[h] ** np.arange(T))[:, None]
    np.testing.assert_allclose(out, par, rtol=2e-4, atol=2e-5)


# ------------------------------------------------------------------------------ forward
@pytest.mark.parametrize("ver", [4, 5.2, 6])
@pytest.mark.parametrize("strat", ["cpu fp32i8", "cuda fp16i8"])
def test_forward_chunk_invariance_and_full_output(ver, strat):
    ck = synth.make_checkpoint(version=ver, n_layer=2, n_embd=128, n_ffn=256, vocab=60, seed=5)
    o = OracleRWKV(ck, strat)
    toks = synth.random_tokens(8, 60, seed=1)
    full, st_full = o.forward(toks, None, full_output=True)
    last, st_last = o.forward(toks, None)
    np.testing.assert_allclose(full[-1], last, rtol=1e-5, atol=1e-6)   # BLAS gemm vs gemv summation order
    s, outs = None, []
    for a, b in ((0, 3), (3, 4), (4, 8)):
        out, s = o.forward(toks[a:b], s)
        outs.append(out)
    tol = 1e-4 if strat.startswith("cpu") else 2e-2
    np.testing.assert_allclose(outs[-1], last, rtol=tol, atol=tol)
    np.testing.assert_allclose(outs[0], full[2], rtol=tol, atol=tol)
    for a, b in zip(s, st_last):
        np.testing.assert_allclose(a.astype(np.float32), b.astype(np.float32), rtol=tol, atol=tol)
    init = o.init_state()
    if ver == 4:
        assert len(init) == 10 and (init[3] == -1e30).all() and init[0].dtype == o.atype and init[1].dtype == np.float32
    else:
        assert len(init) == 6 and init[1].shape == (2, 64, 64) and init[1].dtype == np.float32


def test_rescale_is_invisible_in_logits():
    """fp32 evaluation with and without the x/2 rescale (and the matching weight scaling) agrees:
    ln_out removes the factor."""
    ck = synth.make_checkpoint(version=4, n_layer=7, n_embd=64, n_ffn=128, vocab=40, seed=3)
    toks = synth.random_tokens(5, 40, seed=2)
    a, _ = OracleRWKV(ck, "cpu fp32", rescale_layer=0).forward(toks, None)
    b, _ = OracleRWKV(ck, "cpu fp32", rescale_layer=6).forward(toks, None)
    np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-5)

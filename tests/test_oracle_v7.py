"""The RWKV-7 oracle against the golden vectors written by the reference's own CPU path
(tests/golden/make_goldens_v7.py), and its two restatements of the state recurrence against each
other and against a scalar loop.  A wrong sign, index, transposed state or dropped term fails here."""
import os

import numpy as np
import pytest

from chatrwkv_amd import synth
from oracle import model_v7
from oracle.model_v7 import OracleRWKV7

from tests.golden.make_goldens_v7 import TINY7, CKPT_SEED, CHUNKS

G = os.path.join(os.path.dirname(__file__), "golden")

# fp32: accumulation order only.  fp16: a few half-precision roundings of logits of magnitude ~2.5
# (the reference's CPU half kernels and numpy round the same operations, but sum in different orders)
TOL = {"cpu fp32": 2e-5, "cpu fp16": 1.2e-2}


@pytest.mark.parametrize("strat", ["cpu fp32", "cpu fp16"])
@pytest.mark.parametrize("kernel_form", [False, True])
@pytest.mark.parametrize("de", [False, True])
def test_v7_forward_matches_reference(strat, kernel_form, de):
    """de: the DeepEmbed variant (reference run with RWKV_DE_VERSION=1 on a checkpoint with the ffn.s_* tensors)."""
    g = dict(np.load(os.path.join(G, f"e2e_v7_{'de_' if de else ''}{strat.replace(' ', '_')}.npz")))
    ck = synth.make_checkpoint_v7(seed=CKPT_SEED + (1 if de else 0), deep_embed=de, **TINY7)
    toks = [int(t) for t in g["tokens"]]
    m = OracleRWKV7(ck, strat, kernel_form=kernel_form, deep_embed=de)
    full, st = m.forward(toks, None, full_output=True)
    assert full.shape == g["full_logits"].shape
    assert np.abs(full.astype(np.float32) - g["full_logits"]).max() <= TOL[strat]
    for i, s in enumerate(st):
        ref = g[f"full_state_{i}"]
        assert s.shape == ref.shape
        assert np.abs(s.astype(np.float32) - ref).max() <= TOL[strat], i
    outs, st = [], None
    for a, b in CHUNKS:
        o, st = m.forward(toks[a:b] if b - a > 1 else toks[a], st)
        outs.append(o.astype(np.float32))
    assert np.abs(np.stack(outs) - g["chunk_logits"]).max() <= TOL[strat]
    for i, s in enumerate(st):
        assert np.abs(s.astype(np.float32) - g[f"chunk_state_{i}"]).max() <= TOL[strat], i
    # chunked evaluation equals the one-shot evaluation at the chunk ends
    for j, (a, b) in enumerate(CHUNKS):
        assert np.abs(outs[j] - g["full_logits"][b - 1]).max() <= 4 * TOL[strat]


@pytest.mark.parametrize("kernel_form", [False, True])
def test_v7_exact_mode_is_the_fp32_model_without_rounding(kernel_form):
    """exact=True evaluates the converted model in fp64.  Under 'cpu fp32' the stored weights are the checkpoint's own,
    so the fp64 evaluation must agree with the fp32 one (pinned above by the reference's run) to fp32 rounding; under
    'cpu fp16' (weights rounded to fp16, arithmetic exact) it must lie within the fp16 tolerance of the reference's
    half-precision logits and closer to the fp32 logits than that all-half run is."""
    g32 = dict(np.load(os.path.join(G, "e2e_v7_cpu_fp32.npz")))
    g16 = dict(np.load(os.path.join(G, "e2e_v7_cpu_fp16.npz")))
    ck = synth.make_checkpoint_v7(seed=CKPT_SEED, **TINY7)
    toks = [int(t) for t in g32["tokens"]]
    e32, st = OracleRWKV7(ck, "cpu fp32", kernel_form=kernel_form, exact=True).forward(toks, None, full_output=True)
    assert e32.dtype == np.float64 and st[1].dtype == np.float64
    assert np.abs(e32 - g32["full_logits"]).max() <= TOL["cpu fp32"]
    for i, s in enumerate(st):
        assert np.abs(s - g32[f"full_state_{i}"]).max() <= TOL["cpu fp32"], i
    e16, _ = OracleRWKV7(ck, "cpu fp16", kernel_form=kernel_form, exact=True).forward(toks, None, full_output=True)
    assert np.abs(e16 - g16["full_logits"]).max() <= TOL["cpu fp16"]
    # only the weights are rounded to fp16 in e16: it is closer to the fp32 model than the all-fp16 run
    assert np.abs(e16 - g32["full_logits"]).mean() < np.abs(g16["full_logits"] - g32["full_logits"]).mean()


def test_deep_embed_with_a_unit_gate_is_the_plain_model():
    """s2 = 0 and s0 = 1 make the DeepEmbed gate 1 for every token: the logits must equal the plain model's."""
    ck = synth.make_checkpoint_v7(seed=5, deep_embed=True, **TINY7)
    for i in range(TINY7["n_layer"]):
        ck[f"blocks.{i}.ffn.s2"] = np.zeros_like(ck[f"blocks.{i}.ffn.s2"])
        ck[f"blocks.{i}.ffn.s0"] = np.ones_like(ck[f"blocks.{i}.ffn.s0"])
    toks = synth.random_tokens(7, TINY7["vocab"], seed=6)
    a, _ = OracleRWKV7(ck, "cpu fp32", deep_embed=True).forward(toks, None, full_output=True)
    b, _ = OracleRWKV7(ck, "cpu fp32").forward(toks, None, full_output=True)
    assert np.array_equal(a, b)
    ck2 = synth.make_checkpoint_v7(seed=5, deep_embed=True, **TINY7)
    c, _ = OracleRWKV7(ck2, "cpu fp32", deep_embed=True).forward(toks, None, full_output=True)
    assert np.abs(c - b).max() > 0.1


def _scalar_wkv7(S, r, w_log, k, v, a, b):
    """cuda/rwkv7.cu:24-52 literally, one float at a time (tiny inputs only)."""
    T, C = r.shape
    H, N = S.shape[0], S.shape[1]
    S = S.astype(np.float64).copy()
    y = np.zeros((T, C))
    for t in range(T):
        for h in range(H):
            for i in range(N):
                sa = sum(a[t, h * N + j] * S[h, i, j] for j in range(N))
                acc = 0.0
                for j in range(N):
                    c = h * N + j
                    S[h, i, j] = S[h, i, j] * np.exp(-np.exp(w_log[t, c])) + k[t, c] * v[t, h * N + i] + sa * b[t, c]
                    acc += S[h, i, j] * r[t, c]
                y[t, h * N + i] = acc
    return y, S


def test_wkv7_forms_agree():
    rng = np.random.Generator(np.random.PCG64(5))
    T, H, N = 6, 2, 8
    C = H * N
    r, k, v = (rng.standard_normal((T, C)).astype(np.float32) for _ in range(3))
    kk = rng.standard_normal((T, C)).astype(np.float32)
    kk /= np.linalg.norm(kk.reshape(T, H, N), axis=-1, keepdims=True).repeat(N, -1).reshape(T, C)
    a = rng.random((T, C)).astype(np.float32)
    zw = rng.uniform(-3, 3, (T, C)).astype(np.float32)
    S0 = rng.standard_normal((H, N, N)).astype(np.float32)
    w_log = (-np.logaddexp(0.0, -zw.astype(np.float64)) - 0.5).astype(np.float32)
    dec = np.exp(-0.606531 * (1.0 / (1.0 + np.exp(-zw.astype(np.float64))))).astype(np.float32)
    y1, S1 = model_v7.wkv7_matrix(S0, r, dec, k, v, kk, a)
    y2, S2 = model_v7.wkv7_kernel(S0, r, w_log, k, v, -kk, kk * a)
    y3, S3 = _scalar_wkv7(S0, r, w_log, k, v, -kk, kk * a)
    for y, S in ((y1, S1), (y2, S2)):
        assert np.abs(y - y3).max() < 2e-5
        assert np.abs(S - S3).max() < 2e-5
    # the rank-1 correction is not a no-op in this test: dropping it changes the result
    y4, _ = model_v7.wkv7_kernel(S0, r, w_log, k, v, 0 * kk, kk * a)
    assert np.abs(y4 - y3).max() > 1e-2


def test_wkv7_reduces_to_linear_attention():
    """With a = 0 the update is S = S * w + v k^T, whose closed form after T steps from S = 0 is
    sum_t (prod_{s>t} w_s) v_t k_t^T."""
    rng = np.random.Generator(np.random.PCG64(6))
    T, H, N = 5, 1, 4
    C = H * N
    r, k, v = (rng.standard_normal((T, C)).astype(np.float32) for _ in range(3))
    w_log = rng.uniform(-2, 0, (T, C)).astype(np.float32)
    dec = np.exp(-np.exp(w_log.astype(np.float64)))
    zero = np.zeros((T, C), np.float32)
    y, S = model_v7.wkv7_kernel(np.zeros((H, N, N), np.float32), r, w_log, k, v, zero, zero)
    ref = np.zeros((N, N))
    for t in range(T):
        ref = ref * dec[t][None, :] + np.outer(v[t], k[t])
    assert np.abs(S[0] - ref).max() < 1e-5
    assert np.abs(y[-1] - ref @ r[-1]).max() < 1e-5


def test_normalize_heads():
    rng = np.random.Generator(np.random.PCG64(7))
    x = rng.standard_normal((3, 128)).astype(np.float32)
    y = model_v7.normalize_heads(x, 2)
    assert np.allclose(np.linalg.norm(y.reshape(3, 2, 64), axis=-1), 1.0, atol=1e-6)
    assert np.allclose(y[:, :64] * np.linalg.norm(x[:, :64], axis=-1, keepdims=True), x[:, :64], atol=1e-6)

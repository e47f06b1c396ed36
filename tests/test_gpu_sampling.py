"""Device sampling step (rwkv_sample_logits through chatrwkv_amd.sampling) against the oracle's restatement of
rwkv/utils.py:55-88, 103-123."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import sampling as osamp  # noqa: E402

pytestmark = pytest.mark.gpu
G = os.path.join(ROOT, "tests", "golden")
DEV = "cuda:0"


def logits_for(case_index, vocab, scale):
    rng = np.random.Generator(np.random.PCG64([case_index, 0x5A11]))
    return (rng.standard_normal(vocab) * scale).astype(np.float32)


def _boundary_margin(x, top_p, temperature):
    """Distance of top_p from the nearest cumulative sum of the sorted probabilities: a cut closer than fp32
    summation noise may legitimately land one entry to either side."""
    if temperature == 0 or top_p <= 0:
        return 1.0
    p = np.sort(osamp.softmax32(x).astype(np.float64))[::-1]
    return float(np.abs(np.cumsum(p) - top_p).min())


def _check_probs(got, ref, margin):
    kept_g, kept_r = got > 0, ref > 0
    if margin > 1e-5:
        assert np.array_equal(kept_g, kept_r), (kept_g.sum(), kept_r.sum())
    else:
        assert abs(int(kept_g.sum()) - int(kept_r.sum())) <= 1
    both = kept_g & kept_r
    np.testing.assert_allclose(got[both], ref[both], rtol=2e-4, atol=1e-12)


def test_filter_matches_oracle_on_golden_cases():
    from chatrwkv_amd.sampling import Sampler
    g = np.load(os.path.join(G, "sampler.npz"))
    for ci, (V, scale, temp, top_p, top_k) in enumerate(g["cases"]):
        V = int(V)
        x = logits_for(ci, V, float(scale))
        s = Sampler(V, device=DEV)
        xt = torch.from_numpy(x).to(DEV)
        ref = osamp.filter_probs(x, temperature=float(temp), top_p=float(top_p), top_k=int(top_k)).astype(np.float64)
        margin = _boundary_margin(x, float(top_p), float(temp))
        for u in (0.0, 0.137, 0.5, 0.731, 0.9999):
            tok = int(s.sample(xt, float(temp), float(top_p), int(top_k), u=u, penalties=False))
            got = s.probs.cpu().numpy().astype(np.float64)
            _check_probs(got, ref, margin)
            # the draw: inverse CDF of the device's own filtered vector, recomputed on the host in fp64
            cdf = np.cumsum(got)
            want = osamp.choose(got, u)
            if tok != want:  # fp32 running sums on the device: only an entry adjacent in the CDF may differ
                t = u * cdf[-1]
                assert got[tok] > 0 and abs(cdf[tok] - got[tok] - t) <= 1e-5 * cdf[-1] + 1e-12 or abs(cdf[want] - t) <= 1e-5 * cdf[-1], \
                    (ci, u, tok, want)
            assert ref[tok] > 0 or margin <= 1e-5


def test_temperature_zero_is_argmax_and_top_p_zero():
    from chatrwkv_amd.sampling import Sampler, sample_logits
    x = logits_for(77, 50277, 4.0)
    xt = torch.from_numpy(x).to(DEV)
    s = Sampler(50277, device=DEV)
    for u in (0.0, 0.3, 0.99):
        assert int(s.sample(xt, 0.0, 0.85, 0, u=u, penalties=False)) == int(x.argmax())
        assert int(s.sample(xt, 1.0, 0.0, 0, u=u, penalties=False)) == int(x.argmax())
    assert sample_logits(xt, temperature=0) == int(x.argmax())
    # top_p = 1 within rounding of the total: the reference then keeps everything or, if the fp32 cumulative sum
    # stops short of 1, only the largest entry; the kernel follows the same rule on its own total
    s.sample(xt, 1.0, 1.0, 0, u=0.5, penalties=False)
    kept = int((s.probs > 0).sum())
    assert kept in (1, int((osamp.softmax32(x) > 0).sum()))


def test_ban_penalties_and_occurrence_tables():
    from chatrwkv_amd.sampling import Sampler
    V = 1000
    x = logits_for(5, V, 3.0)
    xt = torch.from_numpy(x).to(DEV)
    ban = [int(np.argmax(x)), 3, 999]
    rng = np.random.Generator(np.random.PCG64(9))
    weight = (rng.random(V) > 0.3).astype(np.float32)      # some ids count for nothing, as blanks / digits do
    s = Sampler(V, device=DEV, token_ban=ban, token_weight=torch.from_numpy(weight), seed=1)
    occ = {}
    pres, freq, decay = 0.2, 0.3, 0.9
    for step in range(40):
        u = float(rng.random())
        adj = osamp.apply_penalties(x, ban, occ, pres, freq)
        ref = osamp.filter_probs(adj, temperature=1.1, top_p=0.9, top_k=50).astype(np.float64)
        tok = int(s.sample(xt, 1.1, 0.9, 50, pres, freq, decay, u=u))
        got = s.probs.cpu().numpy().astype(np.float64)
        _check_probs(got, ref, _boundary_margin(adj, 0.9, 1.1))
        assert tok not in ban and got[tok] > 0
        osamp.update_occurrence(occ, tok, float(weight[tok]), decay)
        seen = s.seen.cpu().numpy()
        assert set(np.nonzero(seen)[0]) == set(occ)
        o = s.occurrence.cpu().numpy()
        np.testing.assert_allclose([o[k] for k in occ], [occ[k] for k in occ], rtol=1e-5, atol=1e-6)
    assert len(occ) > 3


def test_generate_ids_on_tiny_model():
    from chatrwkv_amd import synth
    from chatrwkv_amd.model import RWKV
    from chatrwkv_amd.sampling import PIPELINE_ARGS, generate_ids
    ck = synth.make_checkpoint(version=4, n_layer=2, n_embd=128, n_ffn=512, vocab=211, seed=3)
    m = RWKV(ck, "cuda fp16i8", verbose=False)
    ctx = synth.random_tokens(300, 211, seed=1)              # longer than chunk_len: fed in two calls
    args = PIPELINE_ARGS(temperature=1.0, top_p=0.8, token_ban=[0], chunk_len=256)
    a, _ = generate_ids(m, ctx, 24, args, seed=5)
    b, _ = generate_ids(m, ctx, 24, args, seed=5)
    c, _ = generate_ids(m, ctx, 24, args, seed=6)
    assert a == b and len(a) == 24 and all(0 < t < 211 for t in a)
    assert a != c
    # greedy: temperature 0 equals the argmax loop through forward()
    g, _ = generate_ids(m, ctx, 8, PIPELINE_ARGS(temperature=0, alpha_presence=0, alpha_frequency=0), seed=1)
    out, st = None, None
    for i in range(0, len(ctx), 256):
        out, st = m.forward(ctx[i:i + 256], st)
    want = []
    for _ in range(8):
        t = int(out.argmax())
        want.append(t)
        out, st = m.forward([t], st)
    assert g == want
    # stop token: the output ends before it
    stop = a[5]
    cut, _ = generate_ids(m, ctx, 24, PIPELINE_ARGS(temperature=1.0, top_p=0.8, token_ban=[0], token_stop=[stop]), seed=5)
    assert cut == a[:a.index(stop)]


@pytest.mark.parametrize("vocab", [1, 7, 1000, 8192, 50277, 65536, 70001])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_greedy_token(vocab, dtype):
    """rwkv_greedy_token, the temperature-0 draw without penalties (utils.py:56-58), against numpy's argmax (first
    index of the maximum): random logits, the maximum repeated at several indices, NaN and -inf entries, all entries
    equal; fp32 logits and the fp16 logits RWKV-7 returns; the id is written to the tensor given."""
    from chatrwkv_amd import lib, sampling
    x = logits_for(vocab, vocab, 3.0)
    cases = [x.copy()]
    if vocab >= 7:
        y = x.copy(); y[[vocab - 1, vocab // 2, 3]] = 50.0; cases.append(y)            # ties: the lowest index
        y = x.copy(); y[::3] = np.nan; y[1] = -np.inf; cases.append(y)                    # NaN is never chosen
        y = x.copy(); y[vocab - 1] = 60.0; cases.append(y)                                # the last entry
    cases.append(np.full(vocab, -1.25, np.float32))                                       # all equal: index 0
    out = torch.full((1,), -7, dtype=torch.int32, device=DEV)
    for c in cases:
        t = torch.from_numpy(c).to(DEV).to(dtype)
        ref = c.astype(np.float16 if dtype == torch.float16 else np.float32)
        want = int(np.argmax(np.where(np.isnan(ref), -np.inf, ref)))
        got = sampling.greedy_token(t, out)
        assert got is out and int(out) == want, (vocab, int(out), want)
        assert int(sampling.greedy_token(t)) == want
    L = lib.load()
    assert L.rwkv_greedy_token(None, lib.RWKV_DT_F32, 8, out.data_ptr(), None) == -3
    assert L.rwkv_greedy_token(out.data_ptr(), lib.RWKV_DT_F32, 0, out.data_ptr(), None) == -1
    assert L.rwkv_greedy_token(out.data_ptr(), 7, 8, out.data_ptr(), None) == -5

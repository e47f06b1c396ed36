"""The sampling oracle against the reference's own draws (tests/golden/sampler.npz, written by
tests/golden/make_sampler_goldens.py from rwkv/utils.py:55-75) and against hand-worked cases."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import sampling as osamp  # noqa: E402

G = os.path.join(ROOT, "tests", "golden")


def logits_for(case_index, vocab, scale):
    rng = np.random.Generator(np.random.PCG64([case_index, 0x5A11]))
    return (rng.standard_normal(vocab) * scale).astype(np.float32)


def test_oracle_reproduces_reference_draws():
    g = np.load(os.path.join(G, "sampler.npz"))
    for ci, (V, scale, temp, top_p, top_k) in enumerate(g["cases"]):
        x = logits_for(ci, int(V), float(scale))
        p = osamp.filter_probs(x, temperature=float(temp), top_p=float(top_p), top_k=int(top_k))
        p = p / np.sum(p)
        for d in range(int(g["draws"])):
            np.random.seed(1000 * ci + d)
            assert int(np.random.choice(a=len(p), p=p)) == int(g["tokens"][ci, d]), (ci, d)


def test_nucleus_cut_by_hand():
    # probabilities 0.4, 0.3, 0.2, 0.1: cumulative 0.4, 0.7, 0.9, 1.0
    x = np.log(np.array([0.1, 0.4, 0.2, 0.3], dtype=np.float32))
    keep = lambda **kw: set(np.nonzero(osamp.filter_probs(x, **kw))[0])
    assert keep(top_p=0.35) == {1}
    assert keep(top_p=0.65) == {1, 3}            # 0.7 is the first cumulative sum >= 0.65
    assert keep(top_p=0.7 - 1e-4) == {1, 3}
    assert keep(top_p=0.85) == {1, 2, 3}
    assert keep(top_p=0.95) == {0, 1, 2, 3}
    assert keep(top_p=0.95, top_k=2) == {1, 3}   # the two largest
    assert keep(top_p=0.0) == {1}                # the largest alone
    assert keep(temperature=0, top_p=0.99) == {1}
    # ties at the cut are all kept
    y = np.log(np.array([0.25, 0.25, 0.25, 0.25], dtype=np.float32))
    assert set(np.nonzero(osamp.filter_probs(y, top_p=0.3))[0]) == {0, 1, 2, 3}
    # temperature acts on the kept probabilities: p ** (1 / T)
    p = osamp.filter_probs(x, temperature=0.5, top_p=0.65)
    np.testing.assert_allclose(p[[1, 3]], np.array([0.4, 0.3]) ** 2, rtol=1e-5)


def test_penalties_and_occurrence_by_hand():
    out = osamp.apply_penalties(np.zeros(6, np.float32), token_ban=[5], occurrence={2: 3.0, 4: 0.0},
                                alpha_presence=0.2, alpha_frequency=0.1)
    np.testing.assert_allclose(out[:5], [0, 0, -0.5, 0, -0.2], atol=1e-7)  # a seen token with weight 0 still pays presence
    assert out[5] == -np.inf
    occ = {}
    osamp.update_occurrence(occ, 7, 1.0, 0.5)
    osamp.update_occurrence(occ, 7, 1.0, 0.5)
    osamp.update_occurrence(occ, 3, 0.0, 0.5)
    assert occ == {7: 0.75, 3: 0.0}              # ((1 * .5) + 1) * .5, and a zero-weight entry


def test_choose_inverse_cdf():
    p = np.array([0.0, 2.0, 0.0, 1.0, 1.0])
    assert [osamp.choose(p, u) for u in (0.0, 0.49, 0.5, 0.74, 0.75, 0.999)] == [1, 1, 3, 3, 4, 4]

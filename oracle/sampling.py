"""CPU restatement of the reference's sampling step (test infrastructure: only tests, the smoke
check and the benchmark's CPU leg may import this package).

Follows rwkv_pip_package/src/rwkv/utils.py:
  sample_logits  55-88   (the numpy branch, 63-75; the torch branch 77-88 computes the same filter)
  penalties      103-106 (token ban, presence / frequency penalty over the occurrence table)
  occurrence     112-123 (decay, then add the token's weight)

`filter_probs` returns the probability vector the reference hands to its random draw (un-normalised
in the torch branch, normalised in the numpy branch: same distribution); `choose` is an inverse-CDF
draw for a given uniform number, so that a device implementation fed the same number can be checked
exactly (the reference's own draw uses numpy / torch generators, whose streams no other
implementation can reproduce).
"""
import numpy as np


def softmax32(logits):
    """F.softmax(logits.float(), dim=-1) (utils.py:59)."""
    x = np.asarray(logits, dtype=np.float32)
    e = np.exp(x - x.max())
    return (e / e.sum(dtype=np.float32)).astype(np.float32)


def filter_probs(logits, temperature=1.0, top_p=0.85, top_k=0):
    """utils.py:55-73: temperature 0 means top_p 0; nucleus cut at the first sorted probability whose
    cumulative sum reaches top_p (probabilities below that value are zeroed, ties kept); the top_k
    largest kept; then probs ** (1 / temperature).  Not normalised."""
    if temperature == 0:
        temperature = 1.0
        top_p = 0
    probs = softmax32(logits)
    top_k = int(top_k)
    sorted_ids = np.argsort(probs)
    sorted_probs = probs[sorted_ids][::-1]
    cumulative_probs = np.cumsum(sorted_probs)
    cutoff = float(sorted_probs[np.argmax(cumulative_probs >= top_p)])
    probs[probs < cutoff] = 0
    if top_k < len(probs) and top_k > 0:
        probs[sorted_ids[:-top_k]] = 0
    if temperature != 1.0:
        probs = probs ** (1.0 / temperature)
    return probs


def apply_penalties(out, token_ban=(), occurrence=None, alpha_presence=0.0, alpha_frequency=0.0):
    """utils.py:103-106, on a copy."""
    out = np.array(out, dtype=np.float32, copy=True)
    for n in token_ban:
        out[n] = -np.inf
    for n, v in (occurrence or {}).items():
        out[n] -= (alpha_presence + v * alpha_frequency)
    return out


def update_occurrence(occurrence, token, weight=1.0, alpha_decay=1.0):
    """utils.py:112-123 (the weight is 0 for tokens that decode to blanks / digits, else 1)."""
    for k in occurrence:
        occurrence[k] *= alpha_decay
    occurrence[token] = occurrence[token] + weight if token in occurrence else weight
    return occurrence


def choose(probs, u):
    """Index i with cdf[i-1] <= u * total < cdf[i] over the entries in index order (zero entries are
    never chosen)."""
    p = np.asarray(probs, dtype=np.float64)
    cdf = np.cumsum(p)
    i = int(np.searchsorted(cdf, u * cdf[-1], side="right"))
    i = min(i, len(p) - 1)
    while p[i] == 0 and i > 0:
        i -= 1
    return i

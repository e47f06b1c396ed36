"""Sampling step after the hot path, on the device: the reference's ``PIPELINE.sample_logits`` and the
logit adjustments of ``PIPELINE.generate`` (rwkv_pip_package/src/rwkv/utils.py:10-20, 55-88, 90-135), without a
tokenizer (ids in, ids out) and without copying logits to the host.

``sample_logits`` has the reference's name, arguments and return value.  ``Sampler`` keeps the reference's
``occurrence`` dict as dense device tables, so that a generation loop is  forward -> sample -> forward  with
the token staying on the GPU; ``generate_ids`` is that loop with the semantics of ``PIPELINE.generate``.
The random number of a draw comes from a torch generator on the device (one uniform per token).
"""
import torch

from . import lib as _lib


class PIPELINE_ARGS:
    """Same fields and defaults as the reference's PIPELINE_ARGS (utils.py:10-20)."""

    def __init__(self, temperature=1.0, top_p=0.85, top_k=0, alpha_frequency=0.2, alpha_presence=0.2,
                 alpha_decay=0.996, token_ban=(), token_stop=(), chunk_len=256):
        self.temperature = temperature
        self.top_p = top_p
        self.top_k = top_k
        self.alpha_frequency = alpha_frequency
        self.alpha_presence = alpha_presence
        self.alpha_decay = alpha_decay
        self.token_ban = list(token_ban)
        self.token_stop = list(token_stop)
        self.chunk_len = chunk_len


def _stream():
    return torch.cuda.current_stream().cuda_stream


class Sampler:
    """Device-resident sampling state for one sequence.

    token_weight: optional fp32 [V] tensor, the weight a drawn id adds to its occurrence count (the
    reference uses 0 for ids whose text is a blank or a digit and 1 otherwise, utils.py:116-119)."""

    def __init__(self, vocab, device="cuda:0", token_ban=(), token_weight=None, seed=None):
        if not torch.cuda.is_available():
            raise _lib.RwkvHipError("chatrwkv_amd.sampling needs a ROCm GPU; there is no CPU path")
        self.L = _lib.load()
        self.V = int(vocab)
        self.device = torch.device(device)
        self.seen = torch.zeros(self.V, dtype=torch.uint8, device=self.device)
        self.occurrence = torch.zeros(self.V, dtype=torch.float32, device=self.device)
        self.ban = torch.tensor(list(token_ban), dtype=torch.int32, device=self.device) if len(token_ban) else None
        self.weight = None if token_weight is None else token_weight.to(self.device, torch.float32).contiguous()
        self.probs = torch.empty(self.V, dtype=torch.float32, device=self.device)
        self.token = torch.zeros(1, dtype=torch.int32, device=self.device)
        self.u = torch.zeros(1, dtype=torch.float32, device=self.device)
        self.gen = torch.Generator(device=self.device)
        if seed is not None:
            self.gen.manual_seed(int(seed))

    def reset(self):
        self.seen.zero_()
        self.occurrence.zero_()

    def sample(self, logits, temperature=1.0, top_p=0.85, top_k=0, alpha_presence=0.0, alpha_frequency=0.0,
               alpha_decay=1.0, u=None, penalties=True):
        """One draw.  Returns the int32 device tensor [1] holding the id (valid until the next call);
        ``self.probs`` then holds the filtered probabilities.  ``u``: a float or a device tensor to use
        instead of a fresh uniform number."""
        if logits.dtype != torch.float32 or not logits.is_cuda or logits.numel() != self.V:
            raise _lib.RwkvHipError("sample() takes the fp32 logits [vocab] on the GPU")
        logits = logits.contiguous()
        if u is None:
            self.u.uniform_(generator=self.gen)
        elif isinstance(u, torch.Tensor):
            self.u.copy_(u.reshape(1))
        else:
            self.u.fill_(float(u))
        seen = self.seen.data_ptr() if penalties else None
        occ = self.occurrence.data_ptr() if penalties else None
        rc = self.L.rwkv_sample_logits(
            logits.data_ptr(), self.V, float(temperature), float(top_p), int(top_k),
            self.ban.data_ptr() if self.ban is not None else None, 0 if self.ban is None else self.ban.numel(),
            seen, occ, self.weight.data_ptr() if (self.weight is not None and penalties) else None,
            float(alpha_presence), float(alpha_frequency), float(alpha_decay),
            self.u.data_ptr(), self.probs.data_ptr(), self.token.data_ptr(), _stream())
        _lib.check(rc, "rwkv_sample_logits")
        return self.token


def greedy_token(logits, out=None):
    """The temperature-0 draw of sample_logits (utils.py:56-58) without penalties, i.e. ``logits.argmax()``, as one
    launch: returns the int32 device tensor [1] with the index of the largest logit (``out`` if given), which the
    next ``forward`` takes as its token without a copy to the host."""
    if logits.dtype not in (torch.float32, torch.float16) or not logits.is_cuda or logits.dim() != 1 or not logits.is_contiguous():
        raise _lib.RwkvHipError("greedy_token() takes the contiguous fp32 or fp16 logits [vocab] on the GPU")
    if out is None:
        out = torch.empty(1, dtype=torch.int32, device=logits.device)
    dt = _lib.RWKV_DT_F32 if logits.dtype == torch.float32 else _lib.RWKV_DT_F16
    _lib.check(_lib.load().rwkv_greedy_token(logits.data_ptr(), dt, logits.numel(), out.data_ptr(), _stream()), "rwkv_greedy_token")
    return out


def sample_logits(logits, temperature=1.0, top_p=0.85, top_k=0, generator_seed=None):
    """PIPELINE.sample_logits (utils.py:55-88): returns the drawn id as a Python int."""
    s = Sampler(logits.numel(), device=logits.device, seed=generator_seed)
    return int(s.sample(logits.float(), temperature, top_p, top_k, penalties=False))


def generate_ids(model, ctx_tokens, token_count=100, args=None, state=None, token_weight=None, seed=None,
                 stop_check_every=1):
    """PIPELINE.generate (utils.py:90-135) on token ids: feeds ``ctx_tokens`` in chunks of args.chunk_len, then
    draws ``token_count`` ids with ban / presence / frequency penalties and decaying occurrence counts.
    The drawn id stays on the device between steps.  Stop tokens are looked for every ``stop_check_every``
    steps (one host synchronisation each) and the output is cut at the first one; with the default of 1 the
    loop ends before the stop token is fed, as in the reference, larger values save synchronisations but the
    returned state has then seen the ids drawn after the stop token.  Returns (ids, state)."""
    args = args or PIPELINE_ARGS()
    V = model.w["head.weight"].shape[1] if hasattr(model, "w") else None
    tokens = list(ctx_tokens)
    out = None
    while len(tokens) > 0:
        out, state = model.forward(tokens[:args.chunk_len], state)
        tokens = tokens[args.chunk_len:]
    V = out.numel() if V is None else V
    smp = Sampler(V, device=out.device, token_ban=args.token_ban, token_weight=token_weight, seed=seed)
    drawn = torch.empty(token_count, dtype=torch.int32, device=out.device)
    stop = set(int(t) for t in args.token_stop)
    n = 0
    for i in range(token_count):
        tok = smp.sample(out, args.temperature, args.top_p, args.top_k, args.alpha_presence, args.alpha_frequency,
                         args.alpha_decay)
        drawn[i:i + 1].copy_(tok)
        n = i + 1
        if stop and (n % stop_check_every == 0 or n == token_count):
            ids = drawn[:n].tolist()
            hit = [j for j, t in enumerate(ids) if t in stop]
            if hit:
                return ids[:hit[0]], state
        if n < token_count:
            out, state = model.forward(tok, state)
    return drawn[:n].tolist(), state

"""Oracle: RWKV-7 (``RWKV_x070``) loading and forward, in numpy.

Test infrastructure only (see oracle/__init__.py).

``OracleRWKV7(checkpoint, strategy)`` restates ``RWKV_x070.__init__`` (model.py:224-282),
``forward_one`` / ``forward_seq`` (model.py:336-363, 457-487), the time mix
``RWKV_x070_TMix_one`` / ``_seq`` (model.py:492-572) and the channel mix
``RWKV_x070_CMix_one`` / ``_seq`` (model.py:597-608), and with ``deep_embed=True`` the DeepEmbed variant the
reference selects with ``RWKV_DE_VERSION=1``: the merge of the embedding residual into ``ffn.s_emb``
(model.py:274-277) and the gated channel mix (model.py:578-594).

Strategies: '<device> fp32' runs every operation in fp32; '<device> fp16' keeps activations and
weights in numpy float16, which rounds after every elementwise operation as torch does on fp16
tensors, with fp32 accumulation inside contractions and fp32 for the state and the decay.

The state recurrence exists twice in the reference and both forms are restated here:
  ``wkv7_matrix``  the torch form of model.py:509-512 and 563-568 (outer products rounded to the
                   activation dtype, state cast to it for the read-out);
  ``wkv7_kernel``  the per-row form of cuda/rwkv7.cu:24-52 (fp32 throughout, output rounded once),
                   fed with the log-decay of model.py:537.
They agree to rounding; ``kernel_form`` picks which one sequence mode uses (the reference uses the
kernel when RWKV_CUDA_ON=1, model.py:518-542).  One-token mode always uses the matrix form.
"""
import numpy as np

from . import ops
from .ops import f16, f32, f64

_TRANSPOSED = ('key.weight', 'value.weight', 'receptance.weight', 'output.weight', 'head.weight')


def _np(t):
    return t.detach().cpu().numpy() if hasattr(t, 'detach') else np.asarray(t)


def _acc(dtype):
    """Accumulation / state type beside an activation type: fp32, or fp64 in the exact evaluation."""
    return f64 if dtype == f64 else f32


def _mm(a, b):
    """``a @ b`` on tensors of one dtype: fp32 accumulation, result in that dtype (fp64 throughout in the
    exact evaluation)."""
    F = _acc(a.dtype)
    return (a.astype(F) @ b.astype(F)).astype(a.dtype)


def _sigmoid(x):
    return ops.sigmoid(x)


def _tanh(x):
    return np.tanh(x.astype(f64)).astype(x.dtype)


def normalize_heads(x, H):
    """F.normalize(x.view(T, H, N), dim=-1, p=2) (model.py:503, 532): x / max(||x||, eps) with the norm
    held in x.dtype; eps = 1e-12 (it underflows to 0 in fp16)."""
    T, C = x.shape
    x3 = x.reshape(T, H, C // H)
    n = np.sqrt((x3.astype(f64) ** 2).sum(axis=-1, keepdims=True)).astype(x.dtype)
    n = np.maximum(n, x.dtype.type(1e-12))
    return (x3 / n).reshape(T, C)


def wkv7_matrix(S, r, w, k, v, kk, a):
    """model.py:509-512 (one token) and 563-568 (the same in a loop over T).

    S [H, N(value), N(key)] fp32; r, k, v, kk, a [T, C] in the activation dtype; w [T, C] fp32 decay in
    (0, 1).  Returns y [T, C] in the activation dtype and the new S."""
    T, C = r.shape
    H = S.shape[0]
    N = C // H
    A = r.dtype
    F = _acc(A)
    S = S.astype(F).copy()
    y = np.empty((T, C), dtype=A)
    for t in range(T):
        vk = (v[t].reshape(H, N, 1) * k[t].reshape(H, 1, N)).astype(A)
        ab = ((-kk[t]).reshape(H, N, 1) * (kk[t] * a[t]).astype(A).reshape(H, 1, N)).astype(A)
        S = (S * w[t].reshape(H, 1, N) + np.einsum('him,hmj->hij', S, ab.astype(F), dtype=F)
             + vk.astype(F)).astype(F)
        y[t] = np.einsum('hij,hj->hi', S.astype(A).astype(F), r[t].reshape(H, N).astype(F),
                         dtype=F).astype(A).reshape(C)
    return y, S


def wkv7_kernel(S, r, w_log, k, v, a, b):
    """cuda/rwkv7.cu:24-52: thread i owns row i of the head's state.  Per token
        sa_i = sum_j a_j S_ij ;  S_ij = S_ij * exp(-exp(w_j)) + k_j v_i + sa_i b_j ;  y_i = sum_j S_ij r_j
    r, w_log, k, v, a, b [T, C] (any float dtype, widened to fp32 on load); y is rounded to r.dtype."""
    T, C = r.shape
    H = S.shape[0]
    N = C // H
    F = _acc(r.dtype)
    S = S.astype(F).copy()
    y = np.empty((T, C), dtype=r.dtype)
    for t in range(T):
        r_, k_, v_, a_, b_ = (x[t].astype(F).reshape(H, N) for x in (r, k, v, a, b))
        dec = np.exp(-np.exp(w_log[t].astype(F))).reshape(H, 1, N)
        sa = np.einsum('hij,hj->hi', S, a_, dtype=F)
        S = (S * dec + v_[:, :, None] * k_[:, None, :] + sa[:, :, None] * b_[:, None, :]).astype(F)
        y[t] = np.einsum('hij,hj->hi', S, r_, dtype=F).reshape(C).astype(r.dtype)
    return y, S


class OracleRWKV7:
    def __init__(self, checkpoint, strategy, kernel_form=False, deep_embed=False, exact=False):
        """exact=True: the weights are converted as ``strategy`` says (the same stored fp16 / fp32 values,
        the embedding table normalised and rounded as the loader does), then every operation of the
        forward pass runs in fp64 with no rounding: the value that both half-precision evaluations
        approximate."""
        dev, dt = strategy.split(' ')                                 # model.py:234-243
        if dt not in ('fp16', 'fp32'):
            raise ValueError("oracle supports '<device> fp16' and '<device> fp32' for RWKV-7")
        A = self.atype = f16 if dt == 'fp16' else f32
        self.kernel_form = kernel_form
        self.exact = bool(exact)
        z = {}
        src = {k: _np(v) for k, v in checkpoint.items()}
        self.n_head, self.head_size = src['blocks.0.att.r_k'].shape    # model.py:247
        self.vocab, self.n_embd = src['emb.weight'].shape
        self.n_layer = 0
        for k, t in src.items():                                      # model.py:255-264
            lid = int(k.split('.')[1]) if 'blocks.' in k else 0
            self.n_layer = max(self.n_layer, lid + 1)
            if any(s in k for s in _TRANSPOSED):
                t = t.T
            t = np.squeeze(t)
            if k.endswith('att.r_k'):
                t = t.reshape(-1)
            z[k] = np.ascontiguousarray(t).astype(A)
        # model.py:272: the embedding absorbs ln0, computed on the already-converted table
        z['emb.weight'] = ops.layer_norm(z['emb.weight'], z['blocks.0.ln0.weight'], z['blocks.0.ln0.bias'])
        self.deep_embed = bool(deep_embed)
        if self.deep_embed:                                            # model.py:274-277
            for i in range(self.n_layer):
                p = f'blocks.{i}.ffn.'
                z[p + 's_emb.weight'] = z[p + 's_emb.weight'] + _mm(z['emb.weight'], z[p + 's_emb_x.weight'].T)
        if self.exact:
            z = {k: t.astype(f64) for k, t in z.items()}
            self.atype = f64
        self.z = z

    def generate_zero_state(self):
        """model.py:284-290."""
        C, H, N = self.n_embd, self.n_head, self.head_size
        st = []
        for _ in range(self.n_layer):
            st += [np.zeros(C, self.atype), np.zeros((H, N, N), _acc(self.atype)), np.zeros(C, self.atype)]
        return st

    # ------------------------------------------------------------------ blocks
    def _tmix(self, i, x, x_prev, v_first, S, seq):
        """model.py:492-572.  x [T, C] is the LayerNorm output; returns (out, new x_prev, S, v_first)."""
        z, p = self.z, f'blocks.{i}.att.'
        H, A = self.n_head, self.atype
        one = A(1)
        xx = np.concatenate([x_prev[None, :], x[:-1]], axis=0) - x
        xr, xw, xk, xv, xa, xg = (x + xx * z[p + 'x_' + c] for c in 'rwkvag')
        r = _mm(xr, z[p + 'receptance.weight'])
        w = _mm(_tanh(_mm(xw, z[p + 'w1'])), z[p + 'w2'])
        k = _mm(xk, z[p + 'key.weight'])
        v = _mm(xv, z[p + 'value.weight'])
        a = _sigmoid(z[p + 'a0'] + _mm(_mm(xa, z[p + 'a1']), z[p + 'a2']))
        g = _mm(_sigmoid(_mm(xg, z[p + 'g1'])), z[p + 'g2'])
        kk = normalize_heads(k * z[p + 'k_k'], H)
        k = k * (one + (a - one) * z[p + 'k_a'])
        if i == 0:
            v_first = v
        else:
            v = v + (v_first - v) * _sigmoid(z[p + 'v0'] + _mm(_mm(xv, z[p + 'v1']), z[p + 'v2']))
        zw = z[p + 'w0'] + w
        if seq and self.kernel_form:
            # model.py:537-538: log-decay in the activation dtype, the kernel applies exp(-exp(.))
            z64 = zw.astype(f64)
            w_log = ((-np.logaddexp(0.0, -z64)).astype(A) - A(0.5)).astype(A)
            y, S = wkv7_kernel(S, r, w_log, k, v, -kk, (kk * a).astype(A))
        else:
            # model.py:507, 562
            F = _acc(A)
            dec = np.exp(F(-0.606531) * _sigmoid(zw.astype(F))).astype(F)
            y, S = wkv7_matrix(S, r, dec, k, v, kk, a)
        y = ops.group_norm(y, H, z[p + 'ln_x.weight'], z[p + 'ln_x.bias'])  # eps 64e-5 (model.py:514)
        T, C = y.shape
        rk = (r * k * z[p + 'r_k']).reshape(T, H, -1).astype(_acc(A)).sum(axis=-1, keepdims=True).astype(A)
        y = y + (rk * v.reshape(T, H, -1)).reshape(T, C)
        return _mm(y * g, z[p + 'output.weight']), x[-1], S, v_first

    def _cmix(self, i, x, x_prev, toks=None):
        """model.py:597-608; with DeepEmbed model.py:578-594: the squared-relu keys of token t are scaled by
        ((x_t @ s1) @ E_t) @ s2 + s0, E_t the 32 x 32 matrix stored in row token_t of ffn.s_emb."""
        z, p = self.z, f'blocks.{i}.ffn.'
        xx = np.concatenate([x_prev[None, :], x[:-1]], axis=0) - x
        k = x + xx * z[p + 'x_k']
        k = ops.relu_sq(_mm(k, z[p + 'key.weight']))
        if self.deep_embed:
            T = x.shape[0]
            E = z[p + 's_emb.weight'][np.asarray(toks, dtype=np.int64)].reshape(T, 32, 32)
            sv = _mm(x, z[p + 's1'])                                                     # [T, 32]
            F = _acc(x.dtype)
            ss = np.einsum('ti,tij->tj', sv.astype(F), E.astype(F)).astype(x.dtype)        # [T, 32]
            k = k * (_mm(ss, z[p + 's2']) + z[p + 's0'])
        return _mm(k, z[p + 'value.weight']), x[-1]

    # ------------------------------------------------------------------ forward
    def forward(self, idx, state, full_output=False):
        """model.py:292-302, 336-363, 457-487.  Returns (logits in the activation dtype, state)."""
        if state is None:
            state = self.generate_zero_state()
        z = self.z
        one = not isinstance(idx, (list, tuple)) or len(idx) == 1
        toks = [int(idx)] if not isinstance(idx, (list, tuple)) else [int(t) for t in idx]
        x = z['emb.weight'][np.asarray(toks, dtype=np.int64)]
        v_first = None
        for i in range(self.n_layer):
            b = f'blocks.{i}.'
            xx = ops.layer_norm(x, z[b + 'ln1.weight'], z[b + 'ln1.bias'])
            xx, state[3 * i], state[3 * i + 1], v_first = self._tmix(i, xx, state[3 * i], v_first,
                                                                    state[3 * i + 1], not one)
            x = x + xx
            xx = ops.layer_norm(x, z[b + 'ln2.weight'], z[b + 'ln2.bias'])
            xx, state[3 * i + 2] = self._cmix(i, xx, state[3 * i + 2], toks)
            x = x + xx
        if one or not full_output:
            x = x[-1:]
        x = ops.layer_norm(x, z['ln_out.weight'], z['ln_out.bias'])
        x = _mm(x, z['head.weight'])
        if one or not full_output:
            x = x[0]
        return x, state

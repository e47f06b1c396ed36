"""Oracle: checkpoint conversion and ``forward`` of the reference, in numpy.

Test infrastructure only (see oracle/__init__.py).

``OracleRWKV(checkpoint, strategy)`` restates ``RWKV.__init__`` (model.py:613-903:
version detection, weight transforms, uint8 quantisation) and ``RWKV.forward``
(model.py:1443-1677) for RWKV-4, 5.0, 5.1, 5.2 and 6.0.  Supported strategies are the
single-segment ones:

  'cpu fp32', 'cpu fp32i8'    the arithmetic the reference runs on CPU: fp32 everywhere,
                              RESCALE_LAYER = 0 (model.py:634).  'cpu fp32i8' is the CPU
                              baseline path: every matmul dequantises the whole matrix
                              per call (model.py:91-97).
  'cpu fp16'                  the reference's pure-torch functions on half tensors (what it runs
                              with RWKV_CUDA_ON=0): the same rounding points as 'cuda fp16' except
                              that a float product is rounded to fp16 before any widening
                              (model.py:163); RESCALE_LAYER = 6.  Exists so that the reference
                              itself, run on the CPU, pins where the fp16 path rounds.
  'cuda fp16', 'cuda fp16i8'  emulation of the GPU path: fp16 activations, fp32 WKV, fp32
                              accumulation in every contraction, roundings where the
                              reference's CUDA path rounds, RESCALE_LAYER = 6.

Weights keep the reference's names (``blocks.0.att.key.weight`` and its ``_mx/_rx/_my/_ry``
companions) so converted dicts can be compared key by key with the reference's.
"""
import os
import re

import numpy as np

from . import ops, quant
from .ops import Mat, f16, f32

_SEGMENT = re.compile(r"^ *(cuda(?::0)?|cpu) (fp16|fp32)(i8)?(?: \*(\d+))? *$")


def plan_wtypes(strategy, n_layer):
    """Weight type of each of the n_layer + 1 slots (the last holds ln_out + head) for a chain of segments
    ``device dtype[i8] [*N]`` on ONE device with ONE activation dtype: the slot allocation of
    model.py:694-750 restricted to what the oracle emulates (no streaming, no second device).  Segments with a
    count take that many slots in order, the segments without one share the rest equally, and what is
    still left goes to the last segment.  Returns (device, activation, [is_uint8 per slot])."""
    segs = []
    for part in strategy.split('->'):
        m = _SEGMENT.match(part)
        if not m:
            raise ValueError("oracle supports chains of 'cpu|cuda fp16|fp32[i8] [*N]' segments")
        segs.append((m.group(1).replace(':0', ''), m.group(2), bool(m.group(3)), int(m.group(4)) if m.group(4) else None))
    if len({(d, a) for d, a, _, _ in segs}) != 1:
        raise ValueError("oracle emulates one device and one activation dtype")
    slots = n_layer + 1
    counts = [c or 0 for _, _, _, c in segs]
    dealt = 0
    for i, c in enumerate(counts):                                    # model.py:709-722
        if segs[i][3] is None:
            continue
        dealt += c
        if dealt >= slots:
            counts[i] += slots - dealt
            for j in range(i + 1, len(counts)):
                counts[j] = 0
            dealt = slots
            break
    open_segs = [i for i, s in enumerate(segs) if s[3] is None]
    if dealt < slots and open_segs:                                   # model.py:723-735
        left = len(open_segs)
        for i in open_segs:
            counts[i] = (slots - dealt) // left
            dealt += counts[i]
            left -= 1
    if dealt < slots:
        counts[-1] += slots - dealt
    kinds = []
    for (dev, at, i8, _), c in zip(segs, counts):
        kinds += [i8] * c
    return segs[0][0], segs[0][1], kinds[:slots]

_MATRIX_KEYS = ('key.weight', 'value.weight', 'receptance.weight', 'gate.weight',
                'output.weight', 'head.weight')


def _np(t):
    return t.detach().cpu().numpy() if hasattr(t, 'detach') else np.asarray(t)


class OracleRWKV:
    def __init__(self, checkpoint, strategy, rescale_layer=None, cache_dequant=None, exact=False):
        """exact=True: the weights are converted as ``strategy`` says (same uint8 matrices, same stored scale
        and mix vectors, same rescale), then every step of forward is evaluated in fp64 with no rounding:
        the value both the reference's fp16 path and any emulation of it approximate."""
        self.strategy = strategy
        n_layer = 1 + max(int(k.split('.')[1]) for k in checkpoint if k.startswith('blocks.'))
        self.device, at, self.slot_u8 = plan_wtypes(strategy, n_layer)
        self.atype = f32 if at == 'fp32' else f16
        self.wtype = np.uint8 if all(self.slot_u8) else self.atype      # of a uniform model
        # model.py:631-634
        if rescale_layer is None:
            env = os.environ.get("RWKV_RESCALE_LAYER")
            rescale_layer = int(env) if env not in (None, '') else (6 if at == 'fp16' else 0)
        self.rescale_layer = rescale_layer
        # the CPU baseline path dequantises per call; the emulation may cache
        self.cache = (self.device != 'cpu') if cache_dequant is None else cache_dequant
        self._convert({k: _np(v) for k, v in checkpoint.items()})
        if exact:
            self.atype = np.float64
            self.w = {k: (v if v.dtype == np.uint8 else v.astype(np.float64)) for k, v in self.w.items()}

    @classmethod
    def random_converted_v4(cls, n_layer, n_embd, n_ffn, vocab, seed=0, emb_rows=16):
        """A 'cpu fp32i8' RWKV-4 oracle whose *converted* weights are filled directly with uniform
        random bytes and plausible scales, skipping the (slow, CPU) quantizer.  For timing the CPU
        path only: its speed does not depend on the weight values."""
        self = object.__new__(cls)
        self.device, self.atype, self.wtype = 'cpu', f32, np.uint8
        self.rescale_layer, self.cache = 0, False
        self.n_embd = self.n_att = n_embd
        self.n_ffn, self.n_layer, self.version, self.n_head = n_ffn, n_layer, 4, 0
        rng = np.random.Generator(np.random.PCG64(seed))
        C, F, V = n_embd, n_ffn, vocab
        w = {'emb.weight': rng.standard_normal((emb_rows, C), dtype=f32)}

        def qmat(name, N, M):
            w[name] = rng.integers(0, 256, size=(N, M), dtype=np.uint8)
            w[name + '_mx'] = (rng.standard_normal(M, dtype=f32) * f32(0.01))
            w[name + '_rx'] = (rng.random(M, dtype=f32) * f32(0.01) + f32(0.005))
            w[name + '_my'] = (rng.standard_normal((N, 1), dtype=f32) * f32(0.01))
            w[name + '_ry'] = (rng.random((N, 1), dtype=f32) * f32(0.03) + f32(0.03))

        for i in range(n_layer):
            p = f'blocks.{i}.'
            for ln in ('ln1', 'ln2'):
                w[p + ln + '.weight'], w[p + ln + '.bias'] = np.ones(C, f32), np.zeros(C, f32)
            w[p + 'att.time_decay'] = -np.exp(rng.uniform(-6, -1, C)).astype(f32)
            w[p + 'att.time_first'] = rng.uniform(-1, 1, C).astype(f32)
            for m in 'kvr':
                w[p + 'att.time_mix_' + m] = rng.random(C, dtype=f32)
            for m in 'kr':
                w[p + 'ffn.time_mix_' + m] = rng.random(C, dtype=f32)
            for name in ('key', 'value', 'receptance', 'output'):
                qmat(p + f'att.{name}.weight', C, C)
            qmat(p + 'ffn.key.weight', C, F)
            qmat(p + 'ffn.receptance.weight', C, C)
            qmat(p + 'ffn.value.weight', F, C)
        w['ln_out.weight'], w['ln_out.bias'] = np.ones(C, f32), np.zeros(C, f32)
        qmat('head.weight', C, V)
        self.w, self._mats = w, {}
        return self

    # ------------------------------------------------------------------ conversion
    def _convert(self, w):
        # model.py:658-680
        self.n_embd = w['emb.weight'].shape[1]
        self.n_att = w['blocks.0.att.key.weight'].shape[0]
        self.n_ffn = w['blocks.0.ffn.key.weight'].shape[0]
        self.n_layer = 0
        self.version = 4
        self.n_head = 0
        for x in w:
            lid = int(x.split('.')[1]) if 'blocks.' in x else 0
            self.n_layer = max(self.n_layer, lid + 1)
            if 'ln_x' in x:
                self.version = max(5, self.version)
            if 'gate.weight' in x:
                self.version = max(5.1, self.version)
            if int(self.version) == 5 and 'att.time_decay' in x:
                self.n_head = w[x].shape[0]
                if w[x].ndim > 1 and w[x].shape[1] > 1:
                    self.version = max(5.2, self.version)
            if 'time_maa' in x:
                self.version = max(6, self.version)
            if int(self.version) == 6 and 'time_faaaa' in x:
                self.n_head = w[x].shape[0]
        A, R = self.atype, self.rescale_layer

        # model.py:754-760: embedding absorbs ln0
        w['emb.weight'] = ops.layer_norm(w['emb.weight'].astype(f32),
                                         w['blocks.0.ln0.weight'], w['blocks.0.ln0.bias'])
        del w['blocks.0.ln0.weight'], w['blocks.0.ln0.bias']
        # model.py:764-771
        real_time_first = any('.time_faaaa' in k for k in w)
        w = {k.replace('.time_faaaa', '.time_first'): v for k, v in w.items()}

        out = {}
        for x, t in w.items():
            lid = int(x.split('.')[1]) if 'blocks.' in x else 0
            t = t.astype(f32)
            if R > 0 and ('att.output.weight' in x or 'ffn.value.weight' in x):
                t = t / f32(2 ** int(lid // R))                      # model.py:785-789
            if '.time_' in x:
                t = np.squeeze(t)                                    # model.py:791-792
            if any(s in x for s in _MATRIX_KEYS):
                t = t.T                                              # model.py:793-794 -> [in, out]
            if '.time_decay' in x and '_w' not in x:                 # model.py:796-804
                if self.version == 4:
                    t = -np.exp(t)
                elif int(self.version) == 5:
                    t = np.exp(-np.exp(t)).reshape(-1, 1, 1)
                    if self.version == 5.2:
                        t = t.reshape(self.n_head, -1, 1)
                else:
                    t = t.reshape(self.n_head, -1, 1)
                out[x] = t.astype(f32)
            elif '.time_first' in x:                                 # model.py:805-814
                if self.version != 4:
                    t = (t if real_time_first else np.exp(t)).reshape(-1, 1, 1)
                    if self.version in (5.2, 6):
                        t = t.reshape(self.n_head, -1, 1)
                out[x] = t.astype(f32)
            elif '.ln_x' in x:                                       # model.py:815-816
                out[x] = t.astype(f32)
            elif t.ndim == 2 and 'emb' not in x and '_w1' not in x and '_w2' not in x:
                # the slot of the tensor's layer decides; ln_out / head sit in the last slot (model.py:776-778)
                if not self.slot_u8[lid if 'blocks.' in x else self.n_layer]:   # model.py:819-820
                    out[x] = np.ascontiguousarray(t).astype(self.wtype)
                else:                                                # model.py:821-847
                    q, mx, rx, my, ry = quant.quantize_u8(t, atype=A)
                    out[x] = q
                    out[x + '_mx'], out[x + '_rx'] = mx, rx
                    out[x + '_my'], out[x + '_ry'] = my, ry
            else:
                out[x] = t.astype(A)                                 # model.py:849
        self.w = out
        self._mats = {}

    def mat(self, name):
        m = self._mats.get(name)
        if m is None:
            w = self.w
            if w[name].dtype == np.uint8:
                m = Mat(w[name], w[name + '_mx'], w[name + '_rx'], w[name + '_my'], w[name + '_ry'])
            else:
                m = Mat(w[name])
            self._mats[name] = m
        return m

    def _mm(self, a, name, output_dtype=None):
        # on 'cpu' the reference has no native GEMM: a float product is rounded to the activation dtype first
        return ops.matmul(a, self.mat(name), self.atype, output_dtype, cache=self.cache,
                          via_atype=self.device == 'cpu')

    # ------------------------------------------------------------------ state
    def init_state(self):
        """model.py:1448-1471."""
        L, C, A = self.n_layer, self.n_embd, self.atype
        st = []
        for i in range(L):
            if self.version == 4:
                st += [np.zeros(C, A), np.zeros(self.n_att, f32), np.zeros(self.n_att, f32),
                       np.full(self.n_att, -1e30, f32), np.zeros(C, A)]
            else:
                N = self.n_att // self.n_head
                ts = self.w.get(f'blocks.{i}.att.time_state')            # model.py:765-768, 1467-1468
                kv = (np.zeros((self.n_head, N, N), f32) if ts is None else
                      np.ascontiguousarray(ts.reshape(self.n_head, N, N).transpose(0, 2, 1)).astype(f32))
                st += [np.zeros(C, A), kv, np.zeros(C, A)]
        return st

    # ------------------------------------------------------------------ blocks
    @staticmethod
    def _shift(sx, xx):
        """Token shift (model.py:997, 1060): row t sees the normalised activation of t-1."""
        return np.concatenate([sx[None, :], xx[:-1]], axis=0)

    def _ffn(self, x, sx, i):
        """Channel mix.  v4/v5: model.py:984-1004; v6: model.py:1007-1029."""
        w, p = self.w, f'blocks.{i}.'
        one = self.atype(1)
        xx = ops.layer_norm(x, w[p + 'ln2.weight'], w[p + 'ln2.bias'])
        prev = self._shift(sx, xx)
        if self.version >= 6:
            d = prev - xx
            kx = xx + d * w[p + 'ffn.time_maa_k']
            rx = xx + d * w[p + 'ffn.time_maa_r']
        else:
            mk, mr = w[p + 'ffn.time_mix_k'], w[p + 'ffn.time_mix_r']
            kx = xx * mk + prev * (one - mk)
            rx = xx * mr + prev * (one - mr)
        r = ops.sigmoid(self._mm(rx, p + 'ffn.receptance.weight'))
        vx = ops.relu_sq(self._mm(kx, p + 'ffn.key.weight'))
        out = r * self._mm(vx, p + 'ffn.value.weight')
        return x + out, xx[-1]

    def _att_v4(self, x, sx, aa, bb, pp, i):
        """RWKV-4 time mix.  model.py:1034-1086 and 1346-1360."""
        w, p = self.w, f'blocks.{i}.'
        a = p + 'att.'
        one = self.atype(1)
        xx = ops.layer_norm(x, w[p + 'ln1.weight'], w[p + 'ln1.bias'])
        prev = self._shift(sx, xx)
        mk, mv, mr = w[a + 'time_mix_k'], w[a + 'time_mix_v'], w[a + 'time_mix_r']
        kx = xx * mk + prev * (one - mk)
        vx = xx * mv + prev * (one - mv)
        rx = xx * mr + prev * (one - mr)
        r = ops.sigmoid(self._mm(rx, a + 'receptance.weight'))
        k = self._mm(kx, a + 'key.weight', output_dtype=f32)
        v = self._mm(vx, a + 'value.weight', output_dtype=f32)
        y, aa, bb, pp = ops.wkv4(k, v, w[a + 'time_first'], w[a + 'time_decay'], aa, bb, pp)
        out = self._mm(r * y.astype(self.atype), a + 'output.weight')
        return x + out, xx[-1], aa, bb, pp

    def _att_v56(self, x, sx, S, i):
        """RWKV-5.0 / 5.1 / 5.2 / 6.0 time mix.  model.py:1091-1340, 1363-1439."""
        w, p = self.w, f'blocks.{i}.'
        a = p + 'att.'
        A = self.atype
        f32 = np.float64 if A == np.float64 else np.float32          # exact evaluation: nothing narrower than fp64
        one = A(1)
        T = x.shape[0]
        H = self.n_head
        N = self.n_att // H
        xx = ops.layer_norm(x, w[p + 'ln1.weight'], w[p + 'ln1.bias'])
        prev = self._shift(sx, xx)
        gated = self.version >= 5.1
        if self.version >= 6:
            d = prev - xx
            xxx = xx + d * w[a + 'time_maa_x']
            xxx = np.tanh(ops.small_matmul(xxx, w[a + 'time_maa_w1'], A).astype(f32)).astype(A)
            xxx = xxx.reshape(T, 5, -1).transpose(1, 0, 2)                       # [5, T, 32]
            mm = np.stack([ops.small_matmul(xxx[j], w[a + 'time_maa_w2'][j], A) for j in range(5)])
            wx = xx + d * (w[a + 'time_maa_w'] + mm[0])
            kx = xx + d * (w[a + 'time_maa_k'] + mm[1])
            vx = xx + d * (w[a + 'time_maa_v'] + mm[2])
            rx = xx + d * (w[a + 'time_maa_r'] + mm[3])
            gx = xx + d * (w[a + 'time_maa_g'] + mm[4])
        else:
            mix = lambda name: xx * w[a + name] + prev * (one - w[a + name])
            kx, vx, rx = mix('time_mix_k'), mix('time_mix_v'), mix('time_mix_r')
            if gated:
                gx = mix('time_mix_g')
        # output_dtype fp32 (model.py:1283-1285, 1369-1371).  With fp16 weights the reference's native GEMM writes the
        # fp32 sums unrounded (gemm_fp16_cublas.cpp:31-33) and so does this emulation; the reference's pure-torch
        # 'cpu fp16' run (the goldens) and the HIP path round r, k, v to fp16 once before widening them: one extra
        # fp16 rounding, inside the 2e-2 logit tolerance of the tests that compare the three.
        r = self._mm(rx, a + 'receptance.weight', output_dtype=f32).reshape(T, H, N)
        k = self._mm(kx, a + 'key.weight', output_dtype=f32).reshape(T, H, N)
        v = self._mm(vx, a + 'value.weight', output_dtype=f32).reshape(T, H, N)
        if gated:
            g = ops.silu(self._mm(gx, a + 'gate.weight'))
        if self.version >= 6:
            # model.py:1286-1287, 1324-1325
            lo = np.tanh(ops.small_matmul(wx, w[a + 'time_decay_w1'], A).astype(f32)).astype(A)
            lo = ops.small_matmul(lo, w[a + 'time_decay_w2'], A).astype(f32)
            dec = w[a + 'time_decay'].reshape(1, H, N) + lo.reshape(T, H, N)
            dec = np.exp(-np.exp(dec.astype(f32))).astype(f32)
        else:
            dec = w[a + 'time_decay'].reshape(H, -1)
        out, S = ops.wkv56(r, k, v, dec, w[a + 'time_first'].reshape(H, -1), S)
        out = ops.group_norm(out.reshape(T, H * N), H, w[a + 'ln_x.weight'], w[a + 'ln_x.bias'])
        out = out.astype(A)
        if gated:
            out = out * g
        out = self._mm(out, a + 'output.weight')
        return x + out, xx[-1], S

    # ------------------------------------------------------------------ forward
    def forward(self, tokens, state, full_output=False):
        """model.py:1443-1677.  tokens: list of ints; returns (logits fp32, state list)."""
        w, A = self.w, self.atype
        if state is None:
            state = self.init_state()
        seq_mode = len(tokens) > 1
        x = w['emb.weight'][np.asarray(tokens, dtype=np.int64)].astype(A)
        for i in range(self.n_layer):
            if self.version == 4:
                o = 5 * i
                x, state[o], state[o + 1], state[o + 2], state[o + 3] = self._att_v4(
                    x, state[o], state[o + 1], state[o + 2], state[o + 3], i)
                x, state[o + 4] = self._ffn(x, state[o + 4], i)
            else:
                o = 3 * i
                x, state[o], state[o + 1] = self._att_v56(x, state[o], state[o + 1], i)
                x, state[o + 2] = self._ffn(x, state[o + 2], i)
            if self.rescale_layer > 0 and (i + 1) % self.rescale_layer == 0:
                x = x / A(2)                                         # model.py:1660-1662
        if seq_mode and not full_output:
            x = x[-1:]
        x = ops.layer_norm(x, w['ln_out.weight'], w['ln_out.bias'])
        m = self.mat('head.weight')
        if m.quantized:
            x = ops.matmul(x, m, A, cache=self.cache)               # model.py:1672-1675
        else:
            x = ops.matmul(x, m, A, output_dtype=A, cache=self.cache)  # model.py:1670
        x = x.astype(f32)
        if not (seq_mode and full_output):
            x = x[0]
        return x, state

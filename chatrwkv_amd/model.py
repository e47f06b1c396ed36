"""``RWKV(model, strategy)`` / ``model.forward(tokens, state)`` on one MI355X.

Drop-in for the class of the same name in rwkv_pip_package/src/rwkv/model.py:612-1677 for
the strategies 'cuda fp16i8', 'cuda fp16' and chains of the two on one GPU ('cuda fp16i8 *20 -> cuda
fp16'): same constructor and forward signatures, same
state-list layout, dtypes and initial values (model.py:1448-1471), same chunked-prefill
behaviour (len(tokens) == 1 -> one-token mode, > 1 -> sequence mode, state carried
between calls).  Everything numeric runs in librwkv_hip.so; PyTorch provides device
memory, streams and graph capture only.

Differences a caller can observe, all deliberate:
  * the embedding table lives on the GPU (the reference keeps it on the CPU and copies one
    row per token, model.py:852-853, 1475);
  * weight matrices keep the reference's shape [in, out] but are stored input-contiguous
    (strides (1, in)), the orientation the kernels stream;
  * every state tensor is updated in place (the reference's CUDA sequence path already does
    this for aa, bb, pp); ``copy.deepcopy(state)`` snapshots a state as in v2/chat.py:166-179;
  * ``model`` may also be an in-memory ``{name: tensor}`` dict (tensors on CPU or GPU), and
    ``tokens`` of a one-token call may be a 1-element integer tensor on the GPU, which keeps a
    greedy decode loop free of host synchronisation; such an id cannot be checked without one, so the
    kernels clamp it into [0, vocab) (ids given as Python ints raise IndexError when out of range).
"""
import collections
import ctypes
import gc
import os
import types

import torch

from . import lib as _lib
from . import ops as _ops
from . import strategy as _strategy
from .state import StateList

_MATRIX_KEYS = ('key.weight', 'value.weight', 'receptance.weight', 'gate.weight', 'output.weight', 'head.weight')
# the tensors a streamed slot keeps in pinned host memory (model.py:854)
_STREAMED_KEYS = ('key.weight', 'value.weight', 'receptance.weight', 'output.weight')


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _load_checkpoint(path):
    """The checkpoint dict of ``path`` on the CPU, read without executing anything from the file
    (``weights_only=True``).  Memory-mapped where the file allows it; files in torch's older, non-zip
    serialization, which the reference's plain ``torch.load`` (model.py:641) accepts, cannot be mapped and are
    read whole."""
    try:
        return torch.load(path, map_location='cpu', weights_only=True, mmap=True)
    except RuntimeError as e:
        if 'mmap' not in str(e):
            raise
        return torch.load(path, map_location='cpu', weights_only=True)


class RWKV:
    def __init__(self, model, strategy, verbose=True, convert_and_save_and_exit=None):
        prxxx = (lambda *a, **k: print(*a, **k)) if verbose else (lambda *a, **k: None)
        self._stream_order = _lib.StreamOrder()
        self.args = types.SimpleNamespace()
        args = self.args
        args.strategy_string = _strategy.normalize(strategy)          # ValueError on a bad string
        try:                                                          # model.py:631-634
            self.RESCALE_LAYER = int(os.environ["RWKV_RESCALE_LAYER"])
        except (KeyError, ValueError):
            self.RESCALE_LAYER = 6 if 'fp16' in args.strategy_string else 0

        if isinstance(model, dict):
            args.MODEL_NAME = '<dict>'
            w = dict(model)
        else:
            args.MODEL_NAME = model.strip()
            if not args.MODEL_NAME.endswith('.pth'):
                args.MODEL_NAME += '.pth'
            prxxx(f'Loading {args.MODEL_NAME} ...')
            w = _load_checkpoint(args.MODEL_NAME)

        converted = '_strategy' in w                                  # model.py:646-656
        if converted:
            assert convert_and_save_and_exit is None
            assert w['_strategy'] == args.strategy_string
            assert float(w['_version']) >= 0.7
            assert w['_rescale_layer'] == self.RESCALE_LAYER
            for k in ('_strategy', '_version', '_rescale_layer'):
                del w[k]

        # shape / version detection (model.py:658-680)
        args.n_embd = w['emb.weight'].shape[1]
        args.n_att = w['blocks.0.att.key.weight'].shape[1 if converted else 0]
        args.n_ffn = w['blocks.0.ffn.key.weight'].shape[1 if converted else 0]
        args.n_layer = 0
        args.n_head = 0
        self.version = 4
        for x in list(w.keys()):
            layer_id = int(x.split('.')[1]) if ('blocks.' in x) else 0
            args.n_layer = max(args.n_layer, layer_id + 1)
            if 'ln_x' in x:
                self.version = max(5, self.version)
            if 'gate.weight' in x:
                self.version = max(5.1, self.version)
            if int(self.version) == 5 and 'att.time_decay' in x:
                args.n_head = w[x].shape[0]
                if len(w[x].shape) > 1 and w[x].shape[1] > 1:
                    self.version = max(5.2, self.version)
            if 'time_maa' in x:
                self.version = max(6, self.version)
            if int(self.version) == 6 and 'time_faaaa' in x:
                args.n_head = w[x].shape[0]
        prxxx(f'Model detected: v{self.version:.1f}')

        self.strategy = _strategy.plan(args.strategy_string, args.n_layer)
        for n, s in enumerate(self.strategy):
            prxxx(f"{n}-{s.device}-{str(s.atype).replace('torch.', '')}-{str(s.wtype).replace('torch.', '')}"
                  f"{'-stream' if s.stream else ''}", end=' ')
        prxxx()
        self._wkind = _strategy.require_single_gpu(self.strategy)    # NotImplementedError otherwise
        if self.version not in (4, 5, 5.1, 5.2, 6):
            raise NotImplementedError(f"RWKV v{self.version} is not supported")
        if int(self.version) in (5, 6) and args.n_att // max(args.n_head, 1) != 64:
            raise NotImplementedError("RWKV-5/6 kernels are built for head size 64")
        if args.n_att != args.n_embd:
            raise NotImplementedError("n_att != n_embd")
        _lib.load()                                                   # fail early and loudly
        if not torch.cuda.is_available():
            raise _lib.RwkvHipError("no ROCm GPU visible: chatrwkv_amd has no CPU path")
        self.device = torch.device('cuda:0')
        torch.cuda.set_device(self.device)

        with torch.no_grad():
            self.w = self._convert(w, converted, prxxx)
            if convert_and_save_and_exit:
                self._save_converted(convert_and_save_and_exit, prxxx)
                raise SystemExit(0)                                   # model.py:903
            self._plan_staging()
            if self.version == 4:
                self._build_descriptors()
            else:
                self._build_descriptors_v56()
        self._graphs = collections.OrderedDict()
        self._seq_ws = None
        gc.collect()
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ weights
    def _convert(self, w, converted, prxxx):
        """Weight transforms of model.py:754-849, executed on the GPU: LayerNorm of the embedding,
        rescale, quantisation.  The small time_* vectors follow the reference on the CPU."""
        args, dev, R = self.args, self.device, self.RESCALE_LAYER
        L = _lib.load()
        st = torch.cuda.current_stream().cuda_stream
        out = {}
        real_time_first = any('.time_faaaa' in k for k in w)          # model.py:764-771
        if real_time_first:
            w = {k.replace('.time_faaaa', '.time_first'): v for k, v in w.items()}
        args.time_state = any('.time_state' in k for k in w)
        if not converted:
            emb = w['emb.weight'].to(device=dev, dtype=torch.float32).contiguous()
            ln_w = w['blocks.0.ln0.weight'].to(device=dev, dtype=torch.float32).contiguous()
            ln_b = w['blocks.0.ln0.bias'].to(device=dev, dtype=torch.float32).contiguous()
            emb16 = torch.empty(emb.shape, dtype=torch.float16, device=dev)
            _lib.check(L.rwkv_layernorm_f32_f16(emb.shape[0], emb.shape[1], emb.data_ptr(), ln_w.data_ptr(),
                                                ln_b.data_ptr(), emb16.data_ptr(), st), "rwkv_layernorm_f32_f16")
            out['emb.weight'] = emb16
            del emb
        for x in list(w.keys()):
            if x in ('blocks.0.ln0.weight', 'blocks.0.ln0.bias') and not converted:
                continue
            if x == 'emb.weight' and not converted:
                continue
            t = w[x]
            layer_id = int(x.split('.')[1]) if ('blocks.' in x) else 0
            is_matrix = (any(s in x for s in _MATRIX_KEYS) and not x.endswith(('_mx', '_rx', '_my', '_ry'))
                         and t.dim() == 2)
            if converted:
                if is_matrix:
                    # reference device layout [in, out] with out contiguous -> input-contiguous
                    out[x] = _ops.to_input_contiguous(t.to(dev))
                    if self.strategy[layer_id if 'blocks.' in x else args.n_layer].stream and x.endswith(_STREAMED_KEYS):
                        out[x] = self._to_pinned(out[x])
                elif x.endswith(('_mx', '_rx', '_my', '_ry')) or 'emb.' in x:
                    out[x] = t.to(dev).contiguous()
                else:
                    out[x] = t.to(dev).contiguous()
                continue
            if is_matrix:
                # the slot of the tensor's layer decides its type; ln_out and head sit in the last slot (model.py:776-778)
                slot = self.strategy[layer_id if 'blocks.' in x else args.n_layer]
                u8 = slot.wtype == torch.uint8
                t = t.to(device=dev, dtype=torch.float32)
                if R > 0 and ('att.output.weight' in x or 'ffn.value.weight' in x):
                    t = t / (2 ** int(layer_id // R))                 # model.py:785-789 (exact scaling)
                # checkpoint orientation [out, in] row-major == logical [in, out] input-contiguous
                t = t.contiguous()
                if u8:
                    q, mx, rx, my, ry = _ops.quantize_u8(t.t(), scale_dtype=torch.float16, input_contiguous=True)
                    out[x], out[x + '_mx'], out[x + '_rx'], out[x + '_my'], out[x + '_ry'] = q, mx, rx, my, ry
                else:
                    out[x] = t.to(torch.float16).t()
                del t
                if slot.stream and x.endswith(_STREAMED_KEYS):            # model.py:854-858
                    out[x] = self._to_pinned(out[x])
                continue
            t = t.detach().to('cpu')
            if '.time_' in x:
                t = t.squeeze()
            if '.time_decay' in x and '_w' not in x:                  # model.py:796-804
                if self.version == 4:
                    t = -torch.exp(t.float())
                elif int(self.version) == 5:
                    t = torch.exp(-torch.exp(t.float())).reshape(-1, 1, 1)
                    if self.version == 5.2:
                        t = t.reshape(args.n_head, -1, 1)
                else:
                    t = t.float().reshape(args.n_head, -1, 1)
            elif '.time_first' in x:                                  # model.py:805-814
                if self.version == 4:
                    t = t.float()
                else:
                    t = (t.float() if real_time_first else torch.exp(t.float())).reshape(-1, 1, 1)
                    if self.version in (5.2, 6):
                        t = t.reshape(args.n_head, -1, 1)
            elif '.ln_x' in x:                                        # model.py:815-816
                t = t.float()
            else:
                t = t.to(torch.float16)                               # model.py:849
            out[x] = t.contiguous().to(dev)
        torch.cuda.synchronize()
        return out

    @staticmethod
    def _to_pinned(t):
        """An input-contiguous [N, M] device matrix as a pinned host tensor of the same shape and strides."""
        host = torch.empty((t.shape[1], t.shape[0]), dtype=t.dtype, pin_memory=True)   # allocated pinned
        host.copy_(t.t())
        return host.t()

    def _save_converted(self, path, prxxx):
        """model.py:894-903: the converted dict in the reference's own layout ([in, out] matrices
        with the output index contiguous) so that either implementation can load the file."""
        if not path.endswith('.pth'):
            path += '.pth'
        sd = {}
        for k, v in self.w.items():
            v = v.detach()
            is_matrix = any(s in k for s in _MATRIX_KEYS) and not k.endswith(('_mx', '_rx', '_my', '_ry'))
            sd[k] = (v.contiguous() if is_matrix else v).cpu()
        sd['_strategy'] = self.args.strategy_string
        sd['_rescale_layer'] = self.RESCALE_LAYER
        sd['_version'] = '0.7'
        prxxx(f'Saving to {path}...')
        torch.save(sd, path)
        prxxx('Converted and saved. Now this will exit.')

    def _mat(self, name):
        w = self.w
        t = w[name]
        N, M = t.shape
        assert t.stride(0) == 1, name
        m = _lib.RwkvMat()
        m.w, m.ld, m.N, m.M = t.data_ptr(), t.stride(1), N, M
        if not t.is_cuda:
            m.w = self._stage_ptr[name]       # a streamed matrix: the kernels read its place in the staging buffer
        if t.dtype == torch.uint8:
            m.mx, m.rx = w[name + '_mx'].data_ptr(), w[name + '_rx'].data_ptr()
            m.my, m.ry = w[name + '_my'].data_ptr(), w[name + '_ry'].data_ptr()
        return m

    def _plan_staging(self):
        """Streamed layers (model.py:854-858, 1526-1530, 1617-1620): their key / value / receptance / output matrices
        live in pinned host memory and are copied into one of TWO device staging buffers, each sized for the largest
        such layer; streamed layers alternate between the two, so that the next streamed layer's copy (on a copy
        stream of its own) runs under the current layer's kernels.  Every streamed layer's descriptors point into
        its buffer."""
        self._stage_ptr, self._stage_plan, sizes = {}, {}, {}
        for name, t in self.w.items():
            if isinstance(t, torch.Tensor) and not t.is_cuda and t.dim() == 2 and name.endswith(_STREAMED_KEYS):
                layer = int(name.split('.')[1])
                off = sizes.get(layer, 0)
                nbytes = t.numel() * t.element_size()
                self._stage_plan.setdefault(layer, []).append((name, t.t().reshape(-1).view(torch.uint8), off, nbytes))
                sizes[layer] = off + ((nbytes + 255) & ~255)
        self._staging = None
        if sizes:
            nslot = 2 if len(sizes) > 1 else 1
            self._staging = [torch.empty(max(sizes.values()), dtype=torch.uint8, device=self.device) for _ in range(nslot)]
            self._stage_slot = {layer: k % nslot for k, layer in enumerate(sorted(self._stage_plan))}
            for layer, items in self._stage_plan.items():
                for name, _, off, _ in items:
                    self._stage_ptr[name] = self._staging[self._stage_slot[layer]].data_ptr() + off
            self._copy_stream = torch.cuda.Stream(device=self.device)        # default priority
            self._slot_free = [None] * nslot       # recorded on the compute stream after the kernels that read the slot
            self._streamed_order = sorted(self._stage_plan)
        # the calls one forward pass is made of: runs of resident layers, and every streamed layer alone
        self._segments, i, L = [], 0, self.args.n_layer
        while i < L:
            if i in self._stage_plan:
                self._segments.append((i, i + 1))
                i += 1
            else:
                j = i
                while j < L and j not in self._stage_plan:
                    j += 1
                self._segments.append((i, j))
                i = j

    def _enqueue_stage_copy(self, layer):
        """The host-to-device copies of one streamed layer on the copy stream, once the kernels that last read its
        staging buffer have finished; returns the event its kernels must wait for."""
        slot = self._stage_slot[layer]
        cs = self._copy_stream
        if self._slot_free[slot] is not None:
            cs.wait_event(self._slot_free[slot])
        buf = self._staging[slot]
        with torch.cuda.stream(cs):
            for _, host, off, nbytes in self._stage_plan[layer]:
                buf[off:off + nbytes].copy_(host, non_blocking=True)
            filled = torch.cuda.Event()
            filled.record(cs)
        return filled

    def _run_segments(self, call):
        """call() once per segment with the model's layer range set.  A streamed layer's matrices are copied into
        its staging buffer on the copy stream, one streamed layer ahead of the kernels: the copy of the next
        streamed layer is queued before this segment's kernels, waits only for the kernels that last read that
        buffer (two streamed layers back), and this layer's kernels wait for their own copy."""
        m = self._model
        if not self._stage_plan:
            for lb, le in self._segments:
                m.layer_begin, m.layer_end = lb, le
                call()
            m.layer_begin = m.layer_end = 0
            return
        cur = torch.cuda.current_stream()
        order = self._streamed_order
        filled = {order[0]: self._enqueue_stage_copy(order[0])}
        for lb, le in self._segments:
            if lb in self._stage_plan:
                k = order.index(lb)
                if k + 1 < len(order):         # two buffers whenever there are two streamed layers
                    filled[order[k + 1]] = self._enqueue_stage_copy(order[k + 1])
                cur.wait_event(filled.pop(lb))
            m.layer_begin, m.layer_end = lb, le
            call()
            if lb in self._stage_plan:
                ev = torch.cuda.Event()
                ev.record(cur)
                self._slot_free[self._stage_slot[lb]] = ev
        m.layer_begin = m.layer_end = 0

    def _build_descriptors(self):
        a, w = self.args, self.w
        layers = (_lib.RwkvV4Layer * a.n_layer)()
        for i in range(a.n_layer):
            b, at, ff = f'blocks.{i}.', f'blocks.{i}.att.', f'blocks.{i}.ffn.'
            l = layers[i]
            l.ln1_w, l.ln1_b = w[b + 'ln1.weight'].data_ptr(), w[b + 'ln1.bias'].data_ptr()
            l.ln2_w, l.ln2_b = w[b + 'ln2.weight'].data_ptr(), w[b + 'ln2.bias'].data_ptr()
            l.att_mix_k, l.att_mix_v, l.att_mix_r = (w[at + 'time_mix_' + c].data_ptr() for c in 'kvr')
            l.time_decay, l.time_first = w[at + 'time_decay'].data_ptr(), w[at + 'time_first'].data_ptr()
            l.att_key, l.att_value = self._mat(at + 'key.weight'), self._mat(at + 'value.weight')
            l.att_receptance, l.att_output = self._mat(at + 'receptance.weight'), self._mat(at + 'output.weight')
            l.ffn_mix_k, l.ffn_mix_r = w[ff + 'time_mix_k'].data_ptr(), w[ff + 'time_mix_r'].data_ptr()
            l.ffn_key, l.ffn_receptance = self._mat(ff + 'key.weight'), self._mat(ff + 'receptance.weight')
            l.ffn_value = self._mat(ff + 'value.weight')
        m = _lib.RwkvV4Model()
        m.n_layer, m.n_embd, m.n_ffn = a.n_layer, a.n_embd, a.n_ffn
        m.vocab = w['emb.weight'].shape[0]
        m.rescale_layer = self.RESCALE_LAYER
        m.weights_u8 = {'f16': 0, 'u8': 1, 'mixed': 2}[self._wkind]
        m.emb = w['emb.weight'].data_ptr()
        m.ln_out_w, m.ln_out_b = w['ln_out.weight'].data_ptr(), w['ln_out.bias'].data_ptr()
        m.head = self._mat('head.weight')
        m.layers = layers
        self._layers, self._model = layers, m
        L = _lib.load()
        nbytes = L.rwkv_v4_one_workspace(ctypes.byref(m))
        self._one_ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        self._token_dev = torch.zeros(1, dtype=torch.int32, device=self.device)
        self._logits = torch.empty(m.vocab, dtype=torch.float32, device=self.device)

    def _build_descriptors_v56(self):
        """Descriptors for RWKV-5.x / 6.0.  The per-head decay / bonus tensors are flattened to [C]
        (one value per channel; 5.0 / 5.1 broadcast the per-head value), and the RWKV-6 LoRA
        matrices time_maa_w1 / time_decay_w1 / time_decay_w2 are kept input-contiguous."""
        a, w, dev = self.args, self.w, self.device
        C, H = a.n_embd, a.n_head
        N = C // H
        v6 = self.version == 6
        keep = self._keep = []
        layers = (_lib.RwkvV56Layer * a.n_layer)()

        def per_channel(t):
            t = t.to(torch.float32).reshape(H, -1)
            t = t.expand(H, N).contiguous().reshape(C) if t.shape[1] == 1 else t.reshape(C).contiguous()
            keep.append(t)
            return t.data_ptr()

        def kept(t):
            keep.append(t)
            return t.data_ptr()

        for i in range(a.n_layer):
            b, at, ff = f'blocks.{i}.', f'blocks.{i}.att.', f'blocks.{i}.ffn.'
            l = layers[i]
            l.ln1_w, l.ln1_b = w[b + 'ln1.weight'].data_ptr(), w[b + 'ln1.bias'].data_ptr()
            l.ln2_w, l.ln2_b = w[b + 'ln2.weight'].data_ptr(), w[b + 'ln2.bias'].data_ptr()
            if v6:
                for j, c in enumerate('xwkvrg'):
                    l.att_mix[j] = w[at + 'time_maa_' + c].data_ptr()
                l.tm_w1 = kept(w[at + 'time_maa_w1'].t().contiguous())
                l.tm_w2 = kept(w[at + 'time_maa_w2'].contiguous())
                l.td_w1 = kept(w[at + 'time_decay_w1'].t().contiguous())
                l.td_w2 = kept(w[at + 'time_decay_w2'].t().contiguous())
                l.ffn_mix_k, l.ffn_mix_r = w[ff + 'time_maa_k'].data_ptr(), w[ff + 'time_maa_r'].data_ptr()
            else:
                for j, c in enumerate('kvrg' if self.version >= 5.1 else 'kvr'):
                    l.att_mix[j] = w[at + 'time_mix_' + c].data_ptr()
                l.ffn_mix_k, l.ffn_mix_r = w[ff + 'time_mix_k'].data_ptr(), w[ff + 'time_mix_r'].data_ptr()
            l.time_decay = per_channel(w[at + 'time_decay'])
            l.time_first = per_channel(w[at + 'time_first'])
            l.lnx_w, l.lnx_b = w[at + 'ln_x.weight'].data_ptr(), w[at + 'ln_x.bias'].data_ptr()
            l.att_key, l.att_value = self._mat(at + 'key.weight'), self._mat(at + 'value.weight')
            l.att_receptance, l.att_output = self._mat(at + 'receptance.weight'), self._mat(at + 'output.weight')
            if self.version >= 5.1:
                l.att_gate = self._mat(at + 'gate.weight')
            l.ffn_key, l.ffn_receptance = self._mat(ff + 'key.weight'), self._mat(ff + 'receptance.weight')
            l.ffn_value = self._mat(ff + 'value.weight')
        m = _lib.RwkvV56Model()
        m.version_x10 = int(round(self.version * 10))
        m.n_layer, m.n_embd, m.n_ffn, m.n_head = a.n_layer, C, a.n_ffn, H
        m.vocab = w['emb.weight'].shape[0]
        if v6:
            m.lora_maa = w['blocks.0.att.time_maa_w2'].shape[1]
            m.lora_decay = w['blocks.0.att.time_decay_w1'].shape[1]
        m.rescale_layer = self.RESCALE_LAYER
        m.weights_u8 = {'f16': 0, 'u8': 1, 'mixed': 2}[self._wkind]
        m.emb = w['emb.weight'].data_ptr()
        m.ln_out_w, m.ln_out_b = w['ln_out.weight'].data_ptr(), w['ln_out.bias'].data_ptr()
        m.head = self._mat('head.weight')
        m.layers = layers
        self._layers, self._model = layers, m
        self._token_dev = torch.zeros(1, dtype=torch.int32, device=dev)
        self._logits = torch.empty(m.vocab, dtype=torch.float32, device=dev)
        nbytes = _lib.load().rwkv_v56_workspace(ctypes.byref(m), 1)
        self._one_ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)

    # ------------------------------------------------------------------ state
    def _new_state(self):
        if self.version != 4:
            return self._new_state_v56()
        """model.py:1448-1459: per layer [xx fp16 (C), aa, bb fp32 (C), pp fp32 = -1e30, ffn_xx fp16 (C)],
        carved from two flat buffers."""
        a, dev = self.args, self.device
        C, L = a.n_embd, a.n_layer
        f16 = torch.zeros(L * 2 * C, dtype=torch.float16, device=dev)
        f32 = torch.zeros(L * 3 * C, dtype=torch.float32, device=dev)
        st = StateList()
        for i in range(L):
            st.append(f16[(2 * i) * C:(2 * i + 1) * C])
            st.append(f32[(3 * i) * C:(3 * i + 1) * C])
            st.append(f32[(3 * i + 1) * C:(3 * i + 2) * C])
            pp = f32[(3 * i + 2) * C:(3 * i + 3) * C]
            pp.fill_(-1e30)
            st.append(pp)
            st.append(f16[(2 * i + 1) * C:(2 * i + 2) * C])
        st.flat = (f16, f32)
        st.views = list(st)
        return st

    def _new_state_v56(self):
        """model.py:1460-1471: per layer [xx fp16 (C), kv fp32 (H, N, N) laid out [h][key][value], ffn_xx fp16 (C)]."""
        a, dev = self.args, self.device
        C, L, H = a.n_embd, a.n_layer, a.n_head
        N = C // H
        f16 = torch.zeros(L * 2 * C, dtype=torch.float16, device=dev)
        f32 = torch.zeros(L * H * N * N, dtype=torch.float32, device=dev)
        st = StateList()
        for i in range(L):
            st.append(f16[(2 * i) * C:(2 * i + 1) * C])
            kv = f32[i * H * N * N:(i + 1) * H * N * N].view(H, N, N)
            if a.time_state:                                          # model.py:1467-1468
                kv.copy_(self.w[f'blocks.{i}.att.time_state'].transpose(1, 2).to(torch.float32))
            st.append(kv)
            st.append(f16[(2 * i + 1) * C:(2 * i + 2) * C])
        st.flat = (f16, f32)
        st.views = list(st)
        return st

    def _state_desc_v56(self, state):
        a = self.args
        if len(state) != 3 * a.n_layer:
            raise ValueError(f"state must hold {3 * a.n_layer} tensors")
        H = a.n_head
        N = a.n_embd // H
        arr = (_lib.RwkvV56LayerState * a.n_layer)()
        for i in range(a.n_layer):
            xx, kv, fx = state[3 * i:3 * i + 3]
            ok = (xx.is_cuda and xx.dtype == torch.float16 and xx.is_contiguous() and xx.numel() == a.n_embd and
                  fx.is_cuda and fx.dtype == torch.float16 and fx.is_contiguous() and fx.numel() == a.n_embd and
                  kv.is_cuda and kv.dtype == torch.float32 and tuple(kv.shape) == (H, N, N))
            if not ok:
                raise ValueError("state tensors must be GPU tensors with the layout of model.py:1460-1471")
            if not kv.is_contiguous():
                # the reference's CUDA sequence path hands back a transposed view (model.py:1384)
                kv = state[3 * i + 1] = kv.contiguous()
            s = arr[i]
            s.att_xx, s.att_kv, s.ffn_xx = xx.data_ptr(), kv.data_ptr(), fx.data_ptr()
        return arr

    def _state_desc(self, state):
        a = self.args
        if self.version != 4:
            return self._state_desc_v56(state)
        if len(state) != 5 * a.n_layer:
            raise ValueError(f"state must hold {5 * a.n_layer} tensors")
        arr = (_lib.RwkvV4LayerState * a.n_layer)()
        for i in range(a.n_layer):
            xx, aa, bb, pp, fx = state[5 * i:5 * i + 5]
            for t, dt in ((xx, torch.float16), (aa, torch.float32), (bb, torch.float32), (pp, torch.float32),
                          (fx, torch.float16)):
                if not (t.is_cuda and t.dtype == dt and t.is_contiguous() and t.numel() == a.n_embd):
                    raise ValueError("state tensors must be contiguous GPU tensors with the layout of model.py:1448-1459")
            s = arr[i]
            s.att_xx, s.aa, s.bb, s.pp, s.ffn_xx = (t.data_ptr() for t in (xx, aa, bb, pp, fx))
        return arr

    # ------------------------------------------------------------------ forward
    def _launch_one(self, sdesc):
        L = _lib.load()
        st = torch.cuda.current_stream().cuda_stream

        def call():
            if self.version != 4:
                rc = L.rwkv_v56_forward(ctypes.byref(self._model), sdesc, self._token_dev.data_ptr(), 1, 0,
                                        self._logits.data_ptr(), self._one_ws.data_ptr(), self._one_ws.numel(), st)
                _lib.check(rc, "rwkv_v56_forward")
            else:
                rc = L.rwkv_v4_forward_one(ctypes.byref(self._model), sdesc, self._token_dev.data_ptr(),
                                           self._logits.data_ptr(), self._one_ws.data_ptr(), self._one_ws.numel(), st)
                _lib.check(rc, "rwkv_v4_forward_one")
        self._run_segments(call)

    def _forward_one(self, token, state):
        if isinstance(token, torch.Tensor):
            if token.data_ptr() != self._token_dev.data_ptr():   # the caller wrote the id into token_slot: nothing to copy
                self._token_dev.copy_(token.reshape(1), non_blocking=True)
        else:
            # the id travels as a kernel argument of the fill: no host buffer that a later call
            # could overwrite while this one is still queued
            self._token_dev.fill_(int(token))
        use_graph = os.environ.get("RWKV_HIP_GRAPH", "1") != "0"
        key = None
        if use_graph and not self._stage_plan and isinstance(state, StateList) and state.intact():
            key = tuple(t.data_ptr() for t in state.flat)
        if key is None:
            self._launch_one(self._state_desc(state))
            return self._logits.clone(), state
        entry = self._graphs.get(key)
        if entry is None:
            sdesc = self._state_desc(state)
            # warm-up outside capture must not advance the state: run it on a scratch copy
            scratch = self._new_state()
            self._launch_one(self._state_desc(scratch))
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self._launch_one(sdesc)
            entry = (g, sdesc, state.flat)
            self._graphs[key] = entry
            while len(self._graphs) > 8:
                self._graphs.popitem(last=False)
        else:
            self._graphs.move_to_end(key)
        entry[0].replay()
        return self._logits.clone(), state

    def profile_one(self, token, state):
        """One-token step with a HIP event around every kernel launch (rwkv_v4_profile_one).
        Returns (logits, state, ms) with ms[4 * i + j] the j-th launch of layer i and ms[-1] the head."""
        with torch.no_grad():
            if state is None:
                state = self._new_state()
            self._token_dev.fill_(int(token))
            n = 4 * self.args.n_layer + 1
            ms = (ctypes.c_float * n)()
            rc = _lib.load().rwkv_v4_profile_one(ctypes.byref(self._model), self._state_desc(state),
                                                 self._token_dev.data_ptr(), self._logits.data_ptr(),
                                                 self._one_ws.data_ptr(), self._one_ws.numel(),
                                                 torch.cuda.current_stream().cuda_stream, ms, n)
            _lib.check(rc, "rwkv_v4_profile_one")
            return self._logits.clone(), state, list(ms)

    def time_phase(self, phase, reps=4):
        """Mean duration (ms) of one launch of decode phase 0..4 run back to back over all layers
        (rwkv_v4_time_phase), on a scratch state."""
        scratch = self._new_state()
        ms = ctypes.c_float(0)
        self._token_dev.fill_(0)
        logits = torch.empty_like(self._logits)
        rc = _lib.load().rwkv_v4_time_phase(ctypes.byref(self._model), self._state_desc(scratch),
                                            self._token_dev.data_ptr(), logits.data_ptr(), self._one_ws.data_ptr(),
                                            self._one_ws.numel(), torch.cuda.current_stream().cuda_stream,
                                            int(phase), int(reps), ctypes.byref(ms))
        _lib.check(rc, "rwkv_v4_time_phase")
        return float(ms.value)

    def _forward_seq(self, tokens, state, full_output):
        L = _lib.load()
        T = len(tokens)
        tok = torch.tensor(tokens, dtype=torch.int32).to(self.device)
        if self.version != 4:
            nbytes = L.rwkv_v56_workspace(ctypes.byref(self._model), T)
        else:
            nbytes = L.rwkv_v4_seq_workspace(ctypes.byref(self._model), T, int(full_output))
        if self._seq_ws is None or self._seq_ws.numel() < nbytes:
            self._seq_ws = None
            self._seq_ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        V = self._model.vocab
        logits = torch.empty((T, V) if full_output else (V,), dtype=torch.float32, device=self.device)
        fn = L.rwkv_v4_forward_seq if self.version == 4 else L.rwkv_v56_forward
        sdesc, st = self._state_desc(state), torch.cuda.current_stream().cuda_stream

        def call():
            rc = fn(ctypes.byref(self._model), sdesc, tok.data_ptr(), T, int(full_output), logits.data_ptr(),
                    self._seq_ws.data_ptr(), self._seq_ws.numel(), st)
            _lib.check(rc, "forward (sequence mode)")
        self._run_segments(call)
        return logits, state

    @property
    def token_slot(self):
        """The int32 device tensor [1] the one-token step reads its id from.  A sampler that writes the next id
        here (``greedy_token(out, model.token_slot)``, ``Sampler.sample`` followed by a copy) and passes this
        tensor to ``forward`` saves the step its copy of the id."""
        return self._token_dev

    def forward(self, tokens, state, full_output=False):
        """model.py:1443-1677.  Returns (logits fp32 [vocab] or [T, vocab], state)."""
        cur = self._stream_order.before()
        try:
            return self._forward(tokens, state, full_output)
        finally:
            self._stream_order.after(cur)

    def _forward(self, tokens, state, full_output):
        with torch.no_grad():
            if state is None:
                state = self._new_state()
            if isinstance(tokens, torch.Tensor):
                if tokens.numel() == 1:
                    return self._forward_one(tokens if tokens.is_cuda else int(tokens), state)
                tokens = tokens.tolist()
            tokens = [int(t) for t in tokens]
            V = self._model.vocab
            if any(t < 0 or t >= V for t in tokens):
                raise IndexError("token id out of range")
            if len(tokens) == 1:
                return self._forward_one(tokens[0], state)
            return self._forward_seq(tokens, state, full_output)


if os.environ.get('RWKV_V7_ON') == '1':                               # model.py:1679-1680
    from .model_v7 import RWKV_x070
    RWKV = RWKV_x070

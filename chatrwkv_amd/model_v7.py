"""``RWKV_x070(model, strategy)`` / ``model.forward(idx, state, full_output)`` on one MI355X.

Drop-in for the class of the same name in rwkv_pip_package/src/rwkv/model.py:223-487 (the RWKV-7 model
that replaces ``RWKV`` when RWKV_V7_ON=1, model.py:1679-1680) for the strategy 'cuda fp16': same
constructor and forward signatures (``model`` is the path without '.pth', model.py:245), same state
list (per layer: att_x_prev fp16 [C], att_kv fp32 [H, N, N] laid out [head][value][key], ffn_x_prev
fp16 [C]; model.py:284-290), ``idx`` an int, a one-element list (one-token mode) or a longer list
(sequence mode), logits returned in fp16.  Everything numeric runs in librwkv_hip.so
(rwkv_v7_forward); PyTorch provides device memory, streams and graph capture only.

Differences a caller can observe: state tensors are updated in place; ``model`` may also be an
in-memory ``{name: tensor}`` dict; a one-element integer tensor on the GPU is accepted as ``idx``.
The DeepEmbed variant is selected as in the reference, by RWKV_DE_VERSION=1 in the environment when the object is
built (model.py:274-277, 578-594); the checkpoint must then carry the ffn.s_* tensors.  The fp32 / bf16 strategies
are not implemented.
"""
import collections
import ctypes
import gc
import os
import types

import torch

from . import lib as _lib
from .state import StateList

_TRANSPOSED = ('key.weight', 'value.weight', 'receptance.weight', 'output.weight', 'head.weight')


def _pad64(n):
    return (int(n) + 63) // 64 * 64


class RWKV_x070:
    def __init__(self, model, strategy):
        self._stream_order = _lib.StreamOrder()
        self.args = types.SimpleNamespace()
        args = self.args
        ss = strategy.strip().split(' ')                              # model.py:234-243
        if len(ss) != 2 or ss[1] not in ('fp16', 'fp32', 'bf16'):
            raise AssertionError("currently rwkv7 strategy must be: cuda/cpu fp16/fp32/bf16")
        if not ss[0].startswith('cuda') or ss[0] not in ('cuda', 'cuda:0') or ss[1] != 'fp16':
            raise NotImplementedError("chatrwkv_amd runs RWKV-7 under 'cuda fp16' only")
        self.deep_embed = os.environ.get('RWKV_DE_VERSION') == '1'     # model.py:274, 304
        if isinstance(model, dict):
            args.MODEL_NAME = '<dict>'
            w = dict(model)
        else:
            args.MODEL_NAME = model
            w = torch.load(args.MODEL_NAME + '.pth', map_location='cpu', mmap=True, weights_only=True)
        _lib.load()                                                   # fail early and loudly
        if not torch.cuda.is_available():
            raise _lib.RwkvHipError("no ROCm GPU visible: chatrwkv_amd has no CPU path")
        self.device = dev = torch.device('cuda:0')
        torch.cuda.set_device(dev)

        self.n_head, self.head_size = w['blocks.0.att.r_k'].shape     # model.py:247-249
        args.head_size = self.head_size
        args.vocab_size, args.n_embd = w['emb.weight'].shape
        if self.head_size != 64:
            raise NotImplementedError("RWKV-7 kernels are built for head size 64")
        args.n_layer = 0
        z = self.z = {}
        with torch.no_grad():
            for k in list(w.keys()):                                  # model.py:255-264
                layer_id = int(k.split('.')[1]) if ('blocks.' in k) else 0
                args.n_layer = max(args.n_layer, layer_id + 1)
                t = w[k].to(dev).to(torch.float16)
                if any(s in k for s in _TRANSPOSED):
                    # checkpoint orientation [out, in] row-major == logical [in, out] input-contiguous
                    z[k] = t.contiguous().t()
                    continue
                t = t.squeeze()
                if k.endswith('att.r_k'):
                    t = t.flatten()
                z[k] = t.contiguous()
            self.n_embd, self.n_layer = args.n_embd, args.n_layer
            args.n_ffn = z['blocks.0.ffn.key.weight'].shape[1]
            # model.py:272: LayerNorm of the fp16 table with ln0
            L = _lib.load()
            emb32 = z['emb.weight'].float().contiguous()
            ln_w, ln_b = z['blocks.0.ln0.weight'].float(), z['blocks.0.ln0.bias'].float()
            emb16 = torch.empty_like(z['emb.weight'])
            _lib.check(L.rwkv_layernorm_f32_f16(emb32.shape[0], emb32.shape[1], emb32.data_ptr(), ln_w.data_ptr(),
                                                ln_b.data_ptr(), emb16.data_ptr(),
                                                torch.cuda.current_stream().cuda_stream), "rwkv_layernorm_f32_f16")
            torch.cuda.synchronize()
            z['emb.weight'] = emb16
            del emb32
            if self.deep_embed:
                self._merge_deep_embed()
            self._build_descriptors()
        self._graphs = collections.OrderedDict()
        self._seq_ws = None
        gc.collect()
        torch.cuda.empty_cache()

    def _merge_deep_embed(self):
        """model.py:274-277: ffn.s_emb += emb @ ffn.s_emb_x^T per layer (emb already carries ln0), the product
        through the library's fp16 GEMM (fp32 accumulation, rounded to fp16, then the fp16 add)."""
        z, a, L = self.z, self.args, _lib.load()
        st = torch.cuda.current_stream().cuda_stream
        V, C = z['emb.weight'].shape
        for i in range(a.n_layer):
            ff = f'blocks.{i}.ffn.'
            sx = z[ff + 's_emb_x.weight']                              # [1024, C] row-major = [C][1024] input-contiguous
            if tuple(z[ff + 's_emb.weight'].shape) != (V, 1024) or tuple(sx.shape) != (1024, C):
                raise ValueError("DeepEmbed tensors must be ffn.s_emb.weight [vocab, 1024] and ffn.s_emb_x.weight [1024, n_embd]")
            prod = torch.empty((V, 1024), dtype=torch.float16, device=self.device)
            _lib.check(L.rwkv_gemm_f16(V, C, 1024, z['emb.weight'].data_ptr(), C, sx.data_ptr(), 1, C,
                                       prod.data_ptr(), 1024, _lib.RWKV_DT_F16, st), "rwkv_gemm_f16")
            z[ff + 's_emb.weight'] = (z[ff + 's_emb.weight'] + prod).contiguous()
            z[ff + 's1t'] = z[ff + 's1'].t().contiguous()               # [32][C]
            del z[ff + 's_emb_x.weight']
        torch.cuda.synchronize()

    # ------------------------------------------------------------------ descriptors
    def _mat(self, name):
        t = self.z[name]
        N, M = t.shape
        assert t.stride(0) == 1, name
        m = _lib.RwkvMat()
        m.w, m.ld, m.N, m.M = t.data_ptr(), t.stride(1), N, M
        return m

    def _build_descriptors(self):
        """The four LoRA pairs of a layer are concatenated, every rank padded with zeros to a multiple of
        64: first stages as row blocks of one [R][C] matrix (the checkpoint's [C, rank] transposed),
        second stages as column blocks of one [C][R] matrix."""
        a, z, dev = self.args, self.z, self.device
        C = a.n_embd
        keep = self._keep = []

        ranks = [_pad64(z['blocks.0.att.' + n + '1'].shape[1]) for n in 'wa'] + \
                [_pad64(z['blocks.1.att.v1'].shape[1]) if a.n_layer > 1 else 64,
                 _pad64(z['blocks.0.att.g1'].shape[1])]
        layers = (_lib.RwkvV7Layer * a.n_layer)()
        for i in range(a.n_layer):
            b, at, ff = f'blocks.{i}.', f'blocks.{i}.att.', f'blocks.{i}.ffn.'
            l = layers[i]
            l.ln1_w, l.ln1_b = z[b + 'ln1.weight'].data_ptr(), z[b + 'ln1.bias'].data_ptr()
            l.ln2_w, l.ln2_b = z[b + 'ln2.weight'].data_ptr(), z[b + 'ln2.bias'].data_ptr()
            for j, c in enumerate('rwkvag'):
                l.x_mix[j] = z[at + 'x_' + c].data_ptr()
            l.w0, l.a0 = z[at + 'w0'].data_ptr(), z[at + 'a0'].data_ptr()
            l1 = torch.zeros((sum(ranks), C), dtype=torch.float16, device=dev)
            l2 = torch.zeros((C, sum(ranks)), dtype=torch.float16, device=dev)
            off = 0
            for n, rank in zip('wavg', ranks):
                if not (n == 'v' and i == 0):                         # layer 0 ignores v0, v1, v2 (model.py:279-281, 505)
                    t1, t2 = z[at + n + '1'], z[at + n + '2']         # [C, r], [r, C]
                    l1[off:off + t1.shape[1]] = t1.t()
                    l2[:, off:off + t2.shape[0]] = t2.t()
                off += rank
            keep += [l1, l2]
            l.lora1, l.lora2 = l1.data_ptr(), l2.data_ptr()
            if i > 0:
                l.v0 = z[at + 'v0'].data_ptr()
            l.k_k, l.k_a, l.r_k = z[at + 'k_k'].data_ptr(), z[at + 'k_a'].data_ptr(), z[at + 'r_k'].data_ptr()
            l.lnx_w, l.lnx_b = z[at + 'ln_x.weight'].data_ptr(), z[at + 'ln_x.bias'].data_ptr()
            l.att_receptance, l.att_key = self._mat(at + 'receptance.weight'), self._mat(at + 'key.weight')
            l.att_value, l.att_output = self._mat(at + 'value.weight'), self._mat(at + 'output.weight')
            l.ffn_x_k = z[ff + 'x_k'].data_ptr()
            l.ffn_key, l.ffn_value = self._mat(ff + 'key.weight'), self._mat(ff + 'value.weight')
            if self.deep_embed:
                if tuple(z[ff + 's1t'].shape) != (32, C) or tuple(z[ff + 's2'].shape) != (32, a.n_ffn) or \
                        z[ff + 's0'].numel() != a.n_ffn:
                    raise ValueError("DeepEmbed tensors must be ffn.s1 [n_embd, 32], ffn.s2 [32, n_ffn], ffn.s0 [n_ffn]")
                l.de_emb, l.de_s1 = z[ff + 's_emb.weight'].data_ptr(), z[ff + 's1t'].data_ptr()
                l.de_s2, l.de_s0 = z[ff + 's2'].data_ptr(), z[ff + 's0'].data_ptr()
        m = _lib.RwkvV7Model()
        m.n_layer, m.n_embd, m.n_ffn, m.vocab, m.n_head = a.n_layer, C, a.n_ffn, a.vocab_size, self.n_head
        m.lora_w, m.lora_a, m.lora_v, m.lora_g = ranks
        m.emb = z['emb.weight'].data_ptr()
        m.ln_out_w, m.ln_out_b = z['ln_out.weight'].data_ptr(), z['ln_out.bias'].data_ptr()
        m.head = self._mat('head.weight')
        m.layers = layers
        self._layers, self._model = layers, m
        self._token_dev = torch.zeros(1, dtype=torch.int32, device=dev)
        self._logits = torch.empty(m.vocab, dtype=torch.float32, device=dev)
        nbytes = _lib.load().rwkv_v7_workspace(ctypes.byref(m), 1)
        self._one_ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)

    # ------------------------------------------------------------------ state
    def generate_zero_state(self):
        """model.py:284-290, carved from two flat buffers."""
        a, dev = self.args, self.device
        C, L, H, N = a.n_embd, a.n_layer, self.n_head, self.head_size
        f16 = torch.zeros(L * 2 * C, dtype=torch.float16, device=dev)
        f32 = torch.zeros(L * H * N * N, dtype=torch.float32, device=dev)
        st = StateList()
        for i in range(L):
            st.append(f16[(2 * i) * C:(2 * i + 1) * C])
            st.append(f32[i * H * N * N:(i + 1) * H * N * N].view(H, N, N))
            st.append(f16[(2 * i + 1) * C:(2 * i + 2) * C])
        st.flat = (f16, f32)
        st.views = list(st)
        return st

    def _state_desc(self, state):
        a = self.args
        if len(state) != 3 * a.n_layer:
            raise ValueError(f"state must hold {3 * a.n_layer} tensors")
        H, N = self.n_head, self.head_size
        arr = (_lib.RwkvV56LayerState * a.n_layer)()
        for i in range(a.n_layer):
            xx, kv, fx = state[3 * i:3 * i + 3]
            ok = (xx.is_cuda and xx.dtype == torch.float16 and xx.is_contiguous() and xx.numel() == a.n_embd and
                  fx.is_cuda and fx.dtype == torch.float16 and fx.is_contiguous() and fx.numel() == a.n_embd and
                  kv.is_cuda and kv.dtype == torch.float32 and tuple(kv.shape) == (H, N, N) and kv.is_contiguous())
            if not ok:
                raise ValueError("state tensors must be contiguous GPU tensors with the layout of model.py:284-290")
            s = arr[i]
            s.att_xx, s.att_kv, s.ffn_xx = xx.data_ptr(), kv.data_ptr(), fx.data_ptr()
        return arr

    # ------------------------------------------------------------------ forward
    def _launch_one(self, sdesc):
        rc = _lib.load().rwkv_v7_forward(ctypes.byref(self._model), sdesc, self._token_dev.data_ptr(), 1, 0,
                                         self._logits.data_ptr(), self._one_ws.data_ptr(), self._one_ws.numel(),
                                         torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "rwkv_v7_forward")

    @property
    def token_slot(self):
        """The int32 device tensor [1] the one-token step reads its id from.  A sampler that writes the next id
        here (``greedy_token(out, model.token_slot)``, ``Sampler.sample`` followed by a copy) and passes this
        tensor to ``forward`` saves the step its copy of the id."""
        return self._token_dev

    def forward_one(self, idx, state):
        """model.py:336-363."""
        if isinstance(idx, torch.Tensor):
            if idx.data_ptr() != self._token_dev.data_ptr():   # the caller wrote the id into token_slot: nothing to copy
                self._token_dev.copy_(idx.reshape(1), non_blocking=True)
        else:
            idx = int(idx)
            if idx < 0 or idx >= self._model.vocab:
                raise IndexError("token id out of range")
            self._token_dev.fill_(idx)
        use_graph = os.environ.get("RWKV_HIP_GRAPH", "1") != "0"
        key = None
        if use_graph and isinstance(state, StateList) and state.intact():
            key = tuple(t.data_ptr() for t in state.flat)
        if key is None:
            self._launch_one(self._state_desc(state))
            return self._logits.half(), state
        entry = self._graphs.get(key)
        if entry is None:
            sdesc = self._state_desc(state)
            # warm-up outside capture must not advance the state: run it on a scratch copy
            scratch = self.generate_zero_state()
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
        return self._logits.half(), state

    def forward_seq(self, idx, state, full_output=False):
        """model.py:457-487."""
        L = _lib.load()
        T = len(idx)
        V = self._model.vocab
        idx = [int(t) for t in idx]
        if any(t < 0 or t >= V for t in idx):
            raise IndexError("token id out of range")
        tok = torch.tensor(idx, dtype=torch.int32).to(self.device)
        nbytes = L.rwkv_v7_workspace(ctypes.byref(self._model), T)
        if self._seq_ws is None or self._seq_ws.numel() < nbytes:
            self._seq_ws = None
            self._seq_ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        logits = torch.empty((T, V) if full_output else (V,), dtype=torch.float32, device=self.device)
        rc = L.rwkv_v7_forward(ctypes.byref(self._model), self._state_desc(state), tok.data_ptr(), T,
                               int(full_output), logits.data_ptr(), self._seq_ws.data_ptr(), self._seq_ws.numel(),
                               torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "rwkv_v7_forward")
        return logits.half(), state

    def forward(self, idx, state, full_output=False):
        """model.py:292-302."""
        cur = self._stream_order.before()
        try:
            return self._forward(idx, state, full_output)
        finally:
            self._stream_order.after(cur)

    def _forward(self, idx, state, full_output):
        with torch.no_grad():
            if state is None:
                state = self.generate_zero_state()
            if isinstance(idx, torch.Tensor):
                if idx.numel() == 1:
                    return self.forward_one(idx if idx.is_cuda else int(idx), state)
                idx = idx.tolist()
            if type(idx) is list:
                if len(idx) > 1:
                    return self.forward_seq(idx, state, full_output)
                return self.forward_one(idx[0], state)
            return self.forward_one(idx, state)

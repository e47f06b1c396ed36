"""ctypes binding of librwkv_hip.so (declared in include/rwkv_hip.h).

The library is built in-tree by ``python -m chatrwkv_amd.build`` (hipcc, gfx950) and is the
only compute path of this package: if it is missing, or a call is rejected, an exception is
raised -- there is no fallback.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# RWKV_HIP_LIB: another build of the same library (kernel tuning: two builds side by side)
LIB_PATH = os.environ.get("RWKV_HIP_LIB") or os.path.join(HERE, "librwkv_hip.so")

RWKV_DT_F16, RWKV_DT_F32, RWKV_DT_BF16 = 0, 1, 2

_ERR = {
    -1: "RWKV_E_SHAPE: size not supported by the kernel",
    -2: "RWKV_E_LAYOUT: stride / alignment not supported",
    -3: "RWKV_E_NULL: required pointer is NULL",
    -4: "RWKV_E_WORKSPACE: workspace too small or misaligned",
    -5: "RWKV_E_DTYPE: unknown dtype / mode code",
    -6: "RWKV_E_SCRATCH: size beyond what the library's built-in scratch holds",
}

_i64, _int, _vp, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/rwkv_hip.h
SIGNATURES = {
    "rwkv_abi_version": (_int, []),
    "rwkv_quantize_u8": (_int, [_i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _int, _vp, _sz, _vp]),
    "rwkv_repack_u8": (_int, [_i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp]),
    "rwkv_repack_f16": (_int, [_i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp]),
    "rwkv_mm8_one_f16": (_int, [_i64, _i64, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _int, _vp]),
    "rwkv_mm8_seq_workspace": (_sz, [_i64, _i64]),
    "rwkv_mm8_seq_f16": (_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _sz, _vp]),
    "rwkv_mm8_seq_static_max_elems": (_sz, []),
    "rwkv_mm8_seq_static_max_rows": (_sz, []),
    "rwkv_mm8_seq_time_kernel": (_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _sz, _vp, _int, _vp]),
    "rwkv_mm8_seq_f16_static": (_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "rwkv_gemm_f16": (_int, [_i64, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _vp, _i64, _int, _vp]),
    "rwkv_gemm_f16_batched": (_int, [_i64, _i64, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _int, _vp]),
    "rwkv_release_stream": (_int, [_vp]),
    "rwkv_greedy_token": (_int, [_vp, _int, _i64, _vp, _vp]),
    "rwkv_wkv4_forward": (_int, [_i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _vp, _vp]),
    "rwkv_wkv5_forward": (_int, [_i64, _i64, _i64, _i64, _vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "rwkv_wkv6_forward": (_int, [_i64, _i64, _i64, _i64, _vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
}



class RwkvMat(ctypes.Structure):
    _fields_ = [("w", _vp), ("ld", _i64), ("mx", _vp), ("rx", _vp), ("my", _vp), ("ry", _vp), ("N", _i64), ("M", _i64)]


class RwkvV4Layer(ctypes.Structure):
    _fields_ = [("ln1_w", _vp), ("ln1_b", _vp), ("ln2_w", _vp), ("ln2_b", _vp),
                ("att_mix_k", _vp), ("att_mix_v", _vp), ("att_mix_r", _vp),
                ("time_decay", _vp), ("time_first", _vp),
                ("att_key", RwkvMat), ("att_value", RwkvMat), ("att_receptance", RwkvMat), ("att_output", RwkvMat),
                ("ffn_mix_k", _vp), ("ffn_mix_r", _vp),
                ("ffn_key", RwkvMat), ("ffn_receptance", RwkvMat), ("ffn_value", RwkvMat)]


class RwkvV4LayerState(ctypes.Structure):
    _fields_ = [("att_xx", _vp), ("aa", _vp), ("bb", _vp), ("pp", _vp), ("ffn_xx", _vp)]


class RwkvV4Model(ctypes.Structure):
    _fields_ = [("n_layer", ctypes.c_int32), ("n_embd", ctypes.c_int32), ("n_ffn", ctypes.c_int32),
                ("vocab", ctypes.c_int32), ("rescale_layer", ctypes.c_int32), ("weights_u8", ctypes.c_int32),
                ("emb", _vp), ("ln_out_w", _vp), ("ln_out_b", _vp), ("head", RwkvMat),
                ("layers", ctypes.POINTER(RwkvV4Layer)),
                ("layer_begin", ctypes.c_int32), ("layer_end", ctypes.c_int32)]


class RwkvV56Layer(ctypes.Structure):
    _fields_ = [("ln1_w", _vp), ("ln1_b", _vp), ("ln2_w", _vp), ("ln2_b", _vp),
                ("att_mix", _vp * 6),
                ("tm_w1", _vp), ("tm_w2", _vp), ("td_w1", _vp), ("td_w2", _vp),
                ("time_decay", _vp), ("time_first", _vp), ("lnx_w", _vp), ("lnx_b", _vp),
                ("att_key", RwkvMat), ("att_value", RwkvMat), ("att_receptance", RwkvMat), ("att_gate", RwkvMat),
                ("att_output", RwkvMat),
                ("ffn_mix_k", _vp), ("ffn_mix_r", _vp),
                ("ffn_key", RwkvMat), ("ffn_receptance", RwkvMat), ("ffn_value", RwkvMat)]


class RwkvV56LayerState(ctypes.Structure):
    _fields_ = [("att_xx", _vp), ("att_kv", _vp), ("ffn_xx", _vp)]


class RwkvV56Model(ctypes.Structure):
    _fields_ = [("version_x10", ctypes.c_int32), ("n_layer", ctypes.c_int32), ("n_embd", ctypes.c_int32),
                ("n_ffn", ctypes.c_int32), ("vocab", ctypes.c_int32), ("n_head", ctypes.c_int32),
                ("lora_maa", ctypes.c_int32), ("lora_decay", ctypes.c_int32),
                ("rescale_layer", ctypes.c_int32), ("weights_u8", ctypes.c_int32),
                ("emb", _vp), ("ln_out_w", _vp), ("ln_out_b", _vp), ("head", RwkvMat),
                ("layers", ctypes.POINTER(RwkvV56Layer)),
                ("layer_begin", ctypes.c_int32), ("layer_end", ctypes.c_int32)]


class RwkvV7Layer(ctypes.Structure):
    _fields_ = [("ln1_w", _vp), ("ln1_b", _vp), ("ln2_w", _vp), ("ln2_b", _vp),
                ("x_mix", _vp * 6),
                ("w0", _vp), ("a0", _vp), ("v0", _vp),
                ("lora1", _vp), ("lora2", _vp),
                ("k_k", _vp), ("k_a", _vp), ("r_k", _vp), ("lnx_w", _vp), ("lnx_b", _vp),
                ("att_receptance", RwkvMat), ("att_key", RwkvMat), ("att_value", RwkvMat), ("att_output", RwkvMat),
                ("ffn_x_k", _vp), ("ffn_key", RwkvMat), ("ffn_value", RwkvMat),
                ("de_emb", _vp), ("de_s1", _vp), ("de_s2", _vp), ("de_s0", _vp)]


class RwkvV7Model(ctypes.Structure):
    _fields_ = [("n_layer", ctypes.c_int32), ("n_embd", ctypes.c_int32), ("n_ffn", ctypes.c_int32),
                ("vocab", ctypes.c_int32), ("n_head", ctypes.c_int32),
                ("lora_w", ctypes.c_int32), ("lora_a", ctypes.c_int32), ("lora_v", ctypes.c_int32),
                ("lora_g", ctypes.c_int32),
                ("emb", _vp), ("ln_out_w", _vp), ("ln_out_b", _vp), ("head", RwkvMat),
                ("layers", ctypes.POINTER(RwkvV7Layer))]


SIGNATURES.update({
    "rwkv_wkv7_forward": (_int, [_i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _vp]),
    "rwkv_v7_workspace": (_sz, [ctypes.POINTER(RwkvV7Model), _i64]),
    "rwkv_v7_forward": (_int, [ctypes.POINTER(RwkvV7Model), ctypes.POINTER(RwkvV56LayerState), _vp, _i64, _int, _vp, _vp, _sz, _vp]),
    "rwkv_v56_workspace": (_sz, [ctypes.POINTER(RwkvV56Model), _i64]),
    "rwkv_v56_forward": (_int, [ctypes.POINTER(RwkvV56Model), ctypes.POINTER(RwkvV56LayerState), _vp, _i64, _int, _vp, _vp, _sz, _vp]),
    "rwkv_layernorm_f32_f16": (_int, [_i64, _i64, _vp, _vp, _vp, _vp, _vp]),
    "rwkv_sample_logits": (_int, [_vp, _i64, ctypes.c_float, ctypes.c_float, ctypes.c_int32, _vp, ctypes.c_int32, _vp, _vp, _vp,
                                  ctypes.c_float, ctypes.c_float, ctypes.c_float, _vp, _vp, _vp, _vp]),
    "rwkv_v4_one_workspace": (_sz, [ctypes.POINTER(RwkvV4Model)]),
    "rwkv_v4_forward_one": (_int, [ctypes.POINTER(RwkvV4Model), ctypes.POINTER(RwkvV4LayerState), _vp, _vp, _vp, _sz, _vp]),
    "rwkv_v4_profile_one": (_int, [ctypes.POINTER(RwkvV4Model), ctypes.POINTER(RwkvV4LayerState), _vp, _vp, _vp, _sz, _vp, _vp, _i64]),
    "rwkv_v4_time_phase": (_int, [ctypes.POINTER(RwkvV4Model), ctypes.POINTER(RwkvV4LayerState), _vp, _vp, _vp, _sz, _vp, _int, _int, _vp]),
    "rwkv_v4_seq_workspace": (_sz, [ctypes.POINTER(RwkvV4Model), _i64, _int]),
    "rwkv_v4_forward_seq": (_int, [ctypes.POINTER(RwkvV4Model), ctypes.POINTER(RwkvV4LayerState), _vp, _i64, _int, _vp, _vp, _sz, _vp]),
})

_lib = None


class RwkvHipError(RuntimeError):
    pass


def load():
    """Load the shared library (once) and declare every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RwkvHipError(
            f"{LIB_PATH} not found: build it with `python -m chatrwkv_amd.build` "
            "(hipcc --offload-arch=gfx950). This package has no CPU or PyTorch fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class StreamOrder:
    """Calls on ONE model object issued from different streams are put in one order on the device.

    A model object owns one workspace, one logits buffer and (streamed strategies) one staging buffer, so two of its
    calls must not overlap.  A forward call whose stream differs from the object's previous call first makes its
    stream wait (on the device, no host synchronisation) for the event recorded after that previous call.  Calls
    on one stream cost one event record each and are not delayed; calls on different model objects are not ordered
    against each other and may overlap."""

    def __init__(self):
        self.stream = None
        self.event = None

    def before(self):
        import torch
        cur = torch.cuda.current_stream()
        if self.event is not None and self.stream != cur.cuda_stream:
            cur.wait_event(self.event)
        return cur

    def after(self, cur):
        import torch
        if self.event is None:
            self.event = torch.cuda.Event()
        self.event.record(cur)
        self.stream = cur.cuda_stream


def check(rc, what):
    if rc == 0:
        return
    if rc < 0:
        raise RwkvHipError(f"{what}: {_ERR.get(rc, rc)}")
    raise RwkvHipError(f"{what}: HIP error {rc}")

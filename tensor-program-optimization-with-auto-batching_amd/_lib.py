"""ctypes binding of libmlora_hip.so (the C ABI declared in include/mlora.h).

There is no fallback: if the library has not been built, loading raises and every operator fails.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmlora_hip.so")

F16, F32 = 0, 1
ROWMAJOR, FRAG = 0, 1
STORE, ACCUMULATE = 0, 1
PAGE_SIZE = 16

_p, _i, _f, _z = C.c_void_p, C.c_int, C.c_float, C.c_size_t

# name -> (restype, argtypes); mirrors include/mlora.h one to one
SIGNATURES = {
    "mlora_version": (_i, []),
    "mlora_last_error": (C.c_char_p, []),
    "mlora_gather_mm_workspace_bytes": (_z, [_i, _i, _i]),
    "mlora_gather_mm": (_i, [_p, _i, _i, _p, _i, _p, _p, _p, _f, _i, _i, _i, _i, _i, _p, _z, _p]),
    "mlora_gather_mm_static_max_bytes": (_z, []),
    "mlora_gather_mm_static": (_i, [_p, _i, _i, _p, _i, _p, _p, _p, _f, _i, _i, _i, _i, _i, _p]),
    "mlora_gather_mm_multi": (_i, [_p, _i, _i, _p, _i, _p, _i, _p, _p, _i, _i, _i, _p, _z, _p]),
    "mlora_gather_mm_multi_proj": (_i, [_p, _i, _i, _p, _i, _p, _i, _i, _p, _p, _p, _p, _i, _i, _p, _z, _p]),
    "mlora_gather_mm_batch": (_i, [_p, _i, _i, _i, _i, _p, _f, _i, _i, _i, _i, _i, _p, _z, _p]),
    "mlora_lora_shrink": (_i, [_p, _p, _i, _p, _p, _i, _i, _i, _i, _p]),
    "mlora_lora_expand": (_i, [_p, _i, _i, _p, _p, _p, _f, _i, _i, _i, _i, _i, _p]),
    "mlora_write_tensor_part": (_i, [_p, _p, _p, _p, _i, _i, _i, _p]),
    "mlora_gemv": (_i, [_p, _i, _i, _p, _i, _p, _i, _i, _i, _p]),
    "mlora_gemm": (_i, [_p, _i, _i, _p, _i, _p, _i, _i, _i, _p]),
    "mlora_linear": (_i, [_p, _i, _i, _p, _i, _p, _i, _i, _i, _p]),
    "mlora_packed_weight_elems": (_z, [_i, _i]),
    "mlora_pack_weight": (_i, [_p, _p, _i, _i, _p]),
    "mlora_gemv_packed": (_i, [_p, _i, _i, _p, _i, _p, _i, _i, _i, _p]),
    "mlora_gemm_packed": (_i, [_p, _i, _i, _p, _i, _p, _i, _i, _i, _p]),
    "mlora_linear_packed": (_i, [_p, _i, _i, _p, _i, _p, _i, _i, _i, _p]),
    "mlora_frag_activation_elems": (_z, [_i, _i]),
    "mlora_pack_activation": (_i, [_p, _p, _i, _i, _i, _p]),
    "mlora_gemv_frag": (_i, [_p, _i, _i, _p, _p, _i, _i, _i, _p]),
    "mlora_linear_frag": (_i, [_p, _i, _i, _p, _p, _i, _i, _i, _p]),
    "mlora_gemm_frag_preferred": (_i, [_i, _i, _i]),
    "mlora_lora_block_adapters": (_i, [_p, _p, _p, _i, _i, _p]),
    "mlora_lora_shrink_split": (_i, [_p, _p, _p, _i, _p, _i, _p, _f, _i, _i, _i, _i, _p, _z, _p]),
    "mlora_linear_frag_lora": (_i, [_p, _i, _i, _p, _p, _i, _i, _i, _p, _i, _p, _i, _p]),
    "mlora_linear_frag_silu": (_i, [_p, _p, _p, _i, _i, _i, _p, _i, _p, _i, _p]),
    "mlora_gemv_frag_lora": (_i, [_p, _i, _i, _p, _p, _i, _i, _i, _p, _p, _i, _p, _i, _i, _p]),
    "mlora_gemv_frag_silu": (_i, [_p, _p, _p, _i, _i, _i, _p]),
    "mlora_gemv_frag_split": (_i, [_p, _i, _i, _p, _p, _p, _i, _i, _i, _i, _p]),
    "mlora_gemv_split_kq": (_i, [_i, _i, _i, _i]),
    "mlora_gemv_frag_split_kq": (_i, [_p, _p, _i, _p, _p, _i, _i, _i, _i, _p]),
    "mlora_rope_kv_append_lora": (_i, [_p, _p, _p, _p, _i, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _i, _p, _p, _f, _i, _i, _i, _p]),
    "mlora_rope_attn_decode": (_i, [_p, _i, _p, _p, _p, _p, _i, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _i, _p, _p, _f, _i, _i, _i, _p]),
    "mlora_gemv_ksplit": (_i, [_i, _i, _i]),
    "mlora_gemv_ksplit_bytes": (_z, [_i, _i, _i]),
    "mlora_gemv_shrink_rows": (_i, [_i, _i, _i]),
    "mlora_gemv_frag_acc_ksplit": (_i, [_p, _p, _p, _i, _p, _p, _i, _i, _i, _i, _p, _p, _i, _p, _i, _i, _p]),
    "mlora_gemv_delta_ride_ksplit": (_i, [_i, _i, _i, _i]),
    "mlora_gemv_frag_acc_ksplit_delta": (_i, [_p, _p, _i, _p, _p, _i, _i, _i, _p, _i, _p, _p, _f, _i, _i, _p]),
    "mlora_rope_attn_oshrink_ok": (_i, [_i, _i, _i, _i, _i]),
    "mlora_paged_attn_decode_oshrink": (_i, [_p, _i, _p, _p, _p, _p, _i, _p, _p, _i, _i, _i, _i, _i, _i, _p, _i, _i, _p, _p, _p]),
    "mlora_lora_expand_shares_ok": (_i, [_i, _i]),
    "mlora_lora_expand_shares": (_i, [_p, _p, _i, _p, _p, _f, _i, _i, _i, _i, _p]),
    "mlora_rope_attn_decode_oshrink": (_i, [_p, _i, _p, _p, _p, _p, _i, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _i, _p, _p, _f, _i, _i, _i, _p, _p, _p]),
    "mlora_rmsnorm_ksplit": (_i, [_p, _i, _p, _p, _i, _i, _p, _f, _i, _i, _p, _i, _p, _p, _f, _i, _i, _i, _p]),
    "mlora_lora_expand_rmsnorm": (_i, [_p, _i, _p, _p, _i, _p, _p, _f, _p, _f, _i, _i, _i, _i, _i, _p]),
    "mlora_rmsnorm": (_i, [_p, _i, _p, _i, _p, _f, _i, _i, _p]),
    "mlora_silu_mul": (_i, [_p, _i, _p, _p, _i, _i, _i, _p]),
    "mlora_embed": (_i, [_p, _i, _p, _p, _i, _i, _i, _p]),
    "mlora_argmax": (_i, [_p, _p, _i, _i, _p]),
    "mlora_rope_kv_append": (_i, [_p, _p, _p, _p, _i, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p]),
    "mlora_paged_attn_decode": (_i, [_p, _i, _p, _p, _p, _p, _i, _p, _p, _i, _i, _i, _i, _i, _i, _p]),
    "mlora_paged_attn_prefill": (_i, [_p, _i, _p, _p, _p, _p, _i, _p, _p, _i, _i, _i, _i, _i, _i, _p]),
}



class LoraBucket(C.Structure):
    _fields_ = [("A", _p), ("B", _p), ("r", _i), ("n_ad", _i), ("scaling", _f)]


class FusedLora(C.Structure):
    _fields_ = [("B", _p), ("v_hi", _p), ("v_lo", _p), ("n_begin", _i), ("n_rows", _i)]


class LoraProj(C.Structure):
    _fields_ = [("A", _p), ("B", _p)]


class Layer(C.Structure):
    _fields_ = [("qkv_p", _p), ("o_p", _p), ("gate_up_p", _p), ("gate_up_il_p", _p), ("down_p", _p), ("ln1", _p), ("ln2", _p),
                ("lora", LoraProj * 7), ("k_cache", _p), ("v_cache", _p)]


class DecodePlan(C.Structure):
    _fields_ = [("n_layers", _i), ("hidden", _i), ("inter", _i), ("n_q_heads", _i), ("n_kv_heads", _i), ("head_dim", _i),
                ("vocab", _i), ("eps", _f), ("lora_r", _i), ("lora_n_ad", _i), ("lora_scaling", _f), ("lora_dense", _i),
                ("layers", C.POINTER(Layer)), ("embed", _p), ("norm", _p), ("lm_head_p", _p),
                ("rope_cos", _p), ("rope_sin", _p), ("max_pos", _i),
                ("block_table", _p), ("max_blocks", _i), ("n_pages", _i), ("n_seq", _i),
                ("T", _i), ("tokens", _p), ("rows", _p), ("pos", _p), ("ctx", _p), ("tok_adapter", _p),
                ("resid", _p), ("xn", _p), ("qkv", _p), ("attn", _p), ("gate_up", _p), ("act", _p), ("logits", _p),
                ("lora_ws", _p), ("lora_ws_bytes", _z), ("ksplit_ws", _p), ("ksplit_ws_bytes", _z)]


SIGNATURES["mlora_decode_step"] = (_i, [C.POINTER(DecodePlan), _p])

_lib = None


class MloraError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"mlora error {code}: {msg}")
        self.code = code


def lib() -> C.CDLL:
    """The loaded library; raises if libmlora_hip.so is missing (build it with build.py)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} not found: the HIP library is not built (run build.py). There is no CPU fallback.")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(code: int) -> None:
    if code != 0:
        raise MloraError(code, lib().mlora_last_error().decode())

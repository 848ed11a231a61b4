"""ctypes binding of libohara_decode.so (declared in include/ohara_decode.h).

The HIP library is the only compute path of this package: if it has not been built
(``python -m ohara_amd.build``) loading fails loudly; there is no eager/CPU fallback.
"""

from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libohara_decode.so")

OK, EINVAL, ELAUNCH, ESIZE = 0, -1, -2, -3
_ERR = {EINVAL: "invalid argument", ELAUNCH: "HIP launch failed", ESIZE: "size not supported"}

EPI_STORE, EPI_RESIDUAL, EPI_SWIGLU = 0, 1, 2

_p, _i, _f, _i64 = C.c_void_p, C.c_int, C.c_float, C.c_int64


class OharaLayer(C.Structure):
    _fields_ = [("wqkv", _p), ("wo", _p), ("wgu", _p), ("wdown", _p), ("norm1", _p), ("norm2", _p)]


class OharaModel(C.Structure):
    _fields_ = [
        ("n_layers", _i), ("d_model", _i), ("n_heads", _i), ("n_kv_heads", _i), ("head_dim", _i),
        ("d_ff", _i), ("vocab", _i), ("t_max", _i),
        ("eps", _f), ("reserved", _i),
        ("token_emb", _p), ("final_norm", _p), ("w_vocab", _p), ("cos", _p), ("sin", _p),
        ("layers", C.POINTER(OharaLayer)),
    ]


class OharaBitLayer(C.Structure):
    _fields_ = [("w", _p * 7), ("norm_w", _p * 7), ("gamma", _f * 7), ("reserved", _f), ("norm1", _p), ("norm2", _p)]


class OharaBitModel(C.Structure):
    _fields_ = [
        ("n_layers", _i), ("d_model", _i), ("n_heads", _i), ("n_kv_heads", _i), ("head_dim", _i),
        ("d_ff", _i), ("vocab", _i), ("t_max", _i),
        ("eps", _f), ("reserved", _i),
        ("token_emb", _p), ("final_norm", _p), ("w_vocab", _p), ("cos", _p), ("sin", _p),
        ("layers", C.POINTER(OharaBitLayer)),
    ]


class OharaDecodeState(C.Structure):
    _fields_ = [
        ("batch", _i), ("rows_cap", _i), ("n_split", _i), ("valid_vocab", _i), ("hist_cap", _i), ("prof_kernel", _i),
        ("ids", _p), ("x", _p), ("q", _p), ("attn", _p), ("act", _p), ("xn", _p), ("logits", _p),
        ("attn_ws", _p), ("step_state", _p), ("history", _p),
        ("kcache", C.POINTER(_p)), ("vcache", C.POINTER(_p)),
        ("kv_int8", _i), ("kvstats", C.POINTER(_p)), ("kstage", _p), ("vstage", _p), ("kdeq", _p), ("vdeq", _p),
        ("seq_pos", _p), ("prof_start", _p), ("prof_stop", _p),
    ]


OHARA_LOGITS_NONE, OHARA_LOGITS_LAST, OHARA_LOGITS_ALL = 0, 1, 2

_PROTOS = {
    "ohara_abi_version": (_i, []),
    "ohara_pack_rows_bf16": (_i, [_p, _i, _i, _i, _p, _i, _p, C.POINTER(_i64), _p]),
    "ohara_swiglu_perm": (_i, [_i, _p]),
    "ohara_embed_bf16": (_i, [_p, _p, _p, _i, _i, _i, _p]),
    "ohara_rmsnorm_bf16": (_i, [_p, _p, _p, _i, _i, _f, _p]),
    "ohara_gemm_skinny_bf16": (_i, [_p, _i, _p, _i, _i, _p, _f, _i, _i, _p, _i, _p, _i, _p]),
    "ohara_gemm_bf16": (_i, [_p, _i, _p, _i, _i, _i, _i, _p, _i, _p, _i, _p]),
    "ohara_qkv_rope_append_bf16": (_i, [_p, _i, _p, _i, _p, _f, _i, _i, _i, _i, _i, _p, _p, _i, _p, _p, _p, _p, _i, _p]),
    "ohara_qkv_rope_bf16": (_i, [_p, _i, _p, _i, _p, _f, _i, _i, _i, _i, _i, _p, _p, _i, _p, _i, _p, _p, _p, _p]),
    "ohara_kv_quant_append_int8": (_i, [_p, _p, _i, _i, _i, _i, _i, _p, _p, _p, _p, _i, _p]),
    "ohara_kv_dequant_int8": (_i, [_p, _p, _i, _i, _i, _i, _i, _i, _p, _p]),
    "ohara_attn_cached_int8": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _i, _p, _p, _p]),
    "ohara_attn_workspace_bytes": (_i64, [_i, _i, _i, _i, _i]),
    "ohara_attn_cached_bf16": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _i, _p, _p, _p]),
    "ohara_attn_cached_bf16_noalloc": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _i, _p, _p]),
    "ohara_qkv_rope_ragged_bf16": (_i, [_p, _i, _p, _i, _p, _f, _i, _i, _i, _i, _i, _p, _p, _p, _i, _p, _p, _p, _p]),
    "ohara_kv_quant_append_ragged_int8": (_i, [_p, _p, _i, _i, _i, _i, _p, _p, _p, _p, _i, _p]),
    "ohara_attn_cached_ragged_int8": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p, _i, _p, _p, _p]),
    "ohara_attn_cached_ragged_bf16": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, _p, _i, _p, _p, _p]),
    "ohara_qkv_rope_append_ragged_bf16": (_i, [_p, _i, _p, _i, _p, _f, _i, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _i, _p]),
    "ohara_advance_positions": (_i, [_p, _p, _i, _i, _p]),
    "ohara_advance_ragged": (_i, [_p, _p, _p, _p, _i, _i, _p]),
    "ohara_attn_prefill_bf16": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p]),
    "ohara_argmax_bf16": (_i, [_p, _i, _i, _i, _i, _p, _p, _i, _p, _p]),
    "ohara_sample_topk_topp": (_i, [_p, _i, _i, _i, _i, _i, _f, _i, _f, _p, _i, _p, _p, _i, _p, _p]),
    "ohara_sample_topk_topp_exclusive": (_i, [_p, _i, _i, _i, _i, _i, _f, _i, _f, _p, _i, _p, _p, _i, _p, _p]),
    "ohara_sample_workspace_bytes": (_i64, []),
    "ohara_sample_topk_topp_ws": (_i, [_p, _i, _i, _i, _i, _i, _f, _i, _f, _p, _i, _p, _p, _i, _p, _p, _i64, _p]),
    "ohara_bitlinear_pack_ternary": (_i, [_p, _i, _i, _i, _p, C.POINTER(_i64), _p]),
    "ohara_act_quant_int8": (_i, [_p, _i, _p, _f, _i, _i, _p, _i, _p, _p, _p]),
    "ohara_gemv_ternary_i8": (_i, [_p, _i, _p, _p, _p, _i, _i, _f, _i, _p, _i, _p, _i, _p, _i, _p]),
    "ohara_bitlinear_bf16": (_i, [_p, _i, _p, _p, _f, _p, _i, _i, _f, _i, _p, _i, _p, _i, _p, _i, _p]),
    "ohara_bitlinear_qkv_rope_append_bf16": (_i, [_p, _i, _p, _f, _i, _p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _i, _p, _p, _p,
                                                  _p, _i, _p]),
    "ohara_bitlinear_gate_up_bf16": (_i, [_p, _i, _p, _f, _i, _i, _p, _p, _f, _p, _p, _f, _i, _p, _i, _p]),
    "ohara_silu_mul_bf16": (_i, [_p, _p, _p, _i64, _p]),
    "ohara_rope_append_bf16": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _i, _p, _p, _p, _i, _p]),
    "ohara_moe_route_topk": (_i, [_p, _i, _p, _i, _i, _i, _i, _i, _i, _p, _p, _p]),
    "ohara_moe_sort_pairs": (_i, [_p, _i, _i, _p, _p, _p, _p]),
    "ohara_moe_experts_gate_up": (_i, [_p, _i, _p, _i64, _i, _i, _i, _i, _p, _p, _p, _i, _p]),
    "ohara_moe_experts_down": (_i, [_p, _i, _p, _i64, _i, _i, _i, _i, _p, _p, _p, _p, _i, _p]),
    "ohara_moe_route_fused": (_i, [_p, _i, _p, _f, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _i, _p, _i, _p, _p, _p, _p, _p,
                                   _p, _p]),
    "ohara_moe_experts_gate_up_shared": (_i, [_p, _i, _p, _i64, _i, _i, _i, _i, _p, _p, _p, _i, _p, _i, _i, _p, _i, _p]),
    "ohara_moe_experts_down_shared": (_i, [_p, _i, _p, _i64, _i, _i, _i, _i, _p, _p, _p, _p, _i, _p, _i, _i, _p, _i, _p, _i,
                                           _p]),
    "ohara_moe_combine": (_i, [_p, _i, _p, _p, _i, _i, _p, _i, _p, _i, _p, _i, _i, _p]),
    "ohara_llama_forward": (_i, [C.POINTER(OharaModel), C.POINTER(OharaDecodeState), _i, _i, _i, _i, _i, _p]),
    "ohara_linear_bias_bf16": (_i, [_p, _i, _p, _i, _i, _p, _i, _i, _p, _i, _p, _i, _p, _i, _p]),
    "ohara_phi_block_in_bf16": (_i, [_p, _i, _p, _p, _f, _p, _p, _i, _i, _i, _i, _i, _p, _p, _i, _p, _p, _i, _p, _i, _p]),
    "ohara_layernorm_bf16": (_i, [_p, _i, _p, _p, _p, _i, _i, _i, _f, _p]),
    "ohara_kv_append_bf16": (_i, [_p, _p, _i, _i, _i, _i, _i, _i, _p, _p, _p, _i, _p]),
    "ohara_phi_attn_workspace_bytes": (_i64, [_i, _i, _i, _i]),
    "ohara_phi_attn_bf16": (_i, [_p, _i, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _i, _p, _p, _p]),
    "ohara_persistent_workspace_bytes": (_i64, [C.POINTER(OharaModel), _i, _i, _i]),
    "ohara_persistent_barrier_offset": (_i64, [C.POINTER(OharaModel), _i, _i, _i]),
    "ohara_persistent_polled": (_i, [C.POINTER(OharaModel), _i, _i]),
    "ohara_persistent_error_offset": (_i64, [C.POINTER(OharaModel), _i, _i, _i]),
    "ohara_persistent_profile_offset": (_i64, [C.POINTER(OharaModel), _i, _i, _i]),
    "ohara_llama_decode_persistent": (_i, [C.POINTER(OharaModel), C.POINTER(OharaDecodeState), _p, _i, _i, _i,
                                           C.c_uint, _p]),
    "ohara_bitnet_persistent_workspace_bytes": (_i64, [C.POINTER(OharaBitModel), _i, _i]),
    "ohara_bitnet_persistent_error_offset": (_i64, [C.POINTER(OharaBitModel), _i, _i]),
    "ohara_bitnet_persistent_profile_offset": (_i64, [C.POINTER(OharaBitModel), _i, _i]),
    "ohara_bitnet_decode_persistent": (_i, [C.POINTER(OharaBitModel), C.POINTER(OharaDecodeState), _p, _i, _i, _i,
                                            C.c_uint, _p]),
    "ohara_event_create": (_i, [C.POINTER(_p)]),
    "ohara_event_destroy": (_i, [_p]),
    "ohara_event_record": (_i, [_p, _p]),
    "ohara_event_elapsed_ms": (_i, [_p, _p, C.POINTER(_f)]),
}

_lib = None


def lib():
    """The loaded library; raises if it was never built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP kernels first (python -m ohara_amd.build). "
                "ohara_amd has no fallback path."
            )
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in _PROTOS.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status: int, what: str) -> None:
    if status != OK:
        raise RuntimeError(f"{what}: {_ERR.get(status, 'error')} ({status})")

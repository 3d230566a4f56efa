"""ctypes binding of libhf2q_hip.so — the C ABI declared in include/hf2q_hip.h.

There is no fallback: if the shared library is missing the import of the first
symbol raises, and every non-zero status becomes an ``HqError`` carrying the
library's own message.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libhf2q_hip.so")

HQ_OK, HQ_ERR_INVALID_ARGUMENT, HQ_ERR_UNSUPPORTED, HQ_ERR_HIP = 0, 1, 2, 3
HQ_Q4_0, HQ_Q8_0, HQ_Q4_K, HQ_Q5_K, HQ_Q6_K = 2, 8, 12, 13, 14
HQ_F32, HQ_BF16, HQ_F16 = 0, 1, 2


class HqError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"hq status {status}: {message}")
        self.status = status
        self.message = message


_c = ctypes
_vp, _u32, _u64, _i32, _sz, _f32 = _c.c_void_p, _c.c_uint32, _c.c_uint64, _c.c_int, _c.c_size_t, _c.c_float

HQ_QMATMUL_BATCH_MAX_JOBS = 4


class QmatmulJob(_c.Structure):
    """hq_qmatmul_job of include/hf2q_hip.h, field for field."""
    _fields_ = [("x", _c.c_void_p), ("x_up", _c.c_void_p), ("w", _c.c_void_p), ("ids", _c.c_void_p),
                ("y", _c.c_void_p), ("rows", _c.c_uint32), ("top_k", _c.c_uint32), ("n", _c.c_uint32),
                ("k", _c.c_uint32), ("n_experts", _c.c_uint32), ("expert_stride", _c.c_uint64),
                ("route_logits", _c.c_void_p), ("route_ids", _c.c_void_p), ("route_weights", _c.c_void_p)]


class GgufTensorInfo(_c.Structure):
    """hq_gguf_tensor_info of include/hf2q_hip.h, field for field."""
    _fields_ = [("ggml_type", _c.c_uint32), ("n_dims", _c.c_uint32), ("dims", _c.c_uint64 * 4),
                ("data_offset", _c.c_uint64), ("byte_len", _c.c_uint64)]


# name -> (restype, argtypes); the single source for the symbol-export test.
SIGNATURES = {
    "hq_last_error": (_c.c_char_p, []),
    "hq_version": (_i32, []),
    "hq_block_elems": (_u32, [_i32]),
    "hq_block_bytes": (_u32, [_i32]),
    "hq_dequant_ggml": (_i32, [_vp, _vp, _vp, _i32, _u64, _i32]),
    "hq_quantize_ggml": (_i32, [_vp, _vp, _u64, _u64, _i32, _vp]),
    "hq_quantize_ggml_imatrix_scratch_bytes": (_sz, [_u64, _u64, _i32]),
    "hq_quantize_ggml_imatrix": (_i32, [_vp, _vp, _u64, _u64, _i32, _vp, _vp, _vp, _sz]),
    "hq_qmatmul_ggml": (_i32, [_vp, _vp, _i32, _vp, _vp, _u32, _u32, _u32, _i32]),
    "hq_qmatmul_ggml_workspace_bytes": (_sz, [_u32, _u32, _u32, _i32, _i32]),
    "hq_qmatmul_ggml_k_slices": (_i32, [_u32, _u32, _u32, _i32, _c.POINTER(_u32), _c.POINTER(_u32)]),
    "hq_gemv_flat_plan": (_i32, [_u32, _u32, _i32, _u32] + [_c.POINTER(_u32)] * 5),
    "hq_qmatmul_ggml_ws": (_i32, [_vp, _vp, _i32, _vp, _vp, _u32, _u32, _u32, _i32, _vp, _sz]),
    "hq_qmatmul_id_ggml": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _sz, _u32, _u32, _u32, _u32, _u32, _u64, _i32]),
    "hq_weight_row_scales_ggml": (_i32, [_vp, _vp, _vp, _u64, _u32, _i32]),
    "hq_qmatmul_ggml_ws_prepared": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _u32, _u32, _u32, _i32, _vp, _sz]),
    "hq_qmatmul_id_ggml_prepared": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _u32, _u32, _u32, _u32, _u32, _u64, _i32]),
    "hq_qmatmul_id_swiglu_ggml_workspace_bytes": (_sz, [_u32, _u32, _u32, _u32, _u32, _u64, _i32]),
    "hq_qmatmul_id_swiglu_ggml": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _u32, _u32, _u32, _u32, _u32, _u64, _i32]),
    "hq_qmatmul_gated_ggml_workspace_bytes": (_sz, [_u32, _u32, _u32, _i32, _i32]),
    "hq_qmatmul_gated_ggml_ws": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _i32, _vp, _sz]),
    "hq_qmatmul_swiglu_ggml_workspace_bytes": (_sz, [_u32, _u32, _u32, _i32, _i32]),
    "hq_qmatmul_swiglu_ggml_ws": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _i32, _vp, _sz]),
    "hq_qmatmul_swiglu_decode_supported": (_i32, [_u32, _u32, _i32, _i32]),
    "hq_qmatmul_swiglu_decode": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _u32, _u32, _u32, _i32]),
    "hq_qmatmul_perm021_ggml_workspace_bytes": (_sz, [_u32, _u32, _u32, _i32, _i32]),
    "hq_qmatmul_perm021_ggml_ws": (_i32, [_vp, _vp, _i32, _vp, _vp, _u32, _u32, _u32, _u32, _i32, _vp, _sz]),
    "hq_qmatmul_id_ggml_workspace_bytes": (_sz, [_u32, _u32, _u32, _u32, _u32, _u64, _i32]),
    "hq_qmatmul_id_scratch_bytes": (_sz, [_u32, _u32]),
    "hq_qmatmul_batch_ggml": (_i32, [_vp, _vp, _u32, _i32, _i32]),
    "hq_dense_gemv_bf16": (_i32, [_vp, _vp, _i32, _vp, _vp, _u32, _u32, _u32]),
    "hq_dense_gemv_bf16_pair": (_i32, [_vp, _vp, _i32, _vp, _vp, _u32, _vp, _vp, _u32, _u32, _u32]),
    "hq_moe_softmax_topk": (_i32, [_vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "hq_silu_mul": (_i32, [_vp, _vp, _vp, _vp, _u64]),
    "hq_moe_weighted_reduce": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "hq_moe_ffn_decode_scratch_bytes": (_sz, [_u32, _u32, _u32, _u32, _u32, _u32, _i32, _i32]),
    "hq_moe_ffn_decode_layer_scratch_bytes": (_sz, [_vp, _u32, _i32]),
    "hq_moe_ffn_decode": (_i32, [_vp, _vp, _vp, _i32, _vp, _vp, _u32, _vp, _sz, _vp, _vp]),
    "hq_handover_status": (_i32, [_vp, _vp, _c.POINTER(_u32)]),
    "hq_set_handover_spin_limit": (None, [_u32]),
    "hq_dense_ffn_decode_scratch_bytes": (_sz, [_u32, _u32, _i32, _i32, _i32]),
    "hq_dense_ffn_decode": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _vp, _vp, _u32, _u32, _vp, _sz]),
    "hq_moe_ffn_prefill_scratch_bytes": (_sz, [_vp, _u32, _i32]),
    "hq_moe_ffn_prefill": (_i32, [_vp, _vp, _vp, _vp, _i32, _vp, _vp, _u32, _vp, _sz, _vp, _vp]),
    "hq_dense_ffn_scratch_bytes": (_sz, [_u32, _u32, _u32, _i32, _i32, _i32]),
    "hq_dense_ffn": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp, _sz]),
    "hq_fwht_sign_premult_f32": (_i32, [_vp, _vp, _u32, _u32]),
    "hq_fwht_sign_undo_f32": (_i32, [_vp, _vp, _u32, _u32]),
    "hq_tq_encode_kv": (_i32, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32]),
    "hq_tq_dequantize_kv_seq": (_i32, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _f32, _u32, _i32]),
    "hq_flash_attn_vec_tq": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "hq_flash_attn_vec_tq_undo": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "hq_flash_attn_vec_tq_tmp_bytes": (_sz, [_u32, _u32, _u32]),
    "hq_flash_attn_vec_tq_static": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32]),
    "hq_tqp_indices_bytes": (_sz, [_vp]),
    "hq_tqp_norms_bytes": (_sz, [_vp]),
    "hq_tqp_total_bytes": (_sz, [_vp]),
    "hq_tqp_pack": (_i32, [_vp, _vp, _sz, _vp, _sz, _vp, _sz]),
    "hq_tqp_unpack": (_i32, [_vp, _sz, _vp, _c.POINTER(_sz), _c.POINTER(_sz)]),
    "hq_tq_kv_capture_bytes": (_sz, [_u32, _u32, _u32]),
    "hq_tq_kv_capture": (_i32, [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _vp, _sz]),
    "hq_tq_kv_restore": (_i32, [_vp, _vp, _sz, _vp, _vp, _u32, _u32, _u32, _u32]),
    "hq_matmul_f16_shadow_workspace_bytes": (_sz, [_u32, _u32, _u32]),
    "hq_matmul_f16_shadow": (_i32, [_vp, _vp, _i32, _vp, _vp, _u32, _u32, _u32, _vp, _sz]),
    "hq_dense_matmul_workspace_bytes": (_sz, [_u32, _u32, _u32, _i32, _i32]),
    "hq_dense_matmul": (_i32, [_vp, _vp, _i32, _vp, _i32, _vp, _u32, _u32, _u32, _vp, _sz]),
    "hq_stream_read_probe": (_i32, [_vp, _vp, _sz, _vp]),
    "hq_gguf_open": (_i32, [_c.c_char_p, _c.POINTER(_vp)]),
    "hq_gguf_close": (None, [_vp]),
    "hq_gguf_tensor_count": (_u64, [_vp]),
    "hq_gguf_metadata_count": (_u64, [_vp]),
    "hq_gguf_alignment": (_u64, [_vp]),
    "hq_gguf_tensor_name": (_c.c_char_p, [_vp, _u64]),
    "hq_gguf_metadata_key": (_c.c_char_p, [_vp, _u64]),
    "hq_gguf_tensor_info_by_name": (_i32, [_vp, _c.c_char_p, _c.POINTER(GgufTensorInfo)]),
    "hq_gguf_metadata_u64": (_i32, [_vp, _c.c_char_p, _c.POINTER(_u64)]),
    "hq_gguf_metadata_f64": (_i32, [_vp, _c.c_char_p, _c.POINTER(_c.c_double)]),
    "hq_gguf_metadata_string": (_i32, [_vp, _c.c_char_p, _c.POINTER(_vp), _c.POINTER(_u64)]),
    "hq_gguf_tensor_data": (_vp, [_vp, _c.c_char_p, _c.POINTER(_u64)]),
    "hq_gguf_load_tensor": (_i32, [_vp, _c.c_char_p, _vp, _vp, _sz]),
}


class TqpHeader(ctypes.Structure):
    """hq_tqp_header (include/hf2q_hip.h)."""
    _fields_ = [("codec_version", _u32), ("bits_per_coord", _u32), ("head_dim", _u32), ("n_kv_heads", _u32),
                ("n_tokens", _u32), ("flags", _u32), ("scale", ctypes.c_double)]


class MoeFfnLayer(ctypes.Structure):
    """hq_moe_ffn_layer (include/hf2q_hip.h), field for field."""
    _fields_ = [("router", _vp), ("shared_gate_logit", _vp), ("expert_gate", _vp), ("expert_up", _vp), ("expert_down", _vp),
                ("shared_gate", _vp), ("shared_up", _vp), ("shared_down", _vp), ("hidden", _u32), ("n_experts", _u32),
                ("top_k", _u32), ("inter", _u32), ("shared_inter", _u32), ("ggml_type", _i32),
                ("expert_stride_gate_up", _u64), ("expert_stride_down", _u64), ("down_type", _u32)]


class MoeFfnRowScales(ctypes.Structure):
    """hq_moe_ffn_row_scales (include/hf2q_hip.h)."""
    _fields_ = [("expert_gate", _vp), ("expert_up", _vp), ("expert_down", _vp), ("shared_gate", _vp), ("shared_up", _vp),
                ("shared_down", _vp)]


class TqAttnParams(ctypes.Structure):
    """hq_tq_attn_params (include/hf2q_hip.h)."""
    _fields_ = [("num_heads", _u32), ("num_kv_heads", _u32), ("head_dim", _u32), ("kv_seq_len", _u32),
                ("kv_capacity", _u32), ("scale", _f32), ("mask_type", _u32), ("sliding_window", _u32),
                ("softcap", _f32), ("ring_start", _u32), ("scale_factor_d512", _f32), ("codebook_bits", _u32),
                ("fuse_fwht_pre", _u32), ("nsg", _u32)]

_lib = None


def load() -> ctypes.CDLL:
    """Load libhf2q_hip.so (built by ``python -m hf2q_amd.build``); raises if absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `python -m hf2q_amd.build` "
                "(there is no CPU fallback for this path)")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error() -> str:
    return load().hq_last_error().decode()


def check(status: int) -> None:
    if status != HQ_OK:
        raise HqError(status, last_error())

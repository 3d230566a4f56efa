"""Host-side mirror of the kernel-dispatch interface hf2q's model code calls.

Names and argument meaning follow the reference call sites so that call sites
(and tests) read like the reference's: ``GgmlQuantizedMatmulParams`` +
``quantized_matmul_ggml`` (gpu_ffn.rs:1218-1245), ``GgmlQuantizedMatmulIdParams``
+ ``quantized_matmul_id_ggml`` (gpu_ffn.rs:194-204, 2606-2618),
``FlashAttnVecTqHbParams`` + ``flash_attn_vec_tq_hb`` (forward_mlx.rs:4687-4742).
torch tensors stand in for ``MlxBuffer`` (device memory + the current stream);
all arithmetic happens in libhf2q_hip.so through its C ABI.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import lib as _l
from .lib import HQ_BF16, HQ_F32, HQ_Q4_K, HQ_Q6_K, HQ_Q8_0, HqError  # noqa: F401

BLOCK_ELEMS = {HQ_Q8_0: 32, HQ_Q4_K: 256, HQ_Q6_K: 256}
BLOCK_BYTES = {HQ_Q8_0: 34, HQ_Q4_K: 144, HQ_Q6_K: 210}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, name: str) -> int:
    if not t.is_cuda:
        raise ValueError(f"{name} must live in device memory")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t.data_ptr()


def _act_dtype(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return HQ_F32
    if t.dtype == torch.bfloat16:
        return HQ_BF16
    raise TypeError(f"activation dtype {t.dtype} (f32 or bf16 expected)")


def ggml_row_bytes(ggml_type: int, k: int) -> int:
    """GgmlType::row_size (ggml_type.rs:127-135)."""
    return k // BLOCK_ELEMS[ggml_type] * BLOCK_BYTES[ggml_type]


@dataclass(frozen=True)
class GgmlQuantizedMatmulParams:
    """forward_mlx.rs:408-415 / gpu_ffn.rs:1218-1223."""
    m: int
    n: int
    k: int
    ggml_type: int


@dataclass(frozen=True)
class GgmlQuantizedMatmulIdParams:
    """gpu_ffn.rs:2606-2618."""
    n_tokens: int
    top_k: int
    n: int
    k: int
    n_experts: int
    expert_stride: int  # bytes
    ggml_type: int


def quantized_matmul_ggml(input: torch.Tensor, weight: torch.Tensor, dst: torch.Tensor,
                          params: GgmlQuantizedMatmulParams) -> None:
    """dst[m,n] = input[m,k] . W[n,k]^T, W = raw GGML blocks (uint8 tensor)."""
    if dst.dtype != torch.float32:
        raise TypeError("dst must be float32")
    L = _l.load()
    _l.check(L.hq_qmatmul_ggml(_stream(), _dev(input, "input"), _act_dtype(input), _dev(weight, "weight"),
                               _dev(dst, "dst"), params.m, params.n, params.k, params.ggml_type))


def quantized_matmul_id_ggml(input: torch.Tensor, weight_stack: torch.Tensor, ids: torch.Tensor,
                             output: torch.Tensor, params: GgmlQuantizedMatmulIdParams,
                             scratch: torch.Tensor | None = None) -> None:
    """output[t, s, :] = W[ids[t, s]] . input[t, :]."""
    if output.dtype != torch.float32:
        raise TypeError("output must be float32")
    if ids.dtype not in (torch.int32, torch.uint32):
        raise TypeError("ids must be 32-bit")
    L = _l.load()
    sp = _dev(scratch, "scratch") if scratch is not None else None
    sb = scratch.numel() * scratch.element_size() if scratch is not None else 0
    _l.check(L.hq_qmatmul_id_ggml(_stream(), _dev(input, "input"), _act_dtype(input),
                                  _dev(weight_stack, "weight_stack"), _dev(ids, "ids"), _dev(output, "output"),
                                  sp, sb, params.n_tokens, params.top_k, params.n, params.k, params.n_experts,
                                  params.expert_stride, params.ggml_type))


def id_scratch_bytes(n_experts: int, max_rows: int) -> int:
    return _l.load().hq_qmatmul_id_scratch_bytes(n_experts, max_rows)


def dequantize_ggml(weight: torch.Tensor, n_elems: int, ggml_type: int,
                    dtype: torch.dtype = torch.float32) -> torch.Tensor:
    out = torch.empty(n_elems, dtype=dtype, device=weight.device)
    L = _l.load()
    _l.check(L.hq_dequant_ggml(_stream(), _dev(weight, "weight"), _dev(out, "out"), _act_dtype(out), n_elems,
                               ggml_type))
    return out


def quantize_ggml(src: torch.Tensor, n_per_row: int, ggml_type: int) -> torch.Tensor:
    """f32 rows -> packed GGML blocks on the device (GgmlQuantizer::quantize without imatrix)."""
    if src.dtype != torch.float32:
        raise TypeError("src must be float32")
    n = src.numel()
    be, bb = BLOCK_ELEMS[ggml_type], BLOCK_BYTES[ggml_type]
    out = torch.empty(n // be * bb if n % be == 0 else 0, dtype=torch.uint8, device=src.device)
    L = _l.load()
    _l.check(L.hq_quantize_ggml(_stream(), _dev(src, "src"), n, n_per_row, ggml_type, _dev(out, "out")))
    return out

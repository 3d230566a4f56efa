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

import ctypes
import os
from dataclasses import dataclass

import torch

from . import lib as _l
from .lib import HQ_BF16, HQ_F16, HQ_F32, HQ_Q4_0, HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, HqError  # noqa: F401

BLOCK_ELEMS = {HQ_Q4_0: 32, HQ_Q8_0: 32, HQ_Q4_K: 256, HQ_Q5_K: 256, HQ_Q6_K: 256}
BLOCK_BYTES = {HQ_Q4_0: 18, HQ_Q8_0: 34, HQ_Q4_K: 144, HQ_Q5_K: 176, HQ_Q6_K: 210}


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


def weight_row_scales_ggml(weight: torch.Tensor, n_rows: int, k: int, ggml_type: int) -> torch.Tensor:
    """The f16 tile kernels' scale of every weight row (n_rows floats; a stack counts its experts' rows in order): a
    function of the weights alone, computed once when they are loaded and passed as `w_row_scales` to the matmul
    calls, whose pre-pass then skips the scan of the block headers.  Same results to the bit."""
    out = torch.empty(n_rows, dtype=torch.float32, device=weight.device)
    _l.check(_l.load().hq_weight_row_scales_ggml(_stream(), _dev(weight, "weight"), _dev(out, "scales"), n_rows, k, ggml_type))
    return out


def _check_scales(s: torch.Tensor, rows: int) -> None:
    if s.dtype != torch.float32 or s.numel() < rows or not s.is_contiguous():
        raise ValueError(f"w_row_scales must be {rows} contiguous float32 values")


def quantized_matmul_ggml(input: torch.Tensor, weight: torch.Tensor, dst: torch.Tensor,
                          params: GgmlQuantizedMatmulParams, workspace: torch.Tensor | None = None,
                          w_row_scales: torch.Tensor | None = None) -> None:
    """dst[m,n] = input[m,k] . W[n,k]^T, W = raw GGML blocks (uint8 tensor).  With `workspace`
    (a uint8 device tensor of quantized_matmul_workspace_bytes()) the call allocates nothing; `w_row_scales`
    (weight_row_scales_ggml of this weight; needs `workspace`) saves the pre-pass its scan of the weights."""
    if dst.dtype != torch.float32:
        raise TypeError("dst must be float32")
    L = _l.load()
    if w_row_scales is not None:
        if workspace is None:
            raise ValueError("w_row_scales needs a workspace")
        _check_scales(w_row_scales, params.n)
        _l.check(L.hq_qmatmul_ggml_ws_prepared(_stream(), _dev(input, "input"), _act_dtype(input), _dev(weight, "weight"),
                                               _dev(w_row_scales, "w_row_scales"), _dev(dst, "dst"), params.m, params.n,
                                               params.k, params.ggml_type, _dev(workspace, "workspace"),
                                               workspace.numel() * workspace.element_size()))
        return
    if workspace is not None:
        _l.check(L.hq_qmatmul_ggml_ws(_stream(), _dev(input, "input"), _act_dtype(input), _dev(weight, "weight"),
                                      _dev(dst, "dst"), params.m, params.n, params.k, params.ggml_type,
                                      _dev(workspace, "workspace"), workspace.numel() * workspace.element_size()))
        return
    _l.check(L.hq_qmatmul_ggml(_stream(), _dev(input, "input"), _act_dtype(input), _dev(weight, "weight"),
                               _dev(dst, "dst"), params.m, params.n, params.k, params.ggml_type))


def quantized_matmul_workspace_bytes(params: GgmlQuantizedMatmulParams, act_dtype: torch.dtype) -> int:
    """Device scratch quantized_matmul_ggml(..., workspace=) needs for this shape (0 for most)."""
    L = _l.load()
    xdt = _l.HQ_BF16 if act_dtype == torch.bfloat16 else _l.HQ_F32
    return int(L.hq_qmatmul_ggml_workspace_bytes(params.m, params.n, params.k, xdt, params.ggml_type))


def quantized_matmul_gated_workspace_bytes(params: GgmlQuantizedMatmulParams, act_dtype: torch.dtype) -> int:
    """Device scratch of quantized_matmul_gated_ggml for this shape; 0 where that form does not exist."""
    xdt = _l.HQ_BF16 if act_dtype == torch.bfloat16 else _l.HQ_F32
    return int(_l.load().hq_qmatmul_gated_ggml_workspace_bytes(params.m, params.n, params.k, xdt, params.ggml_type))


def quantized_matmul_gated_ggml(input: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, dst: torch.Tensor,
                                params: GgmlQuantizedMatmulParams, workspace: torch.Tensor,
                                w_row_scales: torch.Tensor | None = None) -> None:
    """dst[m, n] = silu(gate[m, n]) * (input . W^T)[m, n]: the up projection of a dense SwiGLU layer at prefill with
    the gating in its epilogue (gate: the f32 output of the gate projection; dst may be that buffer)."""
    if dst.dtype != torch.float32 or gate.dtype != torch.float32:
        raise TypeError("dst and gate must be float32")
    if gate.numel() < params.m * params.n:
        raise ValueError("gate must hold m * n values")
    if w_row_scales is not None:
        _check_scales(w_row_scales, params.n)
    _l.check(_l.load().hq_qmatmul_gated_ggml_ws(
        _stream(), _dev(input, "input"), _act_dtype(input), _dev(weight, "weight"),
        _dev(w_row_scales, "w_row_scales") if w_row_scales is not None else None, _dev(gate, "gate"), _dev(dst, "dst"),
        params.m, params.n, params.k, params.ggml_type, _dev(workspace, "workspace"), workspace.numel() * workspace.element_size()))


def quantized_matmul_swiglu_workspace_bytes(params: GgmlQuantizedMatmulParams, act_dtype: torch.dtype) -> int:
    """Device scratch of quantized_matmul_swiglu_ggml for this shape; 0 where that form does not exist."""
    xdt = _l.HQ_BF16 if act_dtype == torch.bfloat16 else _l.HQ_F32
    return int(_l.load().hq_qmatmul_swiglu_ggml_workspace_bytes(params.m, params.n, params.k, xdt, params.ggml_type))


def quantized_matmul_swiglu_ggml(input: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, dst: torch.Tensor,
                                 params: GgmlQuantizedMatmulParams, workspace: torch.Tensor,
                                 gate_row_scales: torch.Tensor | None = None, up_row_scales: torch.Tensor | None = None) -> None:
    """dst[m, n] = silu(input . gate^T) * (input . up^T): the two products of a dense SwiGLU layer (or of the MoE
    block's shared expert) and the gating at prefill as one call: the bits of the three separate ones where the plain
    product sums all of k in one tile (quantized_matmul_gated_workspace_bytes > 0), a few units in the last place from
    them where it cuts k into slices."""
    if dst.dtype != torch.float32:
        raise TypeError("dst must be float32")
    for s_ in (gate_row_scales, up_row_scales):
        if s_ is not None:
            _check_scales(s_, params.n)
    _l.check(_l.load().hq_qmatmul_swiglu_ggml_ws(
        _stream(), _dev(input, "input"), _act_dtype(input), _dev(gate, "gate"), _dev(up, "up"),
        _dev(gate_row_scales, "gate_row_scales") if gate_row_scales is not None else None,
        _dev(up_row_scales, "up_row_scales") if up_row_scales is not None else None, _dev(dst, "dst"), params.m, params.n,
        params.k, params.ggml_type, _dev(workspace, "workspace"), workspace.numel() * workspace.element_size()))


def quantized_matmul_swiglu_decode_supported(params: GgmlQuantizedMatmulParams, act_dtype: torch.dtype) -> bool:
    xdt = HQ_BF16 if act_dtype == torch.bfloat16 else HQ_F32
    return bool(_l.load().hq_qmatmul_swiglu_decode_supported(params.n, params.k, params.ggml_type, xdt))


def quantized_matmul_swiglu_decode(input: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, dst: torch.Tensor,
                                   params: GgmlQuantizedMatmulParams) -> None:
    """dst[m, n] = silu(input . gate^T) * (input . up^T) for m <= 8 rows: the gate / up pair of a decode step
    (gpu_ffn.rs:1231-1258) and the silu_mul behind it as one launch per row; the bits of the separate dispatches."""
    _l.check(_l.load().hq_qmatmul_swiglu_decode(_stream(), _dev(input, "input"), _act_dtype(input), _dev(gate, "gate"), _dev(up, "up"),
                                                _dev(dst, "dst"), params.m, params.n, params.k, params.ggml_type))


@dataclass
class GgmlQuantizedMatmulPerm021Params:
    """forward_prefill_batched.rs:2219-2226."""
    m: int
    n: int
    k: int
    head_dim: int
    ggml_type: int


def quantized_matmul_mm_tensor_perm021(input_perm: torch.Tensor, weight: torch.Tensor, output: torch.Tensor,
                                       params: GgmlQuantizedMatmulPerm021Params, workspace: torch.Tensor | None = None) -> None:
    """forward_prefill_batched.rs:2246-2253: output[m, n] = x[m, k] . W[n, k]^T with x stored [k / head_dim, m, head_dim]."""
    if output.dtype != torch.float32:
        raise TypeError("output must be float32")
    L = _l.load()
    xdt = _act_dtype(input_perm)
    need = int(L.hq_qmatmul_perm021_ggml_workspace_bytes(params.m, params.n, params.k, xdt, params.ggml_type))
    if workspace is None:
        workspace = torch.empty(max(need, 256), dtype=torch.uint8, device=input_perm.device)
    _l.check(L.hq_qmatmul_perm021_ggml_ws(_stream(), _dev(input_perm, "input"), xdt, _dev(weight, "weight"), _dev(output, "output"),
                                          params.m, params.n, params.k, params.head_dim, params.ggml_type,
                                          _dev(workspace, "workspace"), workspace.numel() * workspace.element_size()))


def quantized_matmul_id_ggml(input: torch.Tensor, weight_stack: torch.Tensor, ids: torch.Tensor,
                             output: torch.Tensor, params: GgmlQuantizedMatmulIdParams,
                             scratch: torch.Tensor | None = None, w_row_scales: torch.Tensor | None = None) -> None:
    """output[t, s, :] = W[ids[t, s]] . input[t, :].  `w_row_scales`: weight_row_scales_ggml of the whole stack
    (n_experts * n rows), which the grouped (prefill) form then does not work out again."""
    if output.dtype != torch.float32:
        raise TypeError("output must be float32")
    if ids.dtype not in (torch.int32, torch.uint32):
        raise TypeError("ids must be 32-bit")
    L = _l.load()
    sp = _dev(scratch, "scratch") if scratch is not None else None
    sb = scratch.numel() * scratch.element_size() if scratch is not None else 0
    if w_row_scales is not None:
        _check_scales(w_row_scales, params.n_experts * params.n)
        _l.check(L.hq_qmatmul_id_ggml_prepared(_stream(), _dev(input, "input"), _act_dtype(input),
                                               _dev(weight_stack, "weight_stack"), _dev(w_row_scales, "w_row_scales"),
                                               _dev(ids, "ids"), _dev(output, "output"), sp, sb, params.n_tokens, params.top_k,
                                               params.n, params.k, params.n_experts, params.expert_stride, params.ggml_type))
        return
    _l.check(L.hq_qmatmul_id_ggml(_stream(), _dev(input, "input"), _act_dtype(input),
                                  _dev(weight_stack, "weight_stack"), _dev(ids, "ids"), _dev(output, "output"),
                                  sp, sb, params.n_tokens, params.top_k, params.n, params.k, params.n_experts,
                                  params.expert_stride, params.ggml_type))


def quantized_matmul_id_swiglu_workspace_bytes(params) -> int:
    """Device scratch of quantized_matmul_id_swiglu_ggml for this shape; 0 where that form does not exist (the caller
    then runs gate, up and silu_mul as separate calls)."""
    return _l.load().hq_qmatmul_id_swiglu_ggml_workspace_bytes(params.n_tokens, params.top_k, params.n, params.k,
                                                               params.n_experts, params.expert_stride, params.ggml_type)


def quantized_matmul_id_swiglu_ggml(input: torch.Tensor, gate_stack: torch.Tensor, up_stack: torch.Tensor, ids: torch.Tensor,
                                    output: torch.Tensor, params: GgmlQuantizedMatmulIdParams, scratch: torch.Tensor,
                                    gate_row_scales: torch.Tensor | None = None,
                                    up_row_scales: torch.Tensor | None = None) -> None:
    """output[t, s, :] = silu(W_gate[ids[t, s]] . input[t]) * (W_up[ids[t, s]] . input[t]): phases B and D of the MoE
    block (gpu_ffn.rs:2546-2697) at prefill as one grouped product."""
    if output.dtype != torch.float32:
        raise TypeError("output must be float32")
    if ids.dtype not in (torch.int32, torch.uint32):
        raise TypeError("ids must be 32-bit")
    for s_ in (gate_row_scales, up_row_scales):
        if s_ is not None:
            _check_scales(s_, params.n_experts * params.n)
    L = _l.load()
    _l.check(L.hq_qmatmul_id_swiglu_ggml(
        _stream(), _dev(input, "input"), _act_dtype(input), _dev(gate_stack, "gate_stack"), _dev(up_stack, "up_stack"),
        _dev(gate_row_scales, "gate_row_scales") if gate_row_scales is not None else None,
        _dev(up_row_scales, "up_row_scales") if up_row_scales is not None else None, _dev(ids, "ids"), _dev(output, "output"),
        _dev(scratch, "scratch"), scratch.numel() * scratch.element_size(), params.n_tokens, params.top_k, params.n, params.k,
        params.n_experts, params.expert_stride, params.ggml_type))


@dataclass
class QmatmulJob:
    """One product of a batched launch: the arguments of quantized_matmul_id_ggml (ids set) or of
    quantized_matmul_ggml (ids None, m <= 8).  With `input_up` the activations are
    silu(input) * input_up, formed while they are staged."""
    input: torch.Tensor
    weight: torch.Tensor
    output: torch.Tensor
    rows: int
    n: int
    k: int
    ids: torch.Tensor | None = None
    top_k: int = 1
    n_experts: int = 1
    expert_stride: int = 0
    input_up: torch.Tensor | None = None
    # routing inside the launch (ids None): router logits [rows, n_experts] f32; the selection is also written to
    # route_ids / route_weights ([rows * top_k]) when given
    route_logits: torch.Tensor | None = None
    route_ids: torch.Tensor | None = None
    route_weights: torch.Tensor | None = None


def quantized_matmul_batch_ggml(jobs: list[QmatmulJob], ggml_type: int) -> None:
    """The dispatches of one phase of the MoE block, which the reference encodes without a barrier
    between them (gpu_ffn.rs:2485, 2546), as a single launch."""
    if not jobs:
        return
    arr = (_l.QmatmulJob * len(jobs))()
    for c, j in zip(arr, jobs):
        if j.output.dtype != torch.float32:
            raise TypeError("output must be float32")
        if _act_dtype(j.input) != _act_dtype(jobs[0].input):
            raise TypeError("all jobs of a batch share one activation dtype")
        if j.ids is not None and j.ids.dtype not in (torch.int32, torch.uint32):
            raise TypeError("ids must be 32-bit")
        if j.input_up is not None and j.input_up.dtype != torch.float32:
            raise TypeError("input_up must be float32")
        c.x, c.w, c.y = _dev(j.input, "input"), _dev(j.weight, "weight"), _dev(j.output, "output")
        c.x_up = _dev(j.input_up, "input_up") if j.input_up is not None else None
        c.ids = _dev(j.ids, "ids") if j.ids is not None else None
        if j.route_logits is not None and j.route_logits.dtype != torch.float32:
            raise TypeError("route_logits must be float32")
        c.route_logits = _dev(j.route_logits, "route_logits") if j.route_logits is not None else None
        c.route_ids = _dev(j.route_ids, "route_ids") if j.route_ids is not None else None
        c.route_weights = _dev(j.route_weights, "route_weights") if j.route_weights is not None else None
        c.rows, c.top_k, c.n, c.k, c.n_experts, c.expert_stride = j.rows, j.top_k, j.n, j.k, j.n_experts, j.expert_stride
    _l.check(_l.load().hq_qmatmul_batch_ggml(_stream(), arr, len(jobs), _act_dtype(jobs[0].input), ggml_type))


def id_scratch_bytes(n_experts: int, max_rows: int) -> int:
    return _l.load().hq_qmatmul_id_scratch_bytes(n_experts, max_rows)


def quantized_matmul_id_workspace_bytes(params) -> int:
    """Device scratch quantized_matmul_id_ggml(..., scratch=) can use for this shape (0: per-row GEMVs)."""
    return _l.load().hq_qmatmul_id_ggml_workspace_bytes(params.n_tokens, params.top_k, params.n, params.k,
                                                        params.n_experts, params.expert_stride, params.ggml_type)


def dequantize_ggml(weight: torch.Tensor, n_elems: int, ggml_type: int,
                    dtype: torch.dtype = torch.float32) -> torch.Tensor:
    out = torch.empty(n_elems, dtype=dtype, device=weight.device)
    L = _l.load()
    odt = _l.HQ_F16 if dtype == torch.float16 else _act_dtype(out)  # f16: the output dtype of the F16 shadow only
    _l.check(L.hq_dequant_ggml(_stream(), _dev(weight, "weight"), _dev(out, "out"), odt, n_elems, ggml_type))
    return out


def _quantize_ggml_imatrix(src: torch.Tensor, n_per_row: int, ggml_type: int, imatrix: torch.Tensor) -> torch.Tensor:
    if src.dtype != torch.float32 or imatrix.dtype != torch.float32:
        raise TypeError("src and imatrix must be float32")
    if imatrix.numel() != n_per_row:
        raise ValueError("imatrix length must equal n_per_row")  # QuantizeError::ImatrixLenMismatch
    n = src.numel()
    be, bb = BLOCK_ELEMS[ggml_type], BLOCK_BYTES[ggml_type]
    if n_per_row % be or n % n_per_row:
        raise ValueError(f"n_per_row {n_per_row} / len {n} not aligned to block {be}")
    L = _l.load()
    out = torch.empty(n // be * bb, dtype=torch.uint8, device=src.device)
    need = int(L.hq_quantize_ggml_imatrix_scratch_bytes(n, n_per_row, ggml_type))
    scratch = torch.empty(need, dtype=torch.uint8, device=src.device) if need else None
    _l.check(L.hq_quantize_ggml_imatrix(_stream(), _dev(src, "src"), n, n_per_row, ggml_type, _dev(imatrix, "imatrix"), _dev(out, "out"),
                                        _dev(scratch, "scratch") if need else None, need))
    return out


def matmul_f16_shadow_workspace_bytes(m: int, n: int, k: int) -> int:
    return int(_l.load().hq_matmul_f16_shadow_workspace_bytes(m, n, k))


def matmul_f16_shadow(input: torch.Tensor, weight_f16: torch.Tensor, dst: torch.Tensor, m: int, n: int, k: int,
                      workspace: torch.Tensor) -> None:
    """dispatch_mm_v2_f16 (forward_mlx.rs:9790-9817): dst[m, n] = input[m, k] . weight_f16[n, k]^T over the F16 shadow of a
    weight (dequantize_ggml(..., dtype=torch.float16)); f32 or bf16 activations, f32 output, the vendor library's GEMM."""
    if weight_f16.dtype != torch.float16 or weight_f16.numel() < n * k:
        raise ValueError("weight_f16 must hold n * k float16 values")
    if dst.dtype != torch.float32 or dst.numel() < m * n or input.numel() < m * k:
        raise ValueError("dst must hold m * n float32 values and input m * k activations")
    if workspace.dtype != torch.uint8:
        raise TypeError("workspace must be a uint8 tensor")
    _l.check(_l.load().hq_matmul_f16_shadow(_stream(), _dev(input, "input"), _act_dtype(input), _dev(weight_f16, "weight_f16"),
                                            _dev(dst, "dst"), m, n, k, _dev(workspace, "workspace"), workspace.numel()))


# GGML ids of the two plain element types a weight tensor may have (ggml_type.rs:18-53).
GGML_F32, GGML_F16 = 0, 1


def dense_matmul_workspace_bytes(m: int, n: int, k: int, act_dtype: torch.dtype, weight_dtype: torch.dtype) -> int:
    xdt = HQ_BF16 if act_dtype == torch.bfloat16 else HQ_F32
    wdt = HQ_F16 if weight_dtype == torch.float16 else HQ_F32
    return int(_l.load().hq_dense_matmul_workspace_bytes(m, n, k, xdt, wdt))


def dense_matmul(input: torch.Tensor, weight: torch.Tensor, dst: torch.Tensor, m: int, n: int, k: int,
                 workspace: torch.Tensor | None = None) -> None:
    """The branches of dispatch_qmatmul for weights that are not quantized (forward_mlx.rs:9820-9917): dst[m, n] =
    input[m, k] . weight[n, k]^T for float32 or float16 weights, f32 or bf16 activations, f32 output.  Up to eight rows are
    streaming passes over the weights (dispatch_dense_matvec_f32 / dispatch_dense_matvec_f16w_f32io), more rows the vendor
    library's GEMM (dense_matmul_f32_f32_tensor / dispatch_mm_v2_f16)."""
    if weight.dtype not in (torch.float32, torch.float16) or weight.numel() < n * k:
        raise ValueError("weight must hold n * k float32 or float16 values")
    if dst.dtype != torch.float32 or dst.numel() < m * n or input.numel() < m * k:
        raise ValueError("dst must hold m * n float32 values and input m * k activations")
    need = dense_matmul_workspace_bytes(m, n, k, input.dtype, weight.dtype)
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=input.device)
    wdt = HQ_F16 if weight.dtype == torch.float16 else HQ_F32
    _l.check(_l.load().hq_dense_matmul(_stream(), _dev(input, "input"), _act_dtype(input), _dev(weight, "weight"), wdt, _dev(dst, "dst"),
                                       m, n, k, _dev(workspace, "workspace") if need else None, workspace.numel() if need else 0))


# Above this many activation rows dispatch_qmatmul takes the matrix-matrix routes (mlx-native's MM_ROUTING_THRESHOLD,
# forward_mlx.rs:9791).
MM_ROUTING_THRESHOLD = 8


@dataclass
class MlxQWeight:
    """A linear weight as dispatch_qmatmul sees it (forward_mlx.rs:340-402): the raw GGML blocks with their type and
    shape (QuantWeightInfo: rows = n, cols = k) and, optionally, the weight's F16 shadow; or, with ggml_dtype GGML_F32 /
    GGML_F16, the tensor's plain float32 / float16 values."""
    buffer: torch.Tensor
    ggml_dtype: int
    rows: int
    cols: int
    f16_shadow: torch.Tensor | None = None

    def matmul_params(self, m: int) -> GgmlQuantizedMatmulParams:
        """forward_mlx.rs:408-415."""
        return GgmlQuantizedMatmulParams(m, self.rows, self.cols, self.ggml_dtype)

    def populate_f16_shadow(self) -> None:
        """populate_f16_shadow_if_enabled / materialize_f16_shadow (forward_mlx.rs:9403-9440): the blocks dequantised once to
        f16 [rows, cols], kept beside them (2 bytes per weight more)."""
        self.f16_shadow = dequantize_ggml(self.buffer, self.rows * self.cols, self.ggml_dtype, dtype=torch.float16)


def dispatch_qmatmul(input: torch.Tensor, weight: MlxQWeight, output: torch.Tensor, m: int,
                     workspace: torch.Tensor | None = None) -> None:
    """dispatch_qmatmul (forward_mlx.rs:9655-9969): float32 / float16 weights take the dense products (:9820-9917); more than
    MM_ROUTING_THRESHOLD rows over a block weight with an F16 shadow the dense f16 product (:9790-9817); everything else the
    quantized product, whose own routing by m (GEMV, small-batch, tile kernels) is the library's.  `workspace`: device scratch for the route taken
    (matmul_f16_shadow_workspace_bytes / quantized_matmul_workspace_bytes); allocated here when absent."""
    n, k = weight.rows, weight.cols
    if weight.ggml_dtype in (GGML_F32, GGML_F16):  # :9820-9917
        want = torch.float32 if weight.ggml_dtype == GGML_F32 else torch.float16
        if weight.buffer.dtype != want:
            raise TypeError(f"a weight of ggml type {weight.ggml_dtype} must be a {want} tensor")
        return dense_matmul(input, weight.buffer, output, m, n, k, workspace)
    if m > MM_ROUTING_THRESHOLD and weight.f16_shadow is not None:
        need = matmul_f16_shadow_workspace_bytes(m, n, k)
        if workspace is None or workspace.numel() * workspace.element_size() < need:
            workspace = torch.empty(need, dtype=torch.uint8, device=input.device)
        return matmul_f16_shadow(input, weight.f16_shadow, output, m, n, k, workspace)
    quantized_matmul_ggml(input, weight.buffer, output, weight.matmul_params(m), workspace=workspace)


def stream_read_probe(buf: torch.Tensor, sink: torch.Tensor) -> None:
    """One plain streaming read of `buf` (hq_stream_read_probe): what moving that many bytes costs on this device."""
    _l.check(_l.load().hq_stream_read_probe(_stream(), _dev(buf, "buf"), buf.numel() * buf.element_size(), _dev(sink, "sink")))


def quantize_ggml(src: torch.Tensor, n_per_row: int, ggml_type: int, imatrix: torch.Tensor | None = None) -> torch.Tensor:
    """f32 rows -> packed GGML blocks on the device (GgmlQuantizer::quantize, quantizer.rs:51-102); `imatrix`: n_per_row
    float32 importance weights on the device, or None."""
    if imatrix is not None:
        return _quantize_ggml_imatrix(src, n_per_row, ggml_type, imatrix)
    if src.dtype != torch.float32:
        raise TypeError("src must be float32")
    n = src.numel()
    be, bb = BLOCK_ELEMS[ggml_type], BLOCK_BYTES[ggml_type]
    out = torch.empty(n // be * bb if n % be == 0 else 0, dtype=torch.uint8, device=src.device)
    L = _l.load()
    _l.check(L.hq_quantize_ggml(_stream(), _dev(src, "src"), n, n_per_row, ggml_type, _dev(out, "out")))
    return out


# ---- GGUF files ------------------------------------------------------------------------------------

@dataclass(frozen=True)
class QuantWeightInfo:
    """forward_mlx.rs:395-415 (MlxQWeight.info): what the matmul call sites need to know about a loaded
    tensor.  `shape` is in GGUF order (innermost first)."""
    ggml_dtype: int
    rows: int
    cols: int
    shape: tuple
    byte_len: int


class GgufFile:
    """The reader hf2q opens its model files with (mlx_native::gguf::GgufFile as used in
    serve/gpu.rs:157-167 and qwen35/weight_loader.rs:52-118): tensor directory, metadata, and the raw
    GGML blocks of a tensor uploaded to the device."""

    def __init__(self, path: str):
        h = ctypes.c_void_p()
        _l.check(_l.load().hq_gguf_open(os.fsencode(path), ctypes.byref(h)))
        self._h = h

    @classmethod
    def open(cls, path: str) -> "GgufFile":
        return cls(path)

    def close(self) -> None:
        if self._h:
            _l.load().hq_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def tensor_count(self) -> int:
        return _l.load().hq_gguf_tensor_count(self._h)

    def metadata_count(self) -> int:
        return _l.load().hq_gguf_metadata_count(self._h)

    def tensor_names(self) -> list:
        L = _l.load()
        return [L.hq_gguf_tensor_name(self._h, i).decode() for i in range(self.tensor_count())]

    def metadata_keys(self) -> list:
        L = _l.load()
        return [L.hq_gguf_metadata_key(self._h, i).decode() for i in range(self.metadata_count())]

    def tensor_info(self, name: str) -> QuantWeightInfo:
        ti = _l.GgufTensorInfo()
        _l.check(_l.load().hq_gguf_tensor_info_by_name(self._h, name.encode(), ctypes.byref(ti)))
        shape = tuple(ti.dims[i] for i in range(ti.n_dims))
        cols = shape[0] if shape else 1
        rows = 1
        for d in shape[1:]:
            rows *= d
        return QuantWeightInfo(ti.ggml_type, rows, cols, shape, ti.byte_len)

    def metadata_u64(self, key: str) -> int:
        v = ctypes.c_uint64()
        _l.check(_l.load().hq_gguf_metadata_u64(self._h, key.encode(), ctypes.byref(v)))
        return v.value

    def metadata_f64(self, key: str) -> float:
        v = ctypes.c_double()
        _l.check(_l.load().hq_gguf_metadata_f64(self._h, key.encode(), ctypes.byref(v)))
        return v.value

    def metadata_string(self, key: str) -> str:
        p, n = ctypes.c_void_p(), ctypes.c_uint64()
        _l.check(_l.load().hq_gguf_metadata_string(self._h, key.encode(), ctypes.byref(p), ctypes.byref(n)))
        return ctypes.string_at(p.value, n.value).decode()

    def tensor_bytes(self, name: str) -> bytes:
        """The tensor's raw bytes from the host mapping (tests, CPU-side consumers)."""
        n = ctypes.c_uint64()
        p = _l.load().hq_gguf_tensor_data(self._h, name.encode(), ctypes.byref(n))
        if not p:
            raise _l.HqError(_l.HQ_ERR_INVALID_ARGUMENT, _l.last_error())
        return ctypes.string_at(p, n.value)

    def load_tensor(self, name: str, device) -> torch.Tensor:
        """Raw GGML blocks of `name` as a uint8 device tensor (weight_loader.rs:52-118); the matmul entry
        points take it as is.  For an expert stack, expert_stride = byte_len // shape[2]."""
        info = self.tensor_info(name)
        buf = torch.empty(info.byte_len, dtype=torch.uint8, device=device)
        with torch.cuda.device(buf.device):
            _l.check(_l.load().hq_gguf_load_tensor(self._h, name.encode(), _stream(), _dev(buf, name), info.byte_len))
        return buf

    def load_weight(self, name: str, device) -> "MlxQWeight":
        """The tensor as dispatch_qmatmul takes it (MlxQWeight, forward_mlx.rs:340-402): raw blocks for the block types, the
        values themselves for F32 / F16 tensors (router projections, tensors whose rows are not whole super-blocks)."""
        info = self.tensor_info(name)
        buf = self.load_tensor(name, device)
        if info.ggml_dtype == GGML_F32:
            buf = buf.view(torch.float32)
        elif info.ggml_dtype == GGML_F16:
            buf = buf.view(torch.float16)
        return MlxQWeight(buf, info.ggml_dtype, info.rows, info.cols)


# ---- TurboQuant-style 8-bit KV cache ------------------------------------------------------------

@dataclass(frozen=True)
class FlashAttnVecTqHbParams:
    """forward_mlx.rs:4687-4705 / kv_cache.rs:589-614 (Qwen35TqSdpaParams)."""
    num_heads: int
    num_kv_heads: int
    head_dim: int
    kv_seq_len: int
    kv_capacity: int
    scale: float
    mask_type: int = 0
    sliding_window: int = 0
    softcap: float = 0.0
    ring_start: int = 0
    scale_factor_d512: float = 1.0
    codebook_bits: int = 8
    fuse_fwht_pre: int = 0
    nsg: int = 1


def dispatch_fwht_sign_premult_f32(buf: torch.Tensor, num_heads: int, head_dim: int) -> None:
    """forward_mlx.rs:4662-4666: in-place sign x FWHT of buf[num_heads, head_dim] (f32)."""
    if buf.dtype != torch.float32:
        raise TypeError("buf must be float32")
    _l.check(_l.load().hq_fwht_sign_premult_f32(_stream(), _dev(buf, "buf"), num_heads, head_dim))


def dispatch_fwht_sign_undo_f32(buf: torch.Tensor, num_heads: int, head_dim: int) -> None:
    """forward_mlx.rs:4750: in-place FWHT x sign."""
    if buf.dtype != torch.float32:
        raise TypeError("buf must be float32")
    _l.check(_l.load().hq_fwht_sign_undo_f32(_stream(), _dev(buf, "buf"), num_heads, head_dim))


def alloc_tq_kv(n_kv_heads: int, capacity: int, head_dim: int, device) -> tuple[torch.Tensor, torch.Tensor]:
    """kv_cache.rs:2026-2113: codes [n_kv_heads, capacity, head_dim] u8 + norms [.., head_dim/256] f32."""
    codes = torch.zeros((n_kv_heads, capacity, head_dim), dtype=torch.uint8, device=device)
    norms = torch.zeros((n_kv_heads, capacity, max(1, head_dim // 256)), dtype=torch.float32, device=device)
    return codes, norms


def hadamard_quantize_kv(src: torch.Tensor, codes: torch.Tensor, norms: torch.Tensor, write_pos: int) -> None:
    """kv_cache.rs:180-213: encode src [n_tokens, n_kv_heads, head_dim] f32 at slots write_pos.. of the cache."""
    if src.dtype != torch.float32 or codes.dtype != torch.uint8 or norms.dtype != torch.float32:
        raise TypeError("src f32, codes u8, norms f32 expected")
    n_tokens, n_kv_heads, head_dim = src.shape
    capacity = codes.shape[1]
    _l.check(_l.load().hq_tq_encode_kv(_stream(), _dev(src, "src"), _dev(codes, "codes"), _dev(norms, "norms"),
                                       n_tokens, n_kv_heads, head_dim, capacity, write_pos))


def tq_tmp_buffer_bytes(num_heads: int, head_dim: int, kv_seq_len: int) -> int:
    return _l.load().hq_flash_attn_vec_tq_tmp_bytes(num_heads, head_dim, kv_seq_len)


def flash_attn_vec_tq_hb(q: torch.Tensor, k_packed: torch.Tensor, k_norms: torch.Tensor, v_packed: torch.Tensor,
                         v_norms: torch.Tensor, out: torch.Tensor, tmp: torch.Tensor, params: FlashAttnVecTqHbParams,
                         lut256: torch.Tensor | None = None, undo_rotation: bool = False) -> None:
    """forward_mlx.rs:4732-4742: single-query attention over the 8-bit cache (rotated domain in and out).
    undo_rotation: the merge pass also applies dispatch_fwht_sign_undo_f32 to `out` (forward_mlx.rs:4744-4760)."""
    if q.dtype != torch.float32 or out.dtype != torch.float32:
        raise TypeError("q and out must be float32")
    p = _l.TqAttnParams(params.num_heads, params.num_kv_heads, params.head_dim, params.kv_seq_len,
                        params.kv_capacity, params.scale, params.mask_type, params.sliding_window, params.softcap,
                        params.ring_start, params.scale_factor_d512, params.codebook_bits, params.fuse_fwht_pre,
                        params.nsg)
    import ctypes as _ct
    fn = _l.load().hq_flash_attn_vec_tq_undo if undo_rotation else _l.load().hq_flash_attn_vec_tq
    _l.check(fn(
        _stream(), _dev(q, "q"), _dev(k_packed, "k_packed"), _dev(k_norms, "k_norms"), _dev(v_packed, "v_packed"),
        _dev(v_norms, "v_norms"), _dev(lut256, "lut256") if lut256 is not None else None, _dev(out, "out"),
        _dev(tmp, "tmp"), tmp.numel() * tmp.element_size(), _ct.byref(p)))


def flash_attn_vec_tq_hb_static(q: torch.Tensor, k_packed: torch.Tensor, k_norms: torch.Tensor, v_packed: torch.Tensor,
                                v_norms: torch.Tensor, out: torch.Tensor, params: FlashAttnVecTqHbParams,
                                lut256: torch.Tensor | None = None, undo_rotation: bool = False) -> None:
    """flash_attn_vec_tq_hb without the tmp argument: the partial results go to the library's static device buffer
    (hq_flash_attn_vec_tq_static; nothing is allocated, shapes beyond the buffer are rejected)."""
    if q.dtype != torch.float32 or out.dtype != torch.float32:
        raise TypeError("q and out must be float32")
    p = _l.TqAttnParams(params.num_heads, params.num_kv_heads, params.head_dim, params.kv_seq_len,
                        params.kv_capacity, params.scale, params.mask_type, params.sliding_window, params.softcap,
                        params.ring_start, params.scale_factor_d512, params.codebook_bits, params.fuse_fwht_pre,
                        params.nsg)
    import ctypes as _ct
    _l.check(_l.load().hq_flash_attn_vec_tq_static(
        _stream(), _dev(q, "q"), _dev(k_packed, "k_packed"), _dev(k_norms, "k_norms"), _dev(v_packed, "v_packed"),
        _dev(v_norms, "v_norms"), _dev(lut256, "lut256") if lut256 is not None else None, _dev(out, "out"),
        _ct.byref(p), 1 if undo_rotation else 0))


def tq_dequantize_hb_kv_seq(packed: torch.Tensor, norms: torch.Tensor, dst: torch.Tensor, n_kv_heads: int, head_dim: int,
                            cache_capacity: int, start_pos: int, n_tokens: int, scale_factor_d512: float = 1.0,
                            codebook_bits: int = 8, lut256: torch.Tensor | None = None, unrotate: bool = False) -> None:
    """kv_cache.rs:431-495 (dequant_seq_to_temp_f32) / :497-583 (…_unrotated): cache positions
    start_pos .. start_pos + n_tokens - 1 as f32 [n_kv_heads, n_tokens, head_dim]."""
    if dst.dtype != torch.float32 or dst.numel() < n_kv_heads * n_tokens * head_dim:
        raise TypeError("dst must be float32 [n_kv_heads, n_tokens, head_dim]")
    _l.check(_l.load().hq_tq_dequantize_kv_seq(
        _stream(), _dev(packed, "packed"), _dev(norms, "norms"), _dev(lut256, "lut256") if lut256 is not None else None,
        _dev(dst, "dst"), n_kv_heads, head_dim, cache_capacity, start_pos, n_tokens, scale_factor_d512, codebook_bits,
        1 if unrotate else 0))


@dataclass
class TqPackedHeader:
    """TqPackedV1Header / TqPackedV2Header (kv_persist/families/tq_packed.rs:129-153, 376-396)."""
    codec_version: int
    bits_per_coord: int
    head_dim: int
    n_kv_heads: int
    n_tokens: int
    flags: int = 0
    scale: float = 1.0

    def _c(self):
        return _l.TqpHeader(self.codec_version, self.bits_per_coord, self.head_dim, self.n_kv_heads, self.n_tokens,
                            self.flags, self.scale)

    def indices_bytes_len(self) -> int:
        import ctypes as _ct
        return _l.load().hq_tqp_indices_bytes(_ct.byref(self._c()))

    def norms_bytes_len(self) -> int:
        import ctypes as _ct
        return _l.load().hq_tqp_norms_bytes(_ct.byref(self._c()))

    def total_bytes(self) -> int:
        import ctypes as _ct
        return _l.load().hq_tqp_total_bytes(_ct.byref(self._c()))


def pack_tq_payload(header: TqPackedHeader, indices: bytes, norms_le: bytes = b"") -> bytes:
    """pack_tq_v1_payload / pack_tq_v2_payload (tq_packed.rs:199-226, 459-489)."""
    import ctypes as _ct
    out = _ct.create_string_buffer(max(1, header.total_bytes()))
    _l.check(_l.load().hq_tqp_pack(_ct.byref(header._c()), bytes(indices), len(indices), bytes(norms_le), len(norms_le),
                                   out, header.total_bytes()))
    return out.raw[:header.total_bytes()]


def unpack_tq_payload(payload: bytes):
    """unpack_tq_v1_payload / unpack_tq_v2_payload (tq_packed.rs:243-311, 491-566): (header, indices, norms)."""
    import ctypes as _ct
    h = _l.TqpHeader()
    io, no = _ct.c_size_t(), _ct.c_size_t()
    _l.check(_l.load().hq_tqp_unpack(bytes(payload), len(payload), _ct.byref(h), _ct.byref(io), _ct.byref(no)))
    hdr = TqPackedHeader(h.codec_version, h.bits_per_coord, h.head_dim, h.n_kv_heads, h.n_tokens, h.flags, h.scale)
    return hdr, payload[io.value:no.value], payload[no.value:]


def capture_tq_kv(packed: torch.Tensor, norms: torch.Tensor, n_kv_heads: int, head_dim: int, capacity: int,
                  start_pos: int, n_tokens: int) -> bytes:
    """A version-2 envelope of cache positions start_pos .. start_pos + n_tokens - 1 (tq_packed.rs:568-590)."""
    import ctypes as _ct
    need = _l.load().hq_tq_kv_capture_bytes(n_kv_heads, head_dim, n_tokens)
    out = _ct.create_string_buffer(need)
    _l.check(_l.load().hq_tq_kv_capture(_stream(), _dev(packed, "packed"), _dev(norms, "norms"), n_kv_heads, head_dim,
                                        capacity, start_pos, n_tokens, out, need))
    return out.raw[:need]


def restore_tq_kv(payload: bytes, packed: torch.Tensor, norms: torch.Tensor, n_kv_heads: int, head_dim: int,
                  capacity: int, start_pos: int) -> None:
    """Writes an envelope's indices and norms back into the cache at start_pos."""
    _l.check(_l.load().hq_tq_kv_restore(_stream(), bytes(payload), len(payload), _dev(packed, "packed"),
                                        _dev(norms, "norms"), n_kv_heads, head_dim, capacity, start_pos))


# ---- MoE FFN block ------------------------------------------------------------------------------

def dense_gemv_bf16_f32(x: torch.Tensor, w_bf16: torch.Tensor, y: torch.Tensor, m: int, n: int, k: int) -> None:
    """gpu_ffn.rs:597-617: y[m,n] = x[m,k] . W[n,k]^T with bf16 weights."""
    _l.check(_l.load().hq_dense_gemv_bf16(_stream(), _dev(x, "x"), _act_dtype(x), _dev(w_bf16, "w"), _dev(y, "y"), m, n, k))


def dense_gemv_bf16_f32_pair(x: torch.Tensor, w_a: torch.Tensor, y_a: torch.Tensor, n_a: int, w_b: torch.Tensor,
                             y_b: torch.Tensor, n_b: int, m: int, k: int) -> None:
    """Two dense_gemv_bf16_f32 dispatches over the same activations (router + shared gate logit,
    gpu_ffn.rs:2485) in one launch."""
    _l.check(_l.load().hq_dense_gemv_bf16_pair(_stream(), _dev(x, "x"), _act_dtype(x), _dev(w_a, "w_a"), _dev(y_a, "y_a"),
                                               n_a, _dev(w_b, "w_b"), _dev(y_b, "y_b"), n_b, m, k))


def dispatch_moe_softmax_topk(logits: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, n_tokens: int,
                              n_experts: int, top_k: int) -> None:
    _l.check(_l.load().hq_moe_softmax_topk(_stream(), _dev(logits, "logits"), _dev(ids, "ids"), _dev(weights, "weights"),
                                           n_tokens, n_experts, top_k))


def dispatch_silu_mul(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor) -> None:
    _l.check(_l.load().hq_silu_mul(_stream(), _dev(gate, "gate"), _dev(up, "up"), _dev(out, "out"), gate.numel()))


def dispatch_moe_weighted_reduce(y: torch.Tensor, w: torch.Tensor, out: torch.Tensor, n_tokens: int, top_k: int,
                                 hidden: int, shared: torch.Tensor | None = None,
                                 shared_logit: torch.Tensor | None = None, residual: torch.Tensor | None = None) -> None:
    o = lambda t, nm: _dev(t, nm) if t is not None else None  # noqa: E731
    _l.check(_l.load().hq_moe_weighted_reduce(_stream(), _dev(y, "y"), _dev(w, "w"), o(shared, "shared"),
                                              o(shared_logit, "shared_logit"), o(residual, "residual"), _dev(out, "out"),
                                              n_tokens, top_k, hidden))


@dataclass
class DenseFfnWeightsGpuQ:
    """gpu_ffn.rs:260-280: gate / up `[inter, hidden]` and down `[hidden, inter]` as raw GGML blocks."""
    gate_q: torch.Tensor
    up_q: torch.Tensor
    down_q: torch.Tensor
    ggml_type: int
    hidden: int
    inter: int
    down_type: int | None = None  # the down matrix's type where it differs from gate / up (Q6_K in Q4_K_M / Q5_K_M files)


def dense_ffn_decode_scratch_bytes(w: "DenseFfnWeightsGpuQ", act_dtype: torch.dtype) -> int:
    """Bytes of zeroed device scratch dense_ffn_decode needs for this layer; 0: the one-launch form does not take it."""
    xdt = HQ_BF16 if act_dtype == torch.bfloat16 else HQ_F32
    dt = w.down_type if w.down_type is not None else w.ggml_type
    return int(_l.load().hq_dense_ffn_decode_scratch_bytes(w.hidden, w.inter, w.ggml_type, dt, xdt))


def dense_ffn_decode(x: torch.Tensor, w: "DenseFfnWeightsGpuQ", out: torch.Tensor, scratch: torch.Tensor,
                     residual: torch.Tensor | None = None) -> None:
    """build_dense_ffn_layer_gpu_q (gpu_ffn.rs:1017-1351) for ONE token as one launch: out = down(silu(gate x) * (up x))
    (+ residual).  `scratch`: dense_ffn_decode_scratch_bytes() bytes, zeroed once by the caller (torch.zeros), then left
    to the library; the bits of the separate dispatches."""
    if x.numel() != w.hidden or out.numel() != w.hidden:
        raise ValueError("dense_ffn_decode takes one token: x and out of `hidden` values")
    dt = w.down_type if w.down_type is not None else w.ggml_type
    _l.check(_l.load().hq_dense_ffn_decode(_stream(), _dev(x, "x"), _act_dtype(x), _dev(w.gate_q, "gate"), _dev(w.up_q, "up"),
                                           _dev(w.down_q, "down"), w.ggml_type, dt,
                                           _dev(residual, "residual") if residual is not None else None, _dev(out, "out"),
                                           w.hidden, w.inter, _dev(scratch, "scratch"), scratch.numel() * scratch.element_size()))


def handover_status(scratch: torch.Tensor) -> int:
    """The error word of a scratch of dense_ffn_decode / moe_ffn_decode_fused (0: fine); synchronises the stream."""
    err = ctypes.c_uint32(0)
    _l.check(_l.load().hq_handover_status(_stream(), _dev(scratch, "scratch"), ctypes.byref(err)))
    return int(err.value)


def dense_ffn_workspace_bytes(w: "DenseFfnWeightsGpuQ", m: int, act_dtype: torch.dtype) -> int:
    """Device scratch build_dense_ffn_layer_gpu_q_into(..., workspace=) needs for m rows (0: none needed)."""
    return max(quantized_matmul_workspace_bytes(GgmlQuantizedMatmulParams(m, w.inter, w.hidden, w.ggml_type), act_dtype),
               quantized_matmul_workspace_bytes(GgmlQuantizedMatmulParams(m, w.hidden, w.inter, w.down_type if w.down_type is not None else w.ggml_type), torch.float32))


def build_dense_ffn_layer_gpu_q_into(x: torch.Tensor, w: DenseFfnWeightsGpuQ, gate_buf: torch.Tensor,
                                     up_buf: torch.Tensor, act_buf: torch.Tensor | None, out: torch.Tensor,
                                     batched: bool | None = None, workspace: torch.Tensor | None = None) -> None:
    """gpu_ffn.rs:1086-1330: out = down(silu(gate x) * (up x)) for seq_len rows of x.  The reference encodes gate
    and up back to back (one barrier after both), then silu_mul, then down.  `batched` (default: whenever the
    row count is decode-sized) hands gate + up to the library as one launch and folds the SwiGLU into the
    staging of the down projection (for inter <= 8192): two launches instead of four, identical results."""
    m = x.shape[0]
    H, I, t = w.hidden, w.inter, w.ggml_type
    td = w.down_type if w.down_type is not None else t
    if batched is None:
        batched = m <= _BATCH_MAX_DENSE_ROWS
    if batched:
        if m > _BATCH_MAX_DENSE_ROWS:
            raise ValueError(f"batched dense FFN: {m} rows (limit {_BATCH_MAX_DENSE_ROWS})")
        pgu = GgmlQuantizedMatmulParams(m, I, H, t)
        if act_buf is not None and quantized_matmul_swiglu_decode_supported(pgu, x.dtype):
            # gate, up and the SwiGLU as one launch per row, then down over the f32 activations: two launches at batch 1
            quantized_matmul_swiglu_decode(x, w.gate_q, w.up_q, act_buf, pgu)
            quantized_matmul_ggml(act_buf, w.down_q, out, GgmlQuantizedMatmulParams(m, H, I, td))
            return
        quantized_matmul_batch_ggml([QmatmulJob(x, w.gate_q, gate_buf, m, I, H), QmatmulJob(x, w.up_q, up_buf, m, I, H)], t)
        # Every workgroup of the fused down projection forms the whole activation vector itself; past a few
        # thousand activations a separate SwiGLU pass is as fast (measured equal at 12288).
        if I <= _FUSED_SWIGLU_MAX_K or act_buf is None:
            quantized_matmul_batch_ggml([QmatmulJob(gate_buf, w.down_q, out, m, H, I, input_up=up_buf)], td)
        else:
            dispatch_silu_mul(gate_buf[:m], up_buf[:m], act_buf[:m])
            quantized_matmul_ggml(act_buf, w.down_q, out, GgmlQuantizedMatmulParams(m, H, I, td))
        return
    pgu, pdn = GgmlQuantizedMatmulParams(m, I, H, t), GgmlQuantizedMatmulParams(m, H, I, td)
    if workspace is not None and quantized_matmul_gated_workspace_bytes(pgu, x.dtype):
        # a prefill chunk with caller scratch (dense_ffn_workspace_bytes): nothing is allocated, and the up projection
        # finishes the gating in its epilogue -- no SwiGLU pass over both products (the same bits)
        quantized_matmul_ggml(x, w.gate_q, gate_buf, pgu, workspace=workspace)
        quantized_matmul_gated_ggml(x, w.up_q, gate_buf, act_buf, pgu, workspace)
        quantized_matmul_ggml(act_buf, w.down_q, out, pdn, workspace=workspace)
        return
    quantized_matmul_ggml(x, w.gate_q, gate_buf, pgu, workspace=workspace)
    quantized_matmul_ggml(x, w.up_q, up_buf, pgu, workspace=workspace)
    dispatch_silu_mul(gate_buf[:m], up_buf[:m], act_buf[:m])
    quantized_matmul_ggml(act_buf, w.down_q, out, pdn, workspace=workspace)


@dataclass
class MoeFfnWeightsGpuQ:
    """Device weights of one quantized MoE FFN layer (gpu_ffn.rs:214-358): router and shared-gate logit in
    bf16, expert stacks and the shared expert as raw GGML blocks."""
    router: torch.Tensor             # [n_experts, hidden] bf16
    expert_gate: torch.Tensor        # stack [n_experts][inter][hidden/QK] blocks
    expert_up: torch.Tensor
    expert_down: torch.Tensor        # stack [n_experts][hidden][inter/QK] blocks
    shared_gate_logit: torch.Tensor  # [1, hidden] bf16
    shared_gate: torch.Tensor        # [shared_inter][hidden/QK] blocks
    shared_up: torch.Tensor
    shared_down: torch.Tensor        # [hidden][shared_inter/QK] blocks
    ggml_type: int
    hidden: int
    n_experts: int
    top_k: int
    inter: int
    shared_inter: int
    # the tile kernels' weight-row scales of the six quantized matrices, filled by prepare_prefill() (optional)
    row_scales: dict | None = None
    # type of expert_down / shared_down where it differs from ggml_type (Qwen3.6-35B-A3B: gate / up Q5_K, down Q6_K)
    down_type: int | None = None

    @property
    def td(self) -> int:
        return self.down_type if self.down_type is not None else self.ggml_type

    def c_layer(self) -> "_l.MoeFfnLayer":
        """hq_moe_ffn_layer of these weights (contiguous stacks)."""
        rb_h, rb_i = ggml_row_bytes(self.ggml_type, self.hidden), ggml_row_bytes(self.td, self.inter)
        return _l.MoeFfnLayer(_dev(self.router, "router"), _dev(self.shared_gate_logit, "shared_gate_logit"),
                              _dev(self.expert_gate, "expert_gate"), _dev(self.expert_up, "expert_up"), _dev(self.expert_down, "expert_down"),
                              _dev(self.shared_gate, "shared_gate"), _dev(self.shared_up, "shared_up"), _dev(self.shared_down, "shared_down"),
                              self.hidden, self.n_experts, self.top_k, self.inter, self.shared_inter, self.ggml_type, self.inter * rb_h,
                              self.hidden * rb_i, 0 if self.down_type is None else self.down_type)

    def prepare_prefill(self) -> None:
        """Once after the weights are uploaded: the row scales that prefill-sized calls would otherwise work out again in
        every pre-pass (4 bytes per weight row; they depend on the weights alone, so the results do not change)."""
        t, td, H, E, I, SI = self.ggml_type, self.td, self.hidden, self.n_experts, self.inter, self.shared_inter
        if t not in (HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, HQ_Q4_0):
            return
        self.row_scales = {
            "expert_gate": weight_row_scales_ggml(self.expert_gate, E * I, H, t),
            "expert_up": weight_row_scales_ggml(self.expert_up, E * I, H, t),
            "expert_down": weight_row_scales_ggml(self.expert_down, E * H, I, td),
            "shared_gate": weight_row_scales_ggml(self.shared_gate, SI, H, t),
            "shared_up": weight_row_scales_ggml(self.shared_up, SI, H, t),
            "shared_down": weight_row_scales_ggml(self.shared_down, H, SI, td),
        }


class MoeFfnScratch:
    """Caller-owned activations of the block for up to `max_tokens` tokens (the decode pool of
    decode_pool.rs, allocated once)."""

    def __init__(self, w: MoeFfnWeightsGpuQ, max_tokens: int, device):
        f = lambda *s: torch.empty(*s, dtype=torch.float32, device=device)  # noqa: E731
        T, K = max_tokens, w.top_k
        self.logits, self.sh_logit = f(T, w.n_experts), f(T, 1)
        self.ids = torch.empty(T * K, dtype=torch.int32, device=device)
        self.topk_w = f(T * K)
        self.gate, self.up, self.act = f(T * K, w.inter), f(T * K, w.inter), f(T * K, w.inter)
        self.down = f(T * K, w.hidden)
        self.sh_gate, self.sh_up, self.sh_act = f(T, w.shared_inter), f(T, w.shared_inter), f(T, w.shared_inter)
        self.sh_down = f(T, w.hidden)
        # workspace of the grouped (expert-sorted) form that prefill-sized mul_mat_id calls take (IdMmScratch, decode_pool.rs:56-60)
        rb_h, rb_i = ggml_row_bytes(w.ggml_type, w.hidden), ggml_row_bytes(w.td, w.inter)
        need = max(
            quantized_matmul_id_swiglu_workspace_bytes(GgmlQuantizedMatmulIdParams(T, K, w.inter, w.hidden, w.n_experts,
                                                                                   w.inter * rb_h, w.ggml_type)),
            quantized_matmul_id_workspace_bytes(GgmlQuantizedMatmulIdParams(T, K, w.inter, w.hidden, w.n_experts,
                                                                            w.inter * rb_h, w.ggml_type)),
            quantized_matmul_id_workspace_bytes(GgmlQuantizedMatmulIdParams(T * K, 1, w.hidden, w.inter, w.n_experts,
                                                                            w.hidden * rb_i, w.td)))
        self.id_mm = torch.empty(need, dtype=torch.uint8, device=device) if need else None
        # workspace of the shared expert's prefill-sized dense products (the SwiGLU form where it exists, and the down product)
        pg = GgmlQuantizedMatmulParams(T, w.shared_inter, w.hidden, w.ggml_type)
        pd = GgmlQuantizedMatmulParams(T, w.hidden, w.shared_inter, w.td)
        need = max(quantized_matmul_swiglu_workspace_bytes(pg, torch.bfloat16), quantized_matmul_workspace_bytes(pg, torch.bfloat16),
                   quantized_matmul_workspace_bytes(pd, torch.float32))
        self.dense_ws = torch.empty(need, dtype=torch.uint8, device=device) if need else None
        self.max_tokens = T
        # scratch of the one-launch decode block (hq_moe_ffn_decode): zeroed once, then the library's
        _layer = w.c_layer()
        fb = _l.load().hq_moe_ffn_decode_layer_scratch_bytes(ctypes.byref(_layer), min(T, 8), _l.HQ_BF16)
        self.fused = torch.zeros(fb, dtype=torch.uint8, device=device) if fb else None


# Dense products above this many rows take the tile (GEMM) route, which the batched launch does not cover.
_BATCH_MAX_DENSE_ROWS = 8
_ROUTE_IN_LAUNCH_MAX_EXPERTS = 256
_ROUTE_IN_LAUNCH_MAX_TOKENS = 4
_FUSED_SWIGLU_MAX_K = 8192


def moe_ffn_decode_fused(x: torch.Tensor, w: MoeFfnWeightsGpuQ, s: MoeFfnScratch, out: torch.Tensor,
                         residual: torch.Tensor | None = None) -> None:
    """The whole block as one launch (hq_moe_ffn_decode); raises HqError(HQ_ERR_UNSUPPORTED) for shapes it does not take."""
    import ctypes as _ct
    T = x.shape[0]
    layer = w.c_layer()
    if s.fused is None:
        raise _l.HqError(_l.HQ_ERR_UNSUPPORTED, "no scratch for the one-launch MoE block (shape not supported)")
    L = _l.load()
    # more than eight tokens (up to _FUSED_CHUNKED_MAX_TOKENS): one launch per eight, one after the other over the same scratch
    for t0 in range(0, T, 8):
        t1 = min(T, t0 + 8)
        _l.check(L.hq_moe_ffn_decode(
            _stream(), _ct.byref(layer), _dev(x[t0:t1], "x"), _act_dtype(x),
            _dev(residual[t0:t1], "residual") if residual is not None else None, _dev(out[t0:t1], "out"), t1 - t0,
            _dev(s.fused, "scratch"), s.fused.numel(), _dev(s.ids[t0 * w.top_k:], "ids"), _dev(s.topk_w[t0 * w.top_k:], "topk_w")))


# Up to this many tokens the block runs as launches of the one-launch form over eight tokens each (33 us per eight:
# 47 / 67 / 133 us at 9 / 16 / 32 tokens) rather than as separate dispatches with one GEMV per routed row (114 us at
# 9 .. 16 tokens, 178 at 32, 257 at 64, where eight launches would cost the same).
_FUSED_CHUNKED_MAX_TOKENS = 48


def moe_ffn_decode_fused_bytes(x: torch.Tensor, w: MoeFfnWeightsGpuQ) -> int:
    """Scratch bytes of the one-launch form for these tokens; 0: the shape is not one it takes."""
    T = x.shape[0]
    if T > _FUSED_CHUNKED_MAX_TOKENS:
        return 0
    layer = w.c_layer()
    return int(_l.load().hq_moe_ffn_decode_layer_scratch_bytes(ctypes.byref(layer), min(T, 8), _act_dtype(x)))


def moe_ffn_decode_fused_supported(x: torch.Tensor, w: MoeFfnWeightsGpuQ) -> bool:
    return moe_ffn_decode_fused_bytes(x, w) > 0


def build_moe_ffn_layer_gpu_q_into(x: torch.Tensor, w: MoeFfnWeightsGpuQ, s: MoeFfnScratch, out: torch.Tensor,
                                   residual: torch.Tensor | None = None, batched: bool | None = None,
                                   route_in_launch: bool | None = None, fused: bool | None = None) -> None:
    """gpu_ffn.rs:2313-2802, phases A-F, enqueued on the current stream with no host round trip:
    router / shared projections -> softmax top-k + shared SwiGLU -> gate, up mul_mat_id + shared down ->
    SwiGLU -> down mul_mat_id (n_tokens = T*K, top_k = 1) -> weighted reduce (+ sigmoid-gated shared, + residual).

    `batched` (default: whenever the token count allows) hands the dispatches that the reference encodes
    without a barrier between them to the library as one launch each and folds both SwiGLU passes into the
    staging of the down projections: five launches instead of twelve, same arithmetic, same results; with
    `route_in_launch` (default: up to four tokens; up to 256 experts) the gate / up launch also works out the
    softmax / top-k, four launches (measured per layer: 23.9 -> 21.7 us at one token, 35.3 -> 33.8 at four, 50.3 ->
    51.6 at eight, where every one of the many workgroups repeating the routing costs more than the launch saved)."""
    T = x.shape[0]
    K, H, E, I, SI, t, td = w.top_k, w.hidden, w.n_experts, w.inter, w.shared_inter, w.ggml_type, w.td
    rb = ggml_row_bytes(t, H)
    if fused is None:
        # (a scratch made for fewer tokens than this call brings is too small for the one-launch form: separate dispatches then)
        need = moe_ffn_decode_fused_bytes(x, w) if batched is None and route_in_launch is None and s.fused is not None else 0
        fused = need > 0 and s.fused.numel() >= need
    if fused:
        # one launch for the whole block, the bits of the batched dispatches below
        return moe_ffn_decode_fused(x, w, s, out, residual)
    if batched is None:
        batched = T <= _BATCH_MAX_DENSE_ROWS
    if batched:
        if T > _BATCH_MAX_DENSE_ROWS:
            raise ValueError(f"batched MoE block: {T} tokens (limit {_BATCH_MAX_DENSE_ROWS})")
        dense_gemv_bf16_f32_pair(x, w.router, s.logits, E, w.shared_gate_logit, s.sh_logit, 1, T, H)
        if route_in_launch is None:
            route_in_launch = T <= _ROUTE_IN_LAUNCH_MAX_TOKENS
        if E <= _ROUTE_IN_LAUNCH_MAX_EXPERTS and route_in_launch:
            # the gate / up launch works the routing out itself and writes it down for the launches that follow
            r_gate = dict(route_logits=s.logits, route_ids=s.ids, route_weights=s.topk_w)
            r_up = dict(route_logits=s.logits)
        else:
            dispatch_moe_softmax_topk(s.logits, s.ids, s.topk_w, T, E, K)
            r_gate = r_up = dict(ids=s.ids)
        quantized_matmul_batch_ggml([
            QmatmulJob(x, w.expert_gate, s.gate, T, I, H, top_k=K, n_experts=E, expert_stride=I * rb, **r_gate),
            QmatmulJob(x, w.expert_up, s.up, T, I, H, top_k=K, n_experts=E, expert_stride=I * rb, **r_up),
            QmatmulJob(x, w.shared_gate, s.sh_gate, T, SI, H),
            QmatmulJob(x, w.shared_up, s.sh_up, T, SI, H),
        ], t)
        quantized_matmul_batch_ggml([
            QmatmulJob(s.gate, w.expert_down, s.down, T * K, H, I, ids=s.ids, top_k=1, n_experts=E,
                       expert_stride=H * ggml_row_bytes(td, I), input_up=s.up),
            QmatmulJob(s.sh_gate, w.shared_down, s.sh_down, T, H, SI, input_up=s.sh_up),
        ], td)
        dispatch_moe_weighted_reduce(s.down, s.topk_w, out, T, K, H, shared=s.sh_down, shared_logit=s.sh_logit,
                                     residual=residual)
        return
    # A
    dense_gemv_bf16_f32(x, w.router, s.logits, T, E, H)
    dense_gemv_bf16_f32(x, w.shared_gate_logit, s.sh_logit, T, 1, H)
    psh = GgmlQuantizedMatmulParams(T, SI, H, t)
    dws = s.dense_ws if T <= s.max_tokens else None  # sized for max_tokens: enough for any fewer
    shared_one_call = dws is not None and quantized_matmul_swiglu_workspace_bytes(psh, x.dtype) > 0
    rsc = w.row_scales or {}  # kept from load time (prepare_prefill), or worked out by every call's pre-pass
    if shared_one_call:
        # a prefill chunk, Q4_K / Q5_K: the shared expert's gate, up and SwiGLU as one call (the same bits)
        quantized_matmul_swiglu_ggml(x, w.shared_gate, w.shared_up, s.sh_act, psh, dws, rsc.get("shared_gate"), rsc.get("shared_up"))
    else:
        quantized_matmul_ggml(x, w.shared_gate, s.sh_gate, psh)
        quantized_matmul_ggml(x, w.shared_up, s.sh_up, psh)
    # B
    dispatch_moe_softmax_topk(s.logits, s.ids, s.topk_w, T, E, K)
    if not shared_one_call:
        dispatch_silu_mul(s.sh_gate[:T], s.sh_up[:T], s.sh_act[:T])
    # C, D
    pid = GgmlQuantizedMatmulIdParams(T, K, I, H, E, I * rb, t)
    ws = s.id_mm  # sized for max_tokens; fewer tokens need less (or none: decode-sized calls take the GEMV form)
    if ws is not None and quantized_matmul_id_swiglu_workspace_bytes(pid):
        # a prefill chunk of Q4_K / Q5_K experts: gate, up and their SwiGLU as one grouped product (the same bits)
        quantized_matmul_id_swiglu_ggml(x, w.expert_gate, w.expert_up, s.ids, s.act, pid, ws, rsc.get("expert_gate"),
                                        rsc.get("expert_up"))
    else:
        quantized_matmul_id_ggml(x, w.expert_gate, s.ids, s.gate, pid, scratch=ws, w_row_scales=rsc.get("expert_gate"))
        quantized_matmul_id_ggml(x, w.expert_up, s.ids, s.up, pid, scratch=ws, w_row_scales=rsc.get("expert_up"))
        dispatch_silu_mul(s.gate[:T * K], s.up[:T * K], s.act[:T * K])
    pdn = GgmlQuantizedMatmulParams(T, H, SI, td)
    if dws is not None and quantized_matmul_workspace_bytes(pdn, torch.float32):
        quantized_matmul_ggml(s.sh_act, w.shared_down, s.sh_down, pdn, workspace=dws, w_row_scales=rsc.get("shared_down"))
    else:
        quantized_matmul_ggml(s.sh_act, w.shared_down, s.sh_down, pdn)
    # E
    quantized_matmul_id_ggml(s.act, w.expert_down, s.ids, s.down,
                             GgmlQuantizedMatmulIdParams(T * K, 1, H, I, E, H * ggml_row_bytes(td, I), td), scratch=ws,
                             w_row_scales=rsc.get("expert_down"))
    # F
    dispatch_moe_weighted_reduce(s.down, s.topk_w, out, T, K, H, shared=s.sh_down, shared_logit=s.sh_logit,
                                 residual=residual)


def moe_ffn_prefill_scratch_bytes(w: MoeFfnWeightsGpuQ, n_tokens: int, act_dtype: torch.dtype) -> int:
    import ctypes as _ct
    layer = w.c_layer()
    xdt = HQ_BF16 if act_dtype == torch.bfloat16 else HQ_F32
    return int(_l.load().hq_moe_ffn_prefill_scratch_bytes(_ct.byref(layer), n_tokens, xdt))


def moe_ffn_prefill(x: torch.Tensor, w: MoeFfnWeightsGpuQ, out: torch.Tensor, scratch: torch.Tensor,
                    residual: torch.Tensor | None = None, route_ids: torch.Tensor | None = None,
                    route_weights: torch.Tensor | None = None) -> None:
    """build_moe_ffn_layer_gpu_q_into (gpu_ffn.rs:2313-2802) as ONE library call at any token count, every buffer carved
    from `scratch` (moe_ffn_prefill_scratch_bytes); the bits of the separate dispatches above.  Row scales kept by
    prepare_prefill() are passed on."""
    import ctypes as _ct
    layer = w.c_layer()
    rs = None
    if w.row_scales:
        g = lambda k: _dev(w.row_scales[k], k) if w.row_scales.get(k) is not None else None  # noqa: E731
        rs = _l.MoeFfnRowScales(g("expert_gate"), g("expert_up"), g("expert_down"), g("shared_gate"), g("shared_up"), g("shared_down"))
    _l.check(_l.load().hq_moe_ffn_prefill(
        _stream(), _ct.byref(layer), _ct.byref(rs) if rs is not None else None, _dev(x, "x"), _act_dtype(x),
        _dev(residual, "residual") if residual is not None else None, _dev(out, "out"), x.shape[0], _dev(scratch, "scratch"),
        scratch.numel() * scratch.element_size(), _dev(route_ids, "route_ids") if route_ids is not None else None,
        _dev(route_weights, "route_weights") if route_weights is not None else None))


def dense_ffn_scratch_bytes(w: DenseFfnWeightsGpuQ, m: int, act_dtype: torch.dtype) -> int:
    xdt = HQ_BF16 if act_dtype == torch.bfloat16 else HQ_F32
    td = w.down_type if w.down_type is not None else w.ggml_type
    return int(_l.load().hq_dense_ffn_scratch_bytes(m, w.hidden, w.inter, w.ggml_type, td, xdt))


def dense_ffn(x: torch.Tensor, w: DenseFfnWeightsGpuQ, out: torch.Tensor, scratch: torch.Tensor, row_scales: dict | None = None) -> None:
    """build_dense_ffn_layer_gpu_q (gpu_ffn.rs:1017-1351) as ONE library call at any row count, buffers carved from
    `scratch` (dense_ffn_scratch_bytes); the bits of build_dense_ffn_layer_gpu_q_into."""
    td = w.down_type if w.down_type is not None else w.ggml_type
    rs = row_scales or {}
    g = lambda k: _dev(rs[k], k) if rs.get(k) is not None else None  # noqa: E731
    _l.check(_l.load().hq_dense_ffn(_stream(), _dev(x, "x"), _act_dtype(x), _dev(w.gate_q, "gate"), _dev(w.up_q, "up"), _dev(w.down_q, "down"),
                                    w.ggml_type, td, g("gate"), g("up"), g("down"), _dev(out, "out"), x.shape[0], w.hidden, w.inter,
                                    _dev(scratch, "scratch"), scratch.numel() * scratch.element_size()))

/*
 * hf2q_hip.h -- C ABI of libhf2q_hip.so: the MI355X (gfx950) implementation of
 * hf2q's quantized-matmul hot path.
 *
 * Conventions (they mirror the contract hf2q's call sites have with their GPU
 * backend today):
 *   - every buffer pointer is a DEVICE pointer owned by the caller; nothing is
 *     retained by the library (hf2q passes caller-owned MlxBuffers and scratch
 *     the same way, gpu_ffn.rs:194-204, 644-648).  Two entry points allocate
 *     stream-ordered scratch of their own for prefill-sized inputs and say so
 *     (hq_qmatmul_ggml, hq_qmatmul_id_ggml without scratch never does); their
 *     _ws forms take the scratch from the caller and allocate nothing;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     Work is enqueued in order on it and the call returns at once, like an
 *     encoder dispatch without commit; the caller synchronises.  An in-order
 *     stream provides every read-after-write barrier hf2q declares by hand
 *     (gpu_ffn.rs:2538-2544);
 *   - shapes are explicit arguments, never inferred from buffer sizes;
 *   - every function returns HQ_OK (0) or an hq_status error code and never
 *     aborts; the message is available from hq_last_error() on the same thread
 *     ("fail loud", kv_cache.rs:152-153);
 *   - functions are re-entrant per stream; the library's state is the
 *     thread-local error string, a per-device note of which kernels had their
 *     LDS limit raised, and the static device scratch of
 *     hq_flash_attn_vec_tq_static (shared by every call on a GPU);
 *   - data-dependent conditions are not errors: an expert id >= n_experts
 *     gives NaN output rows for that (token, slot), never an out-of-bounds read
 *     and never a status code (the ids live on the device and are not read by
 *     the host); hq_tq_attn_params.nsg is accepted and ignored.
 *
 * Paths cited below are relative to the hf2q source tree.
 */
#ifndef HF2Q_HIP_H
#define HF2Q_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Exported from the shared library (it is built with hidden visibility). */
#define HQ_API __attribute__((visibility("default")))

typedef enum {
    HQ_OK = 0,
    HQ_ERR_INVALID_ARGUMENT = 1, /* shape / alignment / enum the path rejects */
    HQ_ERR_UNSUPPORTED = 2,      /* ggml type or mode not on this path */
    HQ_ERR_HIP = 3               /* a HIP runtime call failed */
} hq_status;

/* Numeric ids are GGML's (src/quantize/ggml_quants/ggml_type.rs:18-53).  Every entry point that takes
 * a type serves all five (block layouts: q4_0.rs:6-12, q8_0.rs, q4_k.rs, q5_k.rs:9-18, q6_k.rs).  Q4_K and
 * Q5_K blocks must be 16-byte aligned, the others 2-byte. */
typedef enum { HQ_Q4_0 = 2, HQ_Q8_0 = 8, HQ_Q4_K = 12, HQ_Q5_K = 13, HQ_Q6_K = 14 } hq_ggml_type;

/* Activation element type.  hf2q's call sites pass F32 (gpu_full_attn.rs:835);
 * BF16 is the serving configuration this library is benchmarked on. */
typedef enum { HQ_F32 = 0, HQ_BF16 = 1, HQ_F16 = 2 /* output of hq_dequant_ggml only */ } hq_act_dtype;

/* Thread-local message of the last failing call on this thread ("" if none). */
HQ_API const char* hq_last_error(void);

/* Library ABI version (major*100 + minor). */
HQ_API int hq_version(void);

/* Block geometry: GgmlType::block_size / type_size (ggml_type.rs:60-135).
 * Return 0 for a type this path does not handle. */
HQ_API uint32_t hq_block_elems(hq_ggml_type t);
HQ_API uint32_t hq_block_bytes(hq_ggml_type t);

/* Dequantise `n_elems` (a whole number of blocks) of packed GGML blocks to
 * f32 (out_dtype HQ_F32, bit-exact: one correctly rounded value per element)
 * or bf16 / f16 (HQ_BF16 / HQ_F16, the f32 value rounded to nearest-even; f16 is
 * the reference's shadow dtype).  Replaces the
 * load-time `materialize_f16_shadow` pre-dequantisation
 * (src/serve/forward_mlx.rs:9426-9440) and doubles as the bit-exactness probe
 * for the in-kernel dequantisers. */
HQ_API int hq_dequant_ggml(void* stream, const void* w_blocks, void* out, hq_act_dtype out_dtype,
                    uint64_t n_elems, hq_ggml_type t);

/* Quantise f32 rows to packed GGML blocks on the device, byte-identical to
 * hf2q's CPU quantizers without an importance matrix
 * (src/quantize/ggml_quants/quantizer.rs:51-102 -> q4_k.rs:50-217,
 * q6_k.rs:40-221, q8_0.rs:31-72, q5_k.rs, q4_0.rs; load-time use:
 * src/inference/models/qwen35/in_memory_loader.rs:70-139).
 * `n_elems` must be a multiple of `n_per_row`, `n_per_row` of the block size. */
HQ_API int hq_quantize_ggml(void* stream, const float* src, uint64_t n_elems, uint64_t n_per_row,
                     hq_ggml_type t, void* out_blocks);

/* The same with an importance matrix: GgmlQuantizer::quantize(src, n_per_row, Some(imatrix))
 * (quantizer.rs:51-102 -> q4_k.rs:220-324, q5_k.rs:246-311, q6_k.rs:40-151 with weights, q4_0.rs:52-87; Q8_0 takes the
 * argument and does not use it, q8_0.rs:31-72), byte-identical to the CPU quantizers.  `imatrix`: n_per_row f32 weights
 * in device memory, one per column, shared by every row.  `scratch`: hq_quantize_ggml_imatrix_scratch_bytes() bytes of
 * device memory (Q4_0: one float per row for the row's mean square; 0 for the other types, `scratch` may then be null). */
HQ_API size_t hq_quantize_ggml_imatrix_scratch_bytes(uint64_t n_elems, uint64_t n_per_row, hq_ggml_type t);
HQ_API int hq_quantize_ggml_imatrix(void* stream, const float* src, uint64_t n_elems, uint64_t n_per_row, hq_ggml_type t,
                             const float* imatrix, void* out_blocks, void* scratch, size_t scratch_bytes);

/* dst[m,n] = x[m,k] . W[n,k]^T with W stored as GGML blocks, row-major
 * [n][k/QK]; fp32 accumulate, f32 output.  Replaces
 * mlx_native quantized_matmul_ggml(encoder, registry, device, input, weight,
 * &mut dst, &GgmlQuantizedMatmulParams{m,n,k,ggml_type})
 * (src/inference/models/qwen35/gpu_ffn.rs:1236-1245; dispatch_qmatmul,
 * src/serve/forward_mlx.rs:9655-9969).  m <= 8 takes the bandwidth-bound GEMV
 * kernels (MM_ROUTING_THRESHOLD, forward_mlx.rs:9791; from two to four rows on, by type, a form that fetches every
 * weight once for all rows), and Q4_K / Q5_K run up to 16 rows as two such passes; larger m takes the MFMA GEMM,
 * whose tiles are 64 (Q4_K / Q5_K), 128 or 256 token rows by m; up to 256 rows k is cut into slices where the
 * weight-row tiles alone would leave CUs idle.
 * A K-quant's k that is not a multiple of 1024 (2816, 3584, 5120 ...) has the small-batch kernel where all of k fits a
 * CU's LDS and the matrix has 8192 rows or more (512 or more from four activation rows on); otherwise up to 16 rows run
 * as per-row GEMVs first.
 * MFMA GEMM.  The K-quant (k % 256 == 0) and Q8_0 / Q4_0 (k % 128 == 0) GEMMs multiply f16-rounded
 * weights and activations like the reference's mul_mm, the other kernels keep
 * every product exact.
 * Requires k % block_elems == 0; Q4_K / Q5_K need a 16-byte aligned `w_blocks`,
 * the other types a 2-byte aligned one. */
HQ_API int hq_qmatmul_ggml(void* stream, const void* x, hq_act_dtype xdt, const void* w_blocks, float* y,
                    uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t);

/* How hq_qmatmul_ggml[_ws] cuts k for up to 256 activation rows on the tile route: `slices` slices of
 * `blocks_per_slice` 256-element runs each (the last one shorter), every slice a launch-time workgroup set of its own whose
 * partial products a second launch adds in slice order.  slices = 1: no cut.  (slices - 1) * blocks_per_slice < k / 256
 * always holds, so no slice starts past the end of a row.  Pure host arithmetic; a query for tests and for sizing. */
HQ_API int hq_qmatmul_ggml_k_slices(uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t, uint32_t* slices,
                             uint32_t* blocks_per_slice);

/* How the single-row product of any k lays its work out (the walk that serves f32 activations, k that is not a multiple
 * of 4096, Q8_0 / Q4_0): a row is `units_per_row` units (a 256-weight super-block, or a 32-weight block); a task is
 * `rows_per_task` (a power of two) whole rows = `windows_per_task` windows of `units_per_window` units, at most
 * `window_capacity` (16 super-blocks or 64 blocks: one wave's 64 lanes); the last window of a task may be ragged
 * (windows_per_task * units_per_window >= rows_per_task * units_per_row > (windows_per_task - 1) * units_per_window always
 * holds: no window is empty).  `waves`: the waves the launch has (CUs x 16).  Pure host arithmetic; a query for tests. */
HQ_API int hq_gemv_flat_plan(uint32_t n, uint32_t k, hq_ggml_type t, uint32_t waves, uint32_t* units_per_row, uint32_t* rows_per_task,
                      uint32_t* windows_per_task, uint32_t* units_per_window, uint32_t* window_capacity);

/* The same product with caller-owned device scratch.  The f16 tile kernels
 * (prefill-sized m; K-quants with k % 256 == 0, Q8_0 / Q4_0 with k % 128 == 0) convert the
 * activations to row-scaled f16 in a pre-pass and need hq_qmatmul_ggml_workspace_bytes() bytes (256-byte
 * aligned) for them -- plus, for up to 256 rows over few weight rows, the partial sums of
 * the slices k is cut into (slices x m x n floats, up to eight slices), which a second launch adds in a fixed order; every other shape needs none (the function returns 0 and
 * `workspace` may be null).  hq_qmatmul_ggml itself takes that scratch from the
 * stream-ordered allocator (hipMallocAsync / hipFreeAsync on `stream`).  The
 * reference has no such buffer: its mul_mm kernel (quantized_matmul_ggml's
 * m > 8 route, src/serve/forward_mlx.rs:9791-9830) casts the activations to
 * half while it stages them. */
HQ_API size_t hq_qmatmul_ggml_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt,
                                       hq_ggml_type t);
HQ_API int hq_qmatmul_ggml_ws(void* stream, const void* x, hq_act_dtype xdt, const void* w_blocks, float* y,
                       uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t, void* workspace,
                       size_t workspace_bytes);

/* The up projection of a dense SwiGLU layer finishing the gating in its epilogue, on the prefill route:
 *   y[m, n] = silu(gate[m, n]) * (x . W^T)[m, n]
 * with `gate` the f32 output of the gate projection computed before it.  Replaces the second quantized_matmul_ggml
 * and the silu_mul of the dense FFN at prefill (gpu_ffn.rs:1236-1306): the stand-alone SwiGLU pass reads both
 * products and writes the activations (300 MB at 2048 x 12288, about 50 us); here the gate values are read while the
 * tiles are stored and the up product never goes to memory.  The bits of the separate calls.  Every weight type of
 * the tile route, any token count above the small-batch kernels' -- except where the product is cut into slices of k
 * (up to 256 rows over few weight rows): hq_qmatmul_gated_ggml_workspace_bytes() is 0 there and the call returns
 * HQ_ERR_UNSUPPORTED.  y may be the gate buffer itself (every element is read before it is written, by the same lane).
 * w_row_scales: null, or from hq_weight_row_scales_ggml. */
HQ_API size_t hq_qmatmul_gated_ggml_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt, hq_ggml_type t);
HQ_API int hq_qmatmul_gated_ggml_ws(void* stream, const void* x, hq_act_dtype xdt, const void* w_blocks,
                             const float* w_row_scales, const float* gate, float* y, uint32_t m, uint32_t n, uint32_t k,
                             hq_ggml_type t, void* workspace, size_t workspace_bytes);

/* The gate and up products of a dense SwiGLU layer and the gating as one call on the prefill route:
 *   y[m, n] = silu(x . W_gate^T) * (x . W_up^T)
 * Replaces the two quantized_matmul_ggml dispatches and the silu_mul between them that the dense FFN and the shared
 * expert of the MoE block encode at prefill (gpu_ffn.rs:1236-1306, 2485-2545): one activation pre-pass, one launch of
 * tiles of 64 or 128 token rows that multiply the same activation rows with the same weight rows of both matrices;
 * the two f32 products never go to memory.  The bits of the three separate calls wherever hq_qmatmul_ggml_ws sums
 * all of k inside one tile (hq_qmatmul_gated_ggml_workspace_bytes() is not 0 for the shape); where that call cuts k
 * into slices (up to 256 rows over few weight rows) this form still sums k in one tile, so the f32 sums associate
 * differently and the results agree to a few units in the last place.  Exists where
 * hq_qmatmul_swiglu_ggml_workspace_bytes() is not 0 (Q4_K /
 * Q5_K on the tile route: more rows than the small-batch kernels take, k % 256 == 0); other calls return
 * HQ_ERR_UNSUPPORTED and the caller issues the separate calls.  The separate calls run 256-row tiles from 257 rows
 * on, which use the matrix cores better: this form pays for few weight rows (the shared expert: 512) or few tokens,
 * not for a 12288-row layer over thousands of tokens.  gate_row_scales / up_row_scales: both null, or both from
 * hq_weight_row_scales_ggml (n floats each). */
HQ_API size_t hq_qmatmul_swiglu_ggml_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt, hq_ggml_type t);
HQ_API int hq_qmatmul_swiglu_ggml_ws(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up,
                              const float* gate_row_scales, const float* up_row_scales, float* y, uint32_t m, uint32_t n,
                              uint32_t k, hq_ggml_type t, void* workspace, size_t workspace_bytes);

/* The same on the decode route (m <= 8 activation rows): one launch per row walks the same weight rows of both matrices
 * and stores silu(gate) * up -- the two f32 products never go to memory and the hq_silu_mul dispatch between them and the
 * down projection disappears (gpu_ffn.rs:1231-1306 at batch 1).  The bits of hq_qmatmul_batch_ggml(gate, up) followed by
 * hq_silu_mul.  Any type, f32 or bf16 activations, any k of whole blocks; matrices too small for the streaming GEMV
 * (hq_qmatmul_swiglu_decode_supported() == 0) return HQ_ERR_UNSUPPORTED and take the separate calls. */
HQ_API int hq_qmatmul_swiglu_decode_supported(uint32_t n, uint32_t k, hq_ggml_type t, hq_act_dtype xdt);
HQ_API int hq_qmatmul_swiglu_decode(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up, float* y,
                             uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t);

/* y[m, n] = sum_k x[m, k] * W[n, k] with the activations stored heads-outermost, [k / head_dim][m][head_dim]
 * (the attention output of a batched prefill): element (row, kk) sits at ((kk / head_dim) * m + row) * head_dim +
 * kk % head_dim.  Replaces quantized_matmul_mm_tensor_perm021(enc, reg, dev, input, weight, dst,
 * GgmlQuantizedMatmulPerm021Params{m, n, k, head_dim, ggml_type}) (forward_prefill_batched.rs:2219-2257), which
 * saves the transpose between attention and the output projection.  The tile GEMM (m > 8) gathers in its
 * activation pre-pass at no extra cost; other shapes copy the activations into row-major order in `workspace`
 * first.  head_dim: a multiple of 8 that divides k. */
HQ_API size_t hq_qmatmul_perm021_ggml_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt, hq_ggml_type t);
HQ_API int hq_qmatmul_perm021_ggml_ws(void* stream, const void* x_perm, hq_act_dtype xdt, const void* w_blocks, float* y,
                               uint32_t m, uint32_t n, uint32_t k, uint32_t head_dim, hq_ggml_type t, void* workspace,
                               size_t workspace_bytes);

/* out[t, s, :] = W[ids[t*top_k + s]] . x[t, :] over an expert stack
 * [n_experts][n][k/QK] whose experts are `expert_stride` BYTES apart;
 * ids [n_tokens*top_k] u32 on the device (no host sync); out
 * [n_tokens*top_k, n] f32.  Replaces quantized_matmul_id_ggml[_pooled]
 * (gpu_ffn.rs:194-204; forward_mlx.rs:5285-5292, 5367-5374) with
 * GgmlQuantizedMatmulIdParams{n_tokens, top_k, n, k, n_experts,
 * expert_stride, ggml_type}.  The "down" projection is the same call with
 * n_tokens = T*K, top_k = 1 (forward_mlx.rs:650-651).  An id >= n_experts
 * makes the affected output rows NaN instead of reading out of bounds.
 * Decode-sized calls run one dequant-fused GEMV per routed row and use no
 * scratch.  With at least 3 routed rows per expert (prefill) and a `scratch`
 * of hq_qmatmul_id_ggml_workspace_bytes() bytes (device, 256-byte aligned),
 * the rows are sorted by expert and every expert's rows go through the tile
 * GEMM of the m > 8 route (the reference's mul_mm_id, forward_mlx.rs:5237-5245);
 * that form needs a contiguous stack (expert_stride = one expert's bytes).
 * With scratch == NULL every size takes the GEMV form. */
HQ_API int hq_qmatmul_id_ggml(void* stream, const void* x, hq_act_dtype xdt, const void* w_stack,
                       const uint32_t* ids, float* y, void* scratch, size_t scratch_bytes,
                       uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k,
                       uint32_t n_experts, uint64_t expert_stride, hq_ggml_type t);

/* The weight-row scales of the f16 tile kernels, kept by the caller.  Those kernels (the prefill-sized routes of
 * hq_qmatmul_ggml[_ws] and the grouped route of hq_qmatmul_id_ggml) multiply every weight row by a power of two taken
 * from the row's block headers before the weights are rounded to f16, and divide it out in the epilogue; every call
 * works the scales out again in its pre-pass, which touches each cache line of the weights for four bytes of every
 * block header (151 MB for a stack of 256 experts of 512 x 2048 Q4_K: 12-17 us of the call at 2048 tokens x top-8).  They
 * are a function of the weights alone, so a caller whose weights do not change (inference) computes them once when the
 * weights are loaded -- hq_weight_row_scales_ggml: `scales` receives n_rows floats, row r of the matrix, or row
 * e * n + r of a contiguous stack -- and passes them to the _prepared forms, which skip that scan and are otherwise the
 * calls they are named after, with the same results to the bit.  Scales that do not belong to the weights give wrong
 * products (possibly inf / nan), never a fault.  Routes that do not use the tile kernels ignore the argument.  No
 * counterpart in the reference, whose mul_mm kernels round the dequantised weights to half without a row scale
 * (forward_mlx.rs:9791-9830). */
HQ_API int hq_weight_row_scales_ggml(void* stream, const void* w_blocks, float* scales, uint64_t n_rows, uint32_t k,
                              hq_ggml_type t);
HQ_API int hq_qmatmul_ggml_ws_prepared(void* stream, const void* x, hq_act_dtype xdt, const void* w_blocks,
                                const float* w_row_scales, float* y, uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t,
                                void* workspace, size_t workspace_bytes);
HQ_API int hq_qmatmul_id_ggml_prepared(void* stream, const void* x, hq_act_dtype xdt, const void* w_stack,
                                const float* w_row_scales, const uint32_t* ids, float* y, void* scratch,
                                size_t scratch_bytes, uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k,
                                uint32_t n_experts, uint64_t expert_stride, hq_ggml_type t);

/* Gate, up and SwiGLU of a prefill-sized MoE block as one grouped product:
 *   y[p, :] = silu(W_gate[ids[p]] . x[p / top_k]) * (W_up[ids[p]] . x[p / top_k])       p < n_tokens * top_k
 * Replaces the two quantized_matmul_id_ggml dispatches of phase B ("gate || up", gpu_ffn.rs:2546, 2623-2683) and the
 * silu_mul of phase D (gpu_ffn.rs:2685-2697) at prefill: the routed rows are sorted and the activations converted
 * once, a tile multiplies the same activation rows with the same weight rows of both stacks, and the two f32
 * products never go to memory.  The result has the bits of hq_qmatmul_id_ggml (grouped form) twice followed by
 * hq_silu_mul.  Exists where hq_qmatmul_id_swiglu_ggml_workspace_bytes() is not 0: Q4_K / Q5_K on the grouped
 * route (at least 3 routed rows per expert and 256 rows, contiguous stacks of equal geometry); other calls return
 * HQ_ERR_UNSUPPORTED and the caller issues the separate calls.  gate_row_scales / up_row_scales: both null, or both
 * from hq_weight_row_scales_ggml (n_experts * n floats each), see there. */
HQ_API size_t hq_qmatmul_id_swiglu_ggml_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k,
                                                 uint32_t n_experts, uint64_t expert_stride, hq_ggml_type t);
HQ_API int hq_qmatmul_id_swiglu_ggml(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate_stack,
                              const void* w_up_stack, const float* gate_row_scales, const float* up_row_scales,
                              const uint32_t* ids, float* y, void* scratch, size_t scratch_bytes, uint32_t n_tokens,
                              uint32_t top_k, uint32_t n, uint32_t k, uint32_t n_experts, uint64_t expert_stride,
                              hq_ggml_type t);

/* Bytes of `scratch` the GEMV form needs for up to `max_rows` = n_tokens*top_k
 * routed rows (the IdMmScratch analogue, decode_pool.rs:56-60): always 0.  Kept
 * so that a port of the reference's scratch sizing call has something to call;
 * new code asks hq_qmatmul_id_ggml_workspace_bytes(), which returns what the
 * grouped (prefill) form needs and 0 where the GEMV form runs. */
HQ_API size_t hq_qmatmul_id_scratch_bytes(uint32_t n_experts, uint32_t max_rows);
/* Bytes of `scratch` for this call's shape: 0 where the GEMV form is used, else
 * the grouped form's workspace (one f16 row per token, row and weight-row
 * scales, the row permutation and the tile table). */
HQ_API size_t hq_qmatmul_id_ggml_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k,
                                          uint32_t n_experts, uint64_t expert_stride, hq_ggml_type t);

/* Up to HQ_QMATMUL_BATCH_MAX_JOBS independent decode-sized products of one weight
 * type and activation dtype in ONE launch.  The reference encodes the dispatches
 * of a phase of the MoE block without a barrier between them, so the GPU runs
 * them side by side (gpu_ffn.rs:2546 "Phase B ... (concurrent)", phases A and C
 * likewise); an in-order HIP stream would serialise separate launches, so the
 * phase is handed over as one batch instead.  A job is hq_qmatmul_id_ggml's
 * argument list when `ids` is set (rows = n_tokens, rows*top_k <= 65535) and
 * hq_qmatmul_ggml's when it is NULL (rows = m <= 8, the decode route).  With
 * `x_up` set (f32 activations only) the job's activations are
 * silu(x[i]) * x_up[i], computed while they are staged: the SwiGLU of phase D
 * folded into the down projection (the quantized_matmul_id_swiglu_q4_0 variant
 * that gpu_ffn.rs:2685-2697 describes), bit-identical to hq_silu_mul followed by
 * the plain product.
 * With `route_logits` set (and `ids` NULL) the job is routed by the launch itself: every workgroup works out
 * hq_moe_softmax_topk of its token's logits (the same arithmetic, the same bits) and takes the expert of its
 * slot, so the dispatch_moe_softmax_topk of phase B (gpu_ffn.rs:2551-2573) needs no launch of its own;
 * `route_ids` / `route_weights`, if not NULL, also receive the selection ([rows*top_k] each) for the
 * launches that follow.  n_experts <= 256, top_k <= 64. */
#define HQ_QMATMUL_BATCH_MAX_JOBS 4
typedef struct hq_qmatmul_job {
    const void* x;        /* [rows, k] activations */
    const void* x_up;     /* NULL, or f32 [rows, k] */
    const void* w;        /* [n][k/QK] blocks, or the expert stack when ids != NULL */
    const uint32_t* ids;  /* NULL (dense) or [rows*top_k] expert ids on the device */
    float* y;             /* [rows, n] (dense) or [rows*top_k, n] */
    uint32_t rows, top_k, n, k, n_experts;
    uint64_t expert_stride; /* bytes between experts of the stack */
    const float* route_logits; /* NULL, or [rows, n_experts] router logits (ids must be NULL) */
    uint32_t* route_ids;       /* NULL, or out [rows*top_k] */
    float* route_weights;      /* NULL, or out [rows*top_k] */
} hq_qmatmul_job;
HQ_API int hq_qmatmul_batch_ggml(void* stream, const hq_qmatmul_job* jobs, uint32_t n_jobs, hq_act_dtype xdt,
                          hq_ggml_type t);

/* ---- MoE block glue (run between the mul_mat_id calls; ffn.rs:179-336 is the specification) ---- */

/* y[m,n] = x[m,k] . W[n,k]^T with W in bf16 (router / shared-expert gate projections).  Replaces
 * dense_gemv_bf16_f32 (src/inference/models/qwen35/gpu_ffn.rs:597-617).  k % 8 == 0. */
HQ_API int hq_dense_gemv_bf16(void* stream, const void* x, hq_act_dtype xdt, const void* w_bf16, float* y,
                       uint32_t m, uint32_t n, uint32_t k);

/* Two such products over the same activations in one launch: the router logits and the
 * shared-expert gate logit of phase A (gpu_ffn.rs:2485, "all read from x, concurrent"), which the reference encodes
 * back to back without a barrier.  y_a [m, n_a], y_b [m, n_b]. */
HQ_API int hq_dense_gemv_bf16_pair(void* stream, const void* x, hq_act_dtype xdt, const void* w_a, float* y_a,
                            uint32_t n_a, const void* w_b, float* y_b, uint32_t n_b, uint32_t m, uint32_t k);

/* Per token: softmax over n_experts logits, the top_k most probable experts (ties: lower id), weights
 * renormalised over the selection.  Replaces dispatch_moe_softmax_topk (gpu_ffn.rs:2551-2573); same
 * results as softmax_topk_renorm_cpu (gpu_ffn.rs:1879-1924).  n_experts <= 1024, top_k <= 64. */
HQ_API int hq_moe_softmax_topk(void* stream, const float* logits, uint32_t* ids, float* weights, uint32_t n_tokens,
                        uint32_t n_experts, uint32_t top_k);

/* out[i] = silu(gate[i]) * up[i]; n % 4 == 0.  Replaces dispatch_silu_mul (gpu_ffn.rs:2701). */
HQ_API int hq_silu_mul(void* stream, const float* gate, const float* up, float* out, uint64_t n);

/* out[t,:] = sum_s w[t,s] * y[t,s,:] + sigmoid(shared_logit[t]) * shared[t,:] + residual[t,:]; shared,
 * shared_logit and residual may each be NULL (term omitted; shared without a logit enters with weight 1).
 * Replaces dispatch_moe_weighted_reduce (gpu_ffn.rs:2777-2792).  hidden % 4 == 0. */
HQ_API int hq_moe_weighted_reduce(void* stream, const float* y, const float* w, const float* shared,
                           const float* shared_logit, const float* residual, float* out, uint32_t n_tokens,
                           uint32_t top_k, uint32_t hidden);

/* ---- TurboQuant-style 8-bit KV cache -------------------------------------------------------
 * Cache layout (src/inference/models/qwen35/kv_cache.rs:1982-2113): codes
 * [n_kv_heads, capacity, head_dim] u8 (1 byte per element) and norms
 * [n_kv_heads, capacity, max(1, head_dim/256)] f32.  K and V are stored in the rotated
 * domain  H.(s (.) x)  (normalised Hadamard, sign table kv_cache.rs:3871-3876). */

/* The whole MoE FFN block of a decode step as ONE launch: router + shared-gate logits, softmax / top-k / renormalise,
 * gate and up of the routed and the shared expert with their SwiGLU, the down projections, and
 * out[t] = sum_s w[t,s] * down[t,s] + sigmoid(shared logit[t]) * shared_down[t] (+ residual[t]).  Replaces
 * build_moe_ffn_layer_gpu_q_into (src/inference/models/qwen35/gpu_ffn.rs:2313-2802: phases A-F of one command
 * buffer); moe_ffn_cpu_ref (ffn.rs:179-336) is the specification.  The result has the bits of the separate dispatches
 * (hq_dense_gemv_bf16_pair, hq_qmatmul_batch_ggml twice with the routing and the SwiGLU folded in,
 * hq_moe_weighted_reduce).  Takes 1..8 tokens of bf16 activations, K-quant experts (Q4_K, Q5_K or Q6_K for all three
 * matrices, or Q4_K / Q5_K gate / up with a Q6_K down: layer->down_type), hidden 2048, expert and shared FFN
 * width 512, n_tokens <= n_experts <= 256, top_k <= 64; anything else is HQ_ERR_UNSUPPORTED (hq_moe_ffn_decode_scratch_bytes
 * returns 0 for it) and runs as the separate dispatches.
 * `scratch`: hq_moe_ffn_decode_scratch_bytes() bytes of device memory, 256-byte aligned, ZEROED ONCE before its first
 * use and then left to the library (it carries a call counter; calls that share a scratch must not overlap, and a
 * scratch serves one (n_experts, top_k) shape).  The workgroups of the launch hand results to each other through it
 * and wait for each other with bounded polling; if a wait ever runs out (it cannot, unless the device is shared with a
 * kernel that starves the launch for seconds) the second 32-bit word of the scratch becomes non-zero and the output is
 * undefined.  route_ids / route_weights: NULL, or where the routing is also written ([n_tokens * top_k] each). */
typedef struct hq_moe_ffn_layer {
    const void* router;            /* [n_experts, hidden] bf16 */
    const void* shared_gate_logit; /* [hidden] bf16, or NULL: the shared expert enters with weight 1 */
    const void* expert_gate;       /* [n_experts][inter][hidden / 256] blocks */
    const void* expert_up;
    const void* expert_down;       /* [n_experts][hidden][inter / 256] blocks */
    const void* shared_gate;       /* [shared_inter][hidden / 256] blocks */
    const void* shared_up;
    const void* shared_down;       /* [hidden][shared_inter / 256] blocks */
    uint32_t hidden, n_experts, top_k, inter, shared_inter;
    hq_ggml_type ggml_type;
    uint64_t expert_stride_gate_up; /* bytes between experts of expert_gate / expert_up */
    uint64_t expert_stride_down;
    uint32_t down_type;             /* hq_ggml_type of expert_down / shared_down where it differs from ggml_type
                                     * (Qwen3.6-35B-A3B stores gate / up in Q5_K and down in Q6_K); 0: ggml_type */
} hq_moe_ffn_layer;
HQ_API size_t hq_moe_ffn_decode_scratch_bytes(uint32_t n_tokens, uint32_t hidden, uint32_t n_experts, uint32_t top_k,
                                       uint32_t inter, uint32_t shared_inter, hq_ggml_type t, hq_act_dtype xdt);
/* The same query from the layer description (its down_type included). */
HQ_API size_t hq_moe_ffn_decode_layer_scratch_bytes(const hq_moe_ffn_layer* layer, uint32_t n_tokens, hq_act_dtype xdt);
HQ_API int hq_moe_ffn_decode(void* stream, const hq_moe_ffn_layer* layer, const void* x, hq_act_dtype xdt,
                      const float* residual, float* out, uint32_t n_tokens, void* scratch, size_t scratch_bytes,
                      uint32_t* route_ids, float* route_weights);

/* The hand-over state of a scratch of hq_moe_ffn_decode or hq_dense_ffn_decode: *error receives the scratch's error
 * word (0: every wait inside the launches so far ended by itself; non-zero: one ran into the polling limit, the output
 * of that call is undefined and the scratch must be zeroed again before its next use).  Waits for `stream` (a 4-byte
 * copy to the host): call it where the serving loop
 * synchronises anyway.  hq_set_handover_spin_limit sets the polling limit of launches made after it (0: the default,
 * about a million polls, seconds): a tiny limit makes every wait give up at once, which is how the tests exercise the
 * bail-out path without hanging anything. */
HQ_API int hq_handover_status(void* stream, const void* scratch, uint32_t* error);
HQ_API void hq_set_handover_spin_limit(uint32_t limit);

/* The dense SwiGLU FFN of ONE decode token as ONE launch:
 *   out[hidden] = W_down . (silu(W_gate . x) * (W_up . x)) (+ residual)
 * Replaces build_dense_ffn_layer_gpu_q (src/inference/models/qwen35/gpu_ffn.rs:1017-1351: gate and up encoded without a
 * barrier between them, :1231-1255, then silu_mul, then down) at batch 1.  One grid of a workgroup per CU streams the
 * three matrices (85 MB at hidden 4096 / inter 12288 in Q4_K): gate and up rows with their SwiGLU, the activations handed
 * to every workgroup through `scratch` as tagged words while the first down-weight fetches are already in flight, then
 * the down rows.  The result has the bits of hq_qmatmul_batch_ggml(gate, up), hq_silu_mul and hq_qmatmul_ggml(down) over
 * the f32 activations.  x: [hidden] f32 or bf16.  Types: gate / up and down of one type (any of the five), or Q4_K / Q5_K
 * gate / up with a Q6_K down; hidden and inter whole blocks (at least two per row) and small enough for the CU's LDS
 * (2 .. 4 bytes per value of hidden plus 4.25 per value of inter within 160 KiB); anything else: HQ_ERR_UNSUPPORTED,
 * hq_dense_ffn_decode_scratch_bytes() returns 0, and the separate calls do the work.
 * `scratch`: hq_dense_ffn_decode_scratch_bytes() bytes of device memory, 256-byte aligned, ZEROED ONCE before its first
 * use and then left to the library (call counter, error word, hand-over words); calls that share a scratch must not
 * overlap.  The waits inside the launch are bounded (hq_handover_status). */
HQ_API size_t hq_dense_ffn_decode_scratch_bytes(uint32_t hidden, uint32_t inter, hq_ggml_type t_gate_up, hq_ggml_type t_down,
                                         hq_act_dtype xdt);
HQ_API int hq_dense_ffn_decode(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up,
                        const void* w_down, hq_ggml_type t_gate_up, hq_ggml_type t_down, const float* residual, float* out,
                        uint32_t hidden, uint32_t inter, void* scratch, size_t scratch_bytes);

/* The whole MoE FFN block at ANY token count, as the sequence of this library's calls that a caller encoding the phases
 * of build_moe_ffn_layer_gpu_q_into (gpu_ffn.rs:2313-2802) one by one would issue, with every intermediate buffer and
 * workspace carved out of ONE caller scratch (the decode pool and IdMmScratch of decode_pool.rs:56-60 in one piece):
 *   up to 8 tokens   the decode dispatches, a phase per launch: router + shared-gate logits, [routing inside] gate / up of
 *                    the routed and the shared expert, both down projections with their SwiGLU folded in, weighted sum;
 *   more             router and shared logits, the shared expert (gate + up + SwiGLU as one tile call where that exists),
 *                    softmax / top-k, the routed experts' gate + up + SwiGLU as one grouped product where that exists (else
 *                    two mul_mat_id calls and hq_silu_mul; the grouped tile form from 3 routed rows per expert, one GEMV
 *                    per routed row below), the down mul_mat_id over n_tokens * top_k rows, the weighted sum.
 * The result has the bits of those calls made by hand.  Per-matrix types: gate / up of layer->ggml_type, down of
 * layer->down_type.  row_scales: NULL, or the weight-row scales of the six matrices kept from load time
 * (hq_weight_row_scales_ggml; any member may be NULL), which take the header scans out of the prefill-sized calls.
 * scratch: hq_moe_ffn_prefill_scratch_bytes() bytes for this token count (more tokens need more), 256-byte aligned,
 * contents irrelevant.  route_ids / route_weights: NULL, or where the routing is also copied ([n_tokens * top_k] each).
 * (hq_moe_ffn_decode is the one-launch form of the same block for the shapes it takes.) */
typedef struct hq_moe_ffn_row_scales {
    const float *expert_gate, *expert_up, *expert_down, *shared_gate, *shared_up, *shared_down;
} hq_moe_ffn_row_scales;
HQ_API size_t hq_moe_ffn_prefill_scratch_bytes(const hq_moe_ffn_layer* layer, uint32_t n_tokens, hq_act_dtype xdt);
HQ_API int hq_moe_ffn_prefill(void* stream, const hq_moe_ffn_layer* layer, const hq_moe_ffn_row_scales* row_scales, const void* x,
                       hq_act_dtype xdt, const float* residual, float* out, uint32_t n_tokens, void* scratch,
                       size_t scratch_bytes, uint32_t* route_ids, float* route_weights);

/* The dense SwiGLU FFN at ANY row count: out[m, hidden] = W_down . (silu(W_gate . x) * (W_up . x)), the sequence of calls
 * that stands for build_dense_ffn_layer_gpu_q (gpu_ffn.rs:1017-1351) with its buffers carved out of one caller scratch:
 *   up to 8 rows   gate + up + SwiGLU as one streaming launch per row (hq_qmatmul_swiglu_decode) and the down GEMV; for
 *                  matrices too small for that, gate and up as one batched launch and the down GEMV with the SwiGLU
 *                  folded into its staging (inter <= 8192) or behind hq_silu_mul;
 *   more           gate, the up projection finishing the gating in its epilogue (hq_qmatmul_gated_ggml_ws; where the tile
 *                  route has no such form: up and hq_silu_mul), down.
 * The bits of those calls made by hand.  *_row_scales: NULL, or from hq_weight_row_scales_ggml.  scratch:
 * hq_dense_ffn_scratch_bytes() bytes for this m, 256-byte aligned, contents irrelevant. */
HQ_API size_t hq_dense_ffn_scratch_bytes(uint32_t m, uint32_t hidden, uint32_t inter, hq_ggml_type t_gate_up, hq_ggml_type t_down,
                                  hq_act_dtype xdt);
HQ_API int hq_dense_ffn(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up, const void* w_down,
                 hq_ggml_type t_gate_up, hq_ggml_type t_down, const float* gate_row_scales, const float* up_row_scales,
                 const float* down_row_scales, float* out, uint32_t m, uint32_t hidden, uint32_t inter, void* scratch,
                 size_t scratch_bytes);

/* In-place  buf <- H.(s (.) buf)  per 256-element block of buf[n_heads][head_dim] (query
 * pre-rotation) and its inverse  buf <- s (.) (H.buf)  (output post-rotation).  Replace
 * dispatch_fwht_sign_premult_f32 / dispatch_fwht_sign_undo_f32(enc, reg, dev, buf, num_heads,
 * head_dim) (src/serve/forward_mlx.rs:4662-4666, 4750; gpu_full_attn.rs:219, 253).
 * head_dim must be 256 or 512. */
HQ_API int hq_fwht_sign_premult_f32(void* stream, float* buf, uint32_t n_heads, uint32_t head_dim);
HQ_API int hq_fwht_sign_undo_f32(void* stream, float* buf, uint32_t n_heads, uint32_t head_dim);

/* Write-side encode of n_tokens K (or V) vectors, src [n_tokens, n_kv_heads, head_dim] f32, into
 * cache slots (write_pos + t) % capacity: rotate, then per 256-block norm = amax/127 and
 * code = round(x/norm) as int8 (two's complement byte).  Stands where
 * dispatch_hadamard_quantize_kv_hb[_seq] stands in the reference (kv_cache.rs:180-213, 278-294);
 * the code->value map is the linear int8 one of the benchmark configuration, not the
 * reference's Lloyd-Max table. */
HQ_API int hq_tq_encode_kv(void* stream, const float* src, uint8_t* codes, float* norms, uint32_t n_tokens,
                    uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t write_pos);

/* Bulk dequantisation of cache positions start_pos .. start_pos + n_tokens - 1 of every kv head into
 * dst [n_kv_heads, n_tokens, head_dim] f32 (head-major), for prefill resume over a TQ-only cache.
 * Replaces dispatch_tq_dequantize_hb_kv_seq(enc, reg, dev, packed, norms, dst, n_kv_heads, head_dim,
 * cache_capacity, start_pos, n_tokens, scale_factor_d512, codebook_bits) as dequant_seq_to_temp_f32
 * calls it (kv_cache.rs:431-495); unrotate != 0 also applies dispatch_fwht_sign_undo_f32 to every
 * (head, token) chunk, i.e. dequant_seq_to_temp_f32_unrotated (kv_cache.rs:497-583) in one launch
 * with the bits of the two.  Values as in hq_flash_attn_vec_tq (lut256 == NULL: norm * int8(code)).
 * Rejects start_pos + n_tokens > capacity (kv_cache.rs:427-428). */
HQ_API int hq_tq_dequantize_kv_seq(void* stream, const uint8_t* codes, const float* norms, const float* lut256, float* dst,
                            uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t start_pos,
                            uint32_t n_tokens, float scale_factor_d512, uint32_t codebook_bits, int unrotate);

/* Field for field FlashAttnVecTqHbParams / Qwen35TqSdpaParams (kv_cache.rs:589-614;
 * forward_mlx.rs:4687-4705). */
typedef struct {
    uint32_t num_heads, num_kv_heads, head_dim;
    uint32_t kv_seq_len, kv_capacity;
    float scale;
    uint32_t mask_type;      /* 0 none, 1 causal, 2 sliding window (single query at the end of the sequence) */
    uint32_t sliding_window; /* mask_type 2: only the last sliding_window positions are visible */
    float softcap;           /* 0 = off, else s <- softcap * tanh(s / softcap) */
    uint32_t ring_start;     /* logical position i lives in slot (ring_start + i) % kv_capacity */
    float scale_factor_d512;
    uint32_t codebook_bits;  /* 5, 6 or 8; 5 and 6 need the centroid table (lut256) */
    uint32_t fuse_fwht_pre;  /* 1: q arrives un-rotated and is rotated inside the kernel */
    uint32_t nsg;            /* accepted for layout compatibility; the split count is chosen here */
} hq_tq_attn_params;

/* out[h] = softmax(scale * q[h] . K[kv(h)]^T) . V[kv(h)], kv(h) = h / (num_heads/num_kv_heads), one
 * query position, K/V dequantised in-kernel, fp32 softmax; q and out are [num_heads, head_dim] f32
 * in the rotated domain.  lut256 == NULL: cached value = norm * int8(code); otherwise
 * lut256[code] * norm / 16 / scale_factor.  Replaces flash_attn_vec_tq_hb(enc, reg, dev, q, k_packed,
 * k_norms, v_packed, v_norms, out, tmp, &params) (forward_mlx.rs:4732-4742; kv_cache.rs:373-386).
 * head_dim 512: codes are [n_kv_heads, capacity, 512], norms [n_kv_heads, capacity, 2] (one per
 * 256-block, kv_cache.rs:2010-2012), table values are also divided by scale_factor_d512, and every
 * 256-block of q / out is rotated on its own.
 * `tmp` is device scratch of hq_flash_attn_vec_tq_tmp_bytes() bytes, 16-byte aligned.  Rejects kv_seq_len == 0,
 * kv_capacity < kv_seq_len (kv_cache.rs:331-333), head_dim not in {256, 512}, codebook_bits not in
 * {5, 6, 8}; codebook_bits 5 / 6 without a centroid table are reported as unsupported. */
HQ_API int hq_flash_attn_vec_tq(void* stream, const float* q, const uint8_t* k_codes, const float* k_norms,
                         const uint8_t* v_codes, const float* v_norms, const float* lut256, float* out,
                         void* tmp, size_t tmp_bytes, const hq_tq_attn_params* p);
/* The same attention with the inverse rotation applied to `out` by the merge pass: stands for the
 * pair flash_attn_vec_tq_hb + dispatch_fwht_sign_undo_f32 that the decode path encodes back to back
 * (forward_mlx.rs:4732-4760; gpu_full_attn.rs:186-294) and gives the bits that pair gives.  With
 * fuse_fwht_pre = 1 the whole rotate - attend - rotate chain is this one call (two launches). */
HQ_API int hq_flash_attn_vec_tq_undo(void* stream, const float* q, const uint8_t* k_codes, const float* k_norms,
                              const uint8_t* v_codes, const float* v_norms, const float* lut256, float* out,
                              void* tmp, size_t tmp_bytes, const hq_tq_attn_params* p);
HQ_API size_t hq_flash_attn_vec_tq_tmp_bytes(uint32_t num_heads, uint32_t head_dim, uint32_t kv_seq_len);
/* The same attention (undo_rotation != 0: hq_flash_attn_vec_tq_undo) without a scratch argument: the partial
 * results live in a buffer of HQ_TQ_STATIC_TMP_BYTES that is part of the library's device image (one copy per GPU,
 * held until the process ends).  It has no counterpart in the reference.  It is for callers that cannot allocate:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc; nothing is allocated or freed
 * here.  Shapes whose hq_flash_attn_vec_tq_tmp_bytes() exceeds the buffer are rejected with
 * HQ_ERR_INVALID_ARGUMENT (16 heads x head_dim 256 at any context fit).  Every call on a GPU uses that GPU's one
 * buffer: calls that overlap on one GPU (two streams) race, and nothing of it needs to be cleared between calls.  The
 * first call on a device looks the buffer's address up (hipGetSymbolAddress); make that call outside stream
 * capture. */
#define HQ_TQ_STATIC_TMP_BYTES (4u << 20)
HQ_API int hq_flash_attn_vec_tq_static(void* stream, const float* q, const uint8_t* k_codes, const float* k_norms,
                                const uint8_t* v_codes, const float* v_norms, const float* lut256, float* out,
                                const hq_tq_attn_params* p, int undo_rotation);

/* ---- TQ block envelope (spilled K / V blocks) ---- */

/* TqPackedV1Header / TqPackedV2Header (kv_persist/families/tq_packed.rs:129-153, 376-396): the two
 * share one 40-byte wire header; codec_version selects the magic ("TQP1" / "TQP2") and whether a
 * stream of f32 norms follows the indices. */
typedef struct {
    uint32_t codec_version;  /* 1 or 2 */
    uint32_t bits_per_coord; /* 1..8 */
    uint32_t head_dim, n_kv_heads, n_tokens;
    uint32_t flags;          /* HQ_TQP_FLAG_* */
    double scale;
} hq_tqp_header;
#define HQ_TQP_HEADER_BYTES 40
#define HQ_TQP_FLAG_HADAMARD_ROTATED 1u
#define HQ_TQP_FLAG_SPLIT_CHANNEL_25BIT 2u

/* indices_bytes_len / norms_bytes_len / total_bytes (tq_packed.rs:167-184, 399-440): ceil(heads *
 * tokens * head_dim * bits / 8); 4 * heads * tokens * max(1, head_dim / 256) at version 2, else 0. */
HQ_API size_t hq_tqp_indices_bytes(const hq_tqp_header* h);
HQ_API size_t hq_tqp_norms_bytes(const hq_tqp_header* h);
HQ_API size_t hq_tqp_total_bytes(const hq_tqp_header* h);
/* pack_tq_v1_payload / pack_tq_v2_payload (tq_packed.rs:199-226, 459-489): header + indices
 * (+ norms) into out; the stream lengths must be exactly the ones above (PayloadSizeMismatch). */
HQ_API int hq_tqp_pack(const hq_tqp_header* h, const void* indices, size_t indices_len, const void* norms_le,
                size_t norms_len, void* out, size_t out_capacity);
/* unpack_tq_v1_payload / unpack_tq_v2_payload (tq_packed.rs:243-311, 491-566): parses and checks
 * (Truncated, BadMagic, UnsupportedCodecVersion, InvalidBitsPerCoord, ReservedNonZero,
 * PayloadSizeMismatch are all HQ_ERR_INVALID_ARGUMENT, told apart by hq_last_error()); returns the
 * byte offsets of the two streams inside payload. */
HQ_API int hq_tqp_unpack(const void* payload, size_t len, hq_tqp_header* h, size_t* indices_offset,
                  size_t* norms_offset);
/* capture / restore of a token range between the device cache and a version-2 envelope in host
 * memory (the raw-bytes helpers of tq_packed.rs:568-590 with the device copy folded in): codes
 * [n_kv_heads, capacity, head_dim] and norms [n_kv_heads, capacity, head_dim / 256], positions
 * start_pos .. start_pos + n_tokens - 1.  Both wait for their copies on `stream`. */
HQ_API size_t hq_tq_kv_capture_bytes(uint32_t n_kv_heads, uint32_t head_dim, uint32_t n_tokens);
HQ_API int hq_tq_kv_capture(void* stream, const uint8_t* codes, const float* norms, uint32_t n_kv_heads, uint32_t head_dim,
                     uint32_t capacity, uint32_t start_pos, uint32_t n_tokens, void* payload, size_t payload_capacity);
HQ_API int hq_tq_kv_restore(void* stream, const void* payload, size_t len, uint8_t* codes, float* norms,
                     uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t start_pos);

/* ---- the F16 shadow of a weight ---- */

/* y[m][n] (f32) = x[m][k] . W[n][k]^T over a weight that was dequantised to f16 once at load time (hq_dequant_ggml with
 * HQ_F16): the route dispatch_qmatmul takes for m > 8 when a weight has a shadow (src/serve/forward_mlx.rs:9790-9817 ->
 * dispatch_mm_v2_f16, F16 weight x F32 input -> F32 output; the shadow itself: materialize_f16_shadow, :9426-9440).
 * Memory for speed: 2 bytes per weight instead of 0.56 - 1.06, no dequantisation inside the product.  x: [m][k] f32 or
 * bf16, cast to f16 (round to nearest even) by a kernel of this library; the product is the vendor library's dense GEMM
 * (hipBLASLt) with f32 accumulation.  k % 8 == 0; x, w_f16 and y 16-byte aligned; `workspace` 256-byte aligned:
 * hq_matmul_f16_shadow_workspace_bytes() bytes of device memory (the f16 activations + what the vendor library may use).
 * The first call for a shape asks the vendor library for its kernel (host time, not capturable in a HIP graph); later
 * calls of that shape only launch. */
HQ_API size_t hq_matmul_f16_shadow_workspace_bytes(uint32_t m, uint32_t n, uint32_t k);
HQ_API int hq_matmul_f16_shadow(void* stream, const void* x, hq_act_dtype xdt, const void* w_f16, float* y, uint32_t m, uint32_t n,
                         uint32_t k, void* workspace, size_t workspace_bytes);

/* ---- weights that are not quantized ---- */

/* y[m][n] (f32) = x[m][k] . W[n][k]^T over a weight stored as f32 or f16 (`wdt`: HQ_F32 or HQ_F16), row-major as in
 * the file: the branches of dispatch_qmatmul for such tensors (src/serve/forward_mlx.rs:9820-9917) -- f32 weights (a
 * router projection): dispatch_dense_matvec_f32 at m = 1, dense_matmul_f32_f32_tensor above; native f16 weights (tensors
 * whose rows are not whole super-blocks, an f16 lm_head): dispatch_dense_matvec_f16w_f32io at m = 1, dispatch_mm_v2_f16
 * above.  Here up to 8 rows take one streaming pass over the weights each (weights widened exactly, f32 multiply-add);
 * more rows the vendor library's GEMM with f32 accumulation (f16 weights: the activations are cast to f16 first, as in
 * hq_matmul_f16_shadow; f32 weights: f32 operands).  x: [m][k] f32 or bf16.  k % 8 == 0; x, w and y 16-byte aligned.
 * `workspace`: hq_dense_matmul_workspace_bytes() bytes of device memory, 256-byte aligned (0 bytes, and the pointer may
 * be null, where the row passes run). */
HQ_API size_t hq_dense_matmul_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt, hq_act_dtype wdt);
HQ_API int hq_dense_matmul(void* stream, const void* x, hq_act_dtype xdt, const void* w, hq_act_dtype wdt, float* y, uint32_t m,
                    uint32_t n, uint32_t k, void* workspace, size_t workspace_bytes);

/* ---- measurement aid ---- */

/* Reads `bytes` (a multiple of 16) of device memory at `buf` (16-byte aligned) once with non-temporal 16-byte loads, eight
 * workgroups of four waves per CU walking the buffer front to back in runs of 8 KiB, and nothing else: the time of this launch over a buffer the caches do not hold is
 * what streaming that many bytes costs on the device, the rate the bandwidth-bound kernels of this library can be read
 * against beside the published peak.  `sink`: 4 writable bytes (written only if the data xor to a value they do not).
 * No counterpart in the reference. */
HQ_API int hq_stream_read_probe(void* stream, const void* buf, size_t bytes, uint32_t* sink);

/* ---- GGUF reader (weights as hf2q loads them) ---- */

/* Replaces mlx_native::gguf::GgufFile as hf2q uses it at load time
 * (src/serve/gpu.rs:157-167, src/inference/models/qwen35/weight_loader.rs:52-118):
 * open, tensor_info(name) -> {ggml_type, shape, byte_len}, load_tensor(name, device) -> the
 * tensor's raw GGML blocks in a device buffer, metadata lookups.  The byte format is the one
 * hf2q's own writer emits (src/backends/gguf/types.rs:20-32, 96-188; writer.rs:171-258).
 * dims are in GGUF order (innermost first: dims[0] = k, dims[1] = n, dims[2] = experts); an expert
 * stack is one contiguous tensor and expert_stride = byte_len / dims[2]
 * (src/serve/forward_mlx.rs:2438-2460).  data_offset is absolute in the file. */
typedef struct hq_gguf hq_gguf;
typedef struct hq_gguf_tensor_info {
    uint32_t ggml_type, n_dims;
    uint64_t dims[4];
    uint64_t data_offset, byte_len;
} hq_gguf_tensor_info;
HQ_API int hq_gguf_open(const char* path, hq_gguf** out);
HQ_API void hq_gguf_close(hq_gguf* g);
HQ_API uint64_t hq_gguf_tensor_count(const hq_gguf* g);
HQ_API uint64_t hq_gguf_metadata_count(const hq_gguf* g);
HQ_API uint64_t hq_gguf_alignment(const hq_gguf* g);
HQ_API const char* hq_gguf_tensor_name(const hq_gguf* g, uint64_t index);   /* NULL past the end */
HQ_API const char* hq_gguf_metadata_key(const hq_gguf* g, uint64_t index);  /* NULL past the end */
HQ_API int hq_gguf_tensor_info_by_name(const hq_gguf* g, const char* name, hq_gguf_tensor_info* out);
/* Integer and bool values widened to u64 (negative: error); f32 / f64 widened to double; strings
 * are returned as pointer + length into the mapping (not NUL-terminated). */
HQ_API int hq_gguf_metadata_u64(const hq_gguf* g, const char* key, uint64_t* out);
HQ_API int hq_gguf_metadata_f64(const hq_gguf* g, const char* key, double* out);
HQ_API int hq_gguf_metadata_string(const hq_gguf* g, const char* key, const char** out, uint64_t* len);
/* The tensor's bytes in the host mapping (valid until hq_gguf_close), NULL if there is no such tensor. */
HQ_API const void* hq_gguf_tensor_data(const hq_gguf* g, const char* name, uint64_t* byte_len);
/* Copies the tensor's raw bytes to `dev_dst` (at least byte_len bytes) on `stream` and waits for it. */
HQ_API int hq_gguf_load_tensor(const hq_gguf* g, const char* name, void* stream, void* dev_dst, size_t dst_bytes);

#ifdef __cplusplus
}
#endif
#endif /* HF2Q_HIP_H */

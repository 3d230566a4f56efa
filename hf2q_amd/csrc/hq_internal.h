// Internal declarations shared by the translation units of libhf2q_hip.so.
// gfx950 (MI355X) only: 64-lane wavefronts are assumed throughout.
#pragma once

#include <hip/hip_runtime.h>

#include <stdint.h>

#include "../../include/hf2q_hip.h"

namespace hq {

// Records the message for hq_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// HQ_OK, or HQ_ERR_HIP with the HIP error string recorded.
int check_hip(hipError_t e, const char* what);
// Checks the launch that was just enqueued.
inline int check_launch(const char* what) { return check_hip(hipGetLastError(), what); }

// Raises a kernel's dynamic-LDS limit to `bytes` (hipFuncAttributeMaxDynamicSharedMemorySize) unless an earlier call
// on this device already set it at least that high: the attribute call costs microseconds of host time per launch.
int ensure_lds_limit(const void* kernel, size_t bytes, const char* what);

inline bool is_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

constexpr int kWave = 64;
constexpr uint32_t Q4K_BYTES = 144, Q5K_BYTES = 176, Q6K_BYTES = 210, Q8_0_BYTES = 34, Q4_0_BYTES = 18;

// ---- launchers (one per .hip file); all validate nothing: the C entry points do ----
int launch_dequant(hipStream_t s, const void* w, void* out, hq_act_dtype odt, uint64_t n_elems,
                   hq_ggml_type t);
// imatrix: nullptr, or n_per_row importance weights shared by every row; row_scratch: one float per row, used by Q4_0
// with an importance matrix only.
int launch_quantize(hipStream_t s, const float* src, uint64_t n_elems, uint64_t n_per_row,
                    hq_ggml_type t, void* out, const float* imatrix = nullptr, float* row_scratch = nullptr);

struct GemvArgs {
    const void* x;        // [x_rows, k] activations
    const void* x2;       // nullptr, or f32 [x_rows, k]: the activations are silu(x) * x2
    const uint8_t* w;     // weight blocks, or the expert stack when ids != nullptr
    const uint32_t* ids;  // [pairs] expert ids, or nullptr for the dense form
    float* y;             // [pairs, n]
    uint32_t pairs;       // dense: m; id form: n_tokens*top_k
    uint32_t top_k;       // id form: x row of pair p is p / top_k; dense: 1
    uint32_t n, k;
    uint32_t n_experts;
    uint64_t expert_stride;  // bytes
    // Routing computed by the launch itself (ids == nullptr, n_experts <= 256): router logits [pairs / top_k, n_experts];
    // the expert of pair p is slot p % top_k of its token's softmax / top-k.  route_ids / route_w: nullptr, or where the
    // selection is also written ([pairs] each) for the launches that follow.
    const float* route_logits;
    uint32_t* route_ids;
    float* route_w;
};
// The F16-shadow product (shadow.hip): activations cast to f16 into `workspace`, then the vendor library's GEMM.
size_t f16_shadow_workspace_bytes(uint32_t m, uint32_t k);
int launch_f16_shadow_matmul(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_f16, float* y, uint32_t m, uint32_t n,
                             uint32_t k, void* workspace, size_t workspace_bytes);
// The same over weights stored as f32 (bf16 activations are widened into the workspace).
size_t f32_dense_workspace_bytes(uint32_t m, uint32_t k, hq_act_dtype xdt);
int launch_f32_dense_matmul(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_f32, float* y, uint32_t m, uint32_t n,
                            uint32_t k, void* workspace, size_t workspace_bytes);
// One row at a time over f16 or f32 weights (dense.hip): k a multiple of 8 (f16) or 4 (f32) that fits LDS as f32.
bool dense_gemv_takes(uint32_t k, hq_act_dtype wdt);
int launch_dense_gemv(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, hq_act_dtype wdt, float* y, uint32_t m, uint32_t n,
                      uint32_t k);
// The current device's CU count (cached).
int cu_count(uint32_t* out);
int launch_gemv(hipStream_t s, const GemvArgs& a, hq_act_dtype xdt, hq_ggml_type t);
// True where a few dense rows are better served by launch_gemv (which takes them up to four at a time, one pass over
// the weights each) than by the small-batch kernel.
bool gemv_stream_passes_preferred(hq_ggml_type t, hq_act_dtype xdt, uint32_t m, uint32_t n, uint32_t k);
void gemv_flat_plan(hq_ggml_type t, uint32_t n, uint32_t k, uint32_t waves, uint32_t* units_per_row, uint32_t* rows_per_task,
                    uint32_t* windows_per_task, uint32_t* units_per_window, uint32_t* window_capacity);
// Up to four independent GEMVs of one weight type and activation dtype in a single launch.
int launch_gemv_jobs(hipStream_t s, const GemvArgs* jobs, uint32_t n_jobs, hq_act_dtype xdt, hq_ggml_type t);

int launch_gemv_swiglu(hipStream_t s, const void* x, hq_act_dtype xdt, const void* wg, const void* wu, float* y, uint32_t m, uint32_t n,
                       uint32_t k, hq_ggml_type t, bool dry);

// 3..8 activation rows sharing one pass over the weights (gemvm.hip); gemv_rows_supported() says
// whether (type, m, k) has such a kernel, otherwise the GEMV runs once per row.
bool gemv_rows_supported(hq_ggml_type t, uint32_t m, uint32_t k);
// bf16 rows the small-batch kernel takes in its stage-once form with the transposed weight fetch (gemvm.hip).
bool gemv_rows_stream_fast(hq_ggml_type t, hq_act_dtype xdt, uint32_t m, uint32_t n, uint32_t k);
// ... and whether the stage-once form takes the product at all (any k of whole super-blocks that fits a CU's LDS).
bool gemv_rows_stream_takes(hq_ggml_type t, hq_act_dtype xdt, uint32_t m, uint32_t n, uint32_t k);
int launch_gemv_rows(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m, uint32_t n,
                     uint32_t k, hq_ggml_type t);
// The same for the 32-weight-block types (Q8_0, Q4_0), 2 <= m <= 8: exact products on the VALU, every weight fetched
// once for all rows.
bool gemv_rows32_supported(hq_ggml_type t, uint32_t m, uint32_t k);
int launch_gemv_rows32(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m, uint32_t n,
                       uint32_t k, hq_ggml_type t);

// MFMA GEMM for m > 8 (prefill).  gemm_supported() says whether (type, k) has a tile kernel.
bool gemm_supported(hq_ggml_type t, uint32_t k);
int launch_gemm(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m, uint32_t n,
                uint32_t k, hq_ggml_type t);
// GEMM on the f16 matrix cores with an activation pre-pass (Q4_K with k % 256 == 0, Q8_0 with
// k % 128 == 0); needs a device workspace of gemm_f16_tile_workspace_bytes().
bool gemm_f16_tile_supported(hq_ggml_type t, uint32_t k);
size_t gemm_f16_tile_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t);
// perm_hd != 0: the activations are stored [k / perm_hd][m][perm_hd] (attention output, heads outermost) and are
// gathered by the pre-pass.
int launch_gemm_f16_tile(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m,
                         uint32_t n, uint32_t k, hq_ggml_type t, void* workspace, uint32_t perm_hd = 0,
                         const float* w_scales = nullptr, const float* gate_in = nullptr);
// Whether launch_gemm_f16_tile takes gate_in for this shape (not where k is cut into slices).
bool gemm_f16_tile_gated_supported(hq_ggml_type t, uint32_t m, uint32_t n, uint32_t k);
// The tile kernels' weight-row scales (n_rows floats, a function of the weights alone): what the pre-pass of every tile
// or grouped call works out when w_scales is null.
int launch_weight_row_scales(hipStream_t s, const void* w, float* scales, uint32_t n_rows, uint32_t k, hq_ggml_type t);

// y = silu(x . Wg^T) * (x . Wu^T) on the tile route (Q4_K / Q5_K, k % 256 == 0): both products of a dense SwiGLU
// layer and the gating as one launch after the pre-pass; gate_scales / up_scales: both null, or both the caller's.
size_t gemm_f16_swiglu_workspace_bytes(uint32_t m, uint32_t n, uint32_t k);
int launch_gemm_f16_swiglu(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up, float* y, uint32_t m,
                           uint32_t n, uint32_t k, hq_ggml_type t, void* workspace, const float* gate_scales, const float* up_scales);

// Grouped form of the tile GEMM for mul_mat_id with many routed rows: rows sorted by expert, one
// tile = up to 256 rows of one expert; needs a contiguous stack (expert_stride = n rows) and a device
// workspace of gemm_f16_grouped_workspace_bytes().
bool gemm_f16_grouped_supported(hq_ggml_type t, uint32_t n, uint32_t k, uint32_t n_experts, uint64_t expert_stride, uint64_t pairs);
size_t gemm_f16_grouped_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t n_experts, uint32_t n, uint32_t k,
                                        uint32_t stacks = 1);
// w_stack2 (Q4_K / Q5_K, see gemm_f16_grouped_swiglu_supported): y = silu(W[ids] . x) * (W2[ids] . x), the gate and up
// projections of a MoE block and their SwiGLU as one grouped product; workspace for stacks = 2.
bool gemm_f16_grouped_swiglu_supported(hq_ggml_type t);
int launch_gemm_f16_grouped(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_stack, const uint32_t* ids, float* y,
                            void* workspace, uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k, uint32_t n_experts,
                            uint64_t expert_stride, hq_ggml_type t, const float* w_scales = nullptr,
                            const void* w_stack2 = nullptr, const float* w_scales2 = nullptr);

// MoE glue (moe.hip)
int launch_dense_gemv_bf16(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m,
                           uint32_t n, uint32_t k);
int launch_dense_gemv_bf16_pair(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_a, float* y_a, uint32_t n_a,
                                const void* w_b, float* y_b, uint32_t n_b, uint32_t m, uint32_t k);
int launch_moe_softmax_topk(hipStream_t s, const float* logits, uint32_t* ids, float* weights, uint32_t n_tokens,
                            uint32_t n_experts, uint32_t top_k);
// dst[m][k] <- src stored [k / head_dim][m][head_dim]; elem_bytes 2 or 4
int launch_unpermute021(hipStream_t s, const void* src, void* dst, uint32_t m, uint32_t k, uint32_t head_dim, uint32_t elem_bytes);
int launch_silu_mul(hipStream_t s, const float* gate, const float* up, float* out, uint64_t n);
int launch_moe_weighted_reduce(hipStream_t s, const float* y, const float* w, const float* shared, const float* shared_logit,
                               const float* residual, float* out, uint32_t n_tokens, uint32_t top_k, uint32_t hidden);

// The whole MoE FFN block of a decode step in one launch (moe_fused.hip).
struct MoeFusedArgs {
    const void* x;                  // [n_tokens, hidden] bf16
    const void* router;             // [n_experts, hidden] bf16
    const void* shared_gate_logit;  // [hidden] bf16 or nullptr
    const void *expert_gate, *expert_up, *expert_down, *shared_gate, *shared_up, *shared_down;
    const float* residual;          // nullptr or [n_tokens, hidden]
    float* out;                     // [n_tokens, hidden]
    uint32_t* route_ids;            // nullptr or out [n_tokens * top_k]
    float* route_weights;
    void* scratch;
    uint32_t n_tokens, n_experts, top_k;
    uint64_t stride_gate_up, stride_down;
    uint32_t spin_limit;            // 0: default
    hq_ggml_type t_gate_up, t_down;
};
bool moe_fused_supported(uint32_t n_tokens, uint32_t hidden, uint32_t n_experts, uint32_t top_k, uint32_t inter,
                         uint32_t shared_inter, hq_ggml_type t, hq_ggml_type t_down, hq_act_dtype xdt);
size_t moe_fused_scratch_bytes(uint32_t n_tokens, uint32_t n_experts, uint32_t top_k);
int launch_moe_fused(hipStream_t s, const MoeFusedArgs& a);

// The dense SwiGLU FFN of one decode token in one launch (dense_ffn.hip).  dry: only say whether the shape is taken.
struct DenseFfnArgs {
    const void* x;  // [hidden]
    hq_act_dtype xdt;
    const void *w_gate, *w_up, *w_down;
    hq_ggml_type t_gate_up, t_down;
    const float* residual;  // nullptr or [hidden]
    float* out;             // [hidden]
    void* scratch;
    uint32_t hidden, inter;
    uint32_t spin_limit;  // 0: default
};
size_t dense_ffn_scratch_bytes(uint32_t inter);
int launch_dense_ffn(hipStream_t s, const DenseFfnArgs& a, bool dry);
void gemm_f16_small_tile_slices(hq_ggml_type t, uint32_t m, uint32_t n, uint32_t k, uint32_t* splits, uint32_t* sb_per);

// TurboQuant KV (tq.hip)
int launch_fwht_sign(hipStream_t s, float* buf, uint32_t n_heads, uint32_t head_dim, bool undo);
int launch_tq_encode(hipStream_t s, const float* src, uint8_t* codes, float* norms, uint32_t n_tokens,
                     uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t write_pos);
int launch_tq_dequantize(hipStream_t s, const uint8_t* codes, const float* norms, const float* lut, float* dst,
                         uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t start_pos, uint32_t n_tokens,
                         float scale_factor_d512, bool unrotate);
size_t tq_attn_tmp_bytes(uint32_t num_heads, uint32_t head_dim, uint32_t kv_seq_len);
int launch_tq_attention(hipStream_t s, const float* q, const uint8_t* k_codes, const float* k_norms,
                        const uint8_t* v_codes, const float* v_norms, const float* lut, float* out, float* tmp,
                        const hq_tq_attn_params& p, bool undo_rotation);

}  // namespace hq

// ---------------------------------------------------------------------------
// Device helpers
// ---------------------------------------------------------------------------
#if defined(__HIPCC__)
namespace hq {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

// IEEE binary16 bits -> f32, exact (v_cvt_f32_f16; subnormals preserved).
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h)));
}
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// silu(g) * u = g / (1 + exp(-g)) * u (ffn.rs:24-26).  Every step is a rounded operation of its own
// (no contraction into an fma), so that the stand-alone SwiGLU kernel and the down projection that
// forms its activations on the fly produce the same bits.
__device__ __forceinline__ float silu_mul_f32(float g, float u) {
#pragma clang fp contract(off)
    const float e = expf(-g);
    const float d = 1.f + e;
    return g / d * u;
}
// f32 -> bf16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// Loads that tolerate 2-byte alignment (Q6_K / Q8_0 blocks are 210 / 34 bytes).
// gfx950 under HSA runs with unaligned access enabled, so these compile to one
// global_load_dwordx4 / dwordx2 each.
__device__ __forceinline__ uint4 ld16_unaligned(const uint8_t* p) {
    uint4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}
__device__ __forceinline__ uint2 ld8_unaligned(const uint8_t* p) {
    uint2 v;
    __builtin_memcpy(&v, p, 8);
    return v;
}
__device__ __forceinline__ uint32_t ld4_unaligned(const uint8_t* p) {
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}
__device__ __forceinline__ uint32_t ld2(const uint8_t* p) {
    return *reinterpret_cast<const uint16_t*>(p);
}
// The same loads marked non-temporal, for data a kernel reads exactly once (the weights of a single-row product): the
// lines are not kept in the caches on their way in, and a streaming read of 510 MB runs at 6.9 instead of 6.0 TB/s.
typedef uint32_t hq_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t hq_u32x2 __attribute__((ext_vector_type(2)));
typedef hq_u32x4 hq_u32x4_a2 __attribute__((aligned(2)));
typedef hq_u32x2 hq_u32x2_a2 __attribute__((aligned(2)));
typedef uint32_t hq_u32_a2 __attribute__((aligned(2)));
__device__ __forceinline__ uint4 ldnt16(const uint8_t* p) {  // 16-byte aligned
    const hq_u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const hq_u32x4*>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ uint4 ldnt16_unaligned(const uint8_t* p) {  // 2-byte aligned, like the ones below
    const hq_u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const hq_u32x4_a2*>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ uint2 ldnt8_unaligned(const uint8_t* p) {
    const hq_u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const hq_u32x2_a2*>(p));
    return make_uint2(t.x, t.y);
}
__device__ __forceinline__ uint32_t ldnt4_unaligned(const uint8_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const hq_u32_a2*>(p));
}
__device__ __forceinline__ uint32_t ldnt2(const uint8_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(p));
}

// a.x*b.x + a.y*b.y + c on two packed bf16 pairs, f32 accumulate (v_dot2c_f32_bf16).
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                           __builtin_bit_cast(bf16x2_t, b), c, false);
}

// Exchanges across the 16-lane rows of a wave without LDS traffic: v_permlane16_swap / v_permlane32_swap hand every
// lane its own value and the one of lane ^ 16 (resp. lane ^ 32) as the pair r[0], r[1] — which of the two is the
// lane's own depends on the row, so they serve commutative operations.  The results have the bits of the
// __shfl_xor forms they replace.
__device__ __forceinline__ float xor16_add(float v) {
    const uint32_t u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor32_add(float v) {
    const uint32_t u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor16_max(float v) {
    const uint32_t u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor32_max(float v) {
    const uint32_t u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// x of lane ^ M without LDS traffic (a __shfl_xor is an LDS permute: a hundred cycles and more in a dependent chain).
// Inside a row of 16 lanes two DPP moves compose the xor from the mirrors the hardware has (half mirror = l ^ 7, row
// mirror = l ^ 15, quad reverse = l ^ 3); across rows a permlane swap delivers the pair (own row's value, partner
// row's value) and the lane picks the partner's: r[0] holds the even rows' (lower half's) values, r[1] the odd rows'.
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int M>
__device__ __forceinline__ float lane_xor(float x, uint32_t lane) {
    static_assert(M == 1 || M == 2 || M == 4 || M == 8 || M == 16 || M == 32, "one bit of the lane index");
    if constexpr (M == 1) {
        return dpp_mov<0xB1>(x);  // quad_perm [1,0,3,2]
    } else if constexpr (M == 2) {
        return dpp_mov<0x4E>(x);  // quad_perm [2,3,0,1]
    } else if constexpr (M == 4) {
        return dpp_mov<0x1B>(dpp_mov<0x141>(x));  // half mirror, then quad_perm [3,2,1,0]
    } else if constexpr (M == 8) {
        return dpp_mov<0x141>(dpp_mov<0x140>(x));  // row mirror, then half mirror
    } else if constexpr (M == 16) {
        const uint32_t u = __float_as_uint(x);
        const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
        return __uint_as_float(lane & 16u ? r[0] : r[1]);
    } else {
        const uint32_t u = __float_as_uint(x);
        const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        return __uint_as_float(lane & 32u ? r[0] : r[1]);
    }
}

// Butterfly reductions over aligned groups of lanes with the partners taken in the order of the xor distances
// given (the order fixes the rounding of a sum); every lane of a group gets the result.
template <int M, int... REST>
__device__ __forceinline__ float xor_sum(float v, uint32_t lane) {
    v += lane_xor<M>(v, lane);
    if constexpr (sizeof...(REST) > 0) v = xor_sum<REST...>(v, lane);
    return v;
}
template <int M, int... REST>
__device__ __forceinline__ float xor_max(float v, uint32_t lane) {
    v = fmaxf(v, lane_xor<M>(v, lane));
    if constexpr (sizeof...(REST) > 0) v = xor_max<REST...>(v, lane);
    return v;
}

// (a & b) | c in one VALU op.  The compiler splits this into v_and + v_or when b
// and c are literals (gfx9 VOP3 takes no literal operands), so the constants are
// passed in registers and the instruction is written out.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t b, uint32_t c) {
    // Plain C on purpose: the compiler fuses it into one v_and_or_b32 when b and c sit in VGPRs, and, unlike an
    // inline-asm instruction, counts it as a VALU write when it spaces a dependent MFMA (a matrix instruction that
    // reads a register less than two wait states after an asm-hidden write gets the old contents).
    return (a & b) | c;
}

// Q4_K: 6-bit scale / min of sub-blocks (2c, 2c+1) for chunk c in [0,4) from the
// 12 packed bytes held as three little-endian words (y = bytes 0..3, z = 4..7,
// w = 8..11).  Same bit fields as get_scale_min_k4
// (src/quantize/ggml_quants/q4_k.rs:329-337), evaluated branch-free.
__device__ __forceinline__ void q4k_scales(uint32_t y, uint32_t z, uint32_t w, int c, uint32_t& sc0,
                                           uint32_t& sc1, uint32_t& m0, uint32_t& m1) {
    // c < 2: sc = y.byte & 63, m = z.byte & 63.
    // c >= 2: sc = (w.byte & 15) | ((y.byte >> 6) << 4), m = (w.byte >> 4) | ((z.byte >> 6) << 4).
    // Selected with masks that depend on c only, so no divergent branch is formed.
    const int sh = (c & 1) * 16;
    const uint32_t sel = c < 2 ? 0xffffffffu : 0u;  // take y/z bytes directly
    const uint32_t lo = c < 2 ? 63u : 15u;
    const uint32_t hb = c < 2 ? 0u : 0x30u;
    const uint32_t ys = y >> sh, zs = z >> sh, ws = w >> sh;
    const uint32_t a = (ys & sel) | (ws & ~sel);
    const uint32_t b = (zs & sel) | ((ws >> 4) & ~sel);
    sc0 = (a & lo) | ((ys >> 2) & hb);
    sc1 = ((a >> 8) & lo) | ((ys >> 10) & hb);
    m0 = (b & lo) | ((zs >> 2) & hb);
    m1 = ((b >> 8) & lo) | ((zs >> 10) & hb);
}

__device__ __forceinline__ float ubyte0(uint32_t v) { return static_cast<float>(v & 0xffu); }
__device__ __forceinline__ float ubyte1(uint32_t v) { return static_cast<float>((v >> 8) & 0xffu); }
__device__ __forceinline__ float ubyte2(uint32_t v) { return static_cast<float>((v >> 16) & 0xffu); }
__device__ __forceinline__ float ubyte3(uint32_t v) { return static_cast<float>(v >> 24); }
__device__ __forceinline__ float sbyte(uint32_t v, int i) {
    return static_cast<float>(static_cast<int>(static_cast<int8_t>((v >> (8 * i)) & 0xffu)));
}

}  // namespace hq
#endif

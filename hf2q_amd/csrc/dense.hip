// Products with weights that are not quantized: y[m][n] = x[m][k] . W[n][k]^T for W in f16 or f32, row-major as in the
// file.  dispatch_qmatmul routes such tensors past the block kernels (src/serve/forward_mlx.rs:9820-9917): f32
// weights (a router projection) to dispatch_dense_matvec_f32 at m = 1 and dense_matmul_f32_f32_tensor above, native f16
// weights (tensors whose row length is not a multiple of 256, an f16 lm_head) to dispatch_dense_matvec_f16w_f32io and
// dispatch_mm_v2_f16.  Here: up to eight rows take the GEMV below, one pass over the weights per row; more rows the
// vendor library's GEMM (shadow.hip), f32 accumulation in both.
//
// The GEMV is a plain streaming read: one workgroup of 16 waves per CU stages x once as f32, a wave takes steps of 64 / L
// weight rows, L lanes a row (L = 64 from 64 16-byte pieces per row on), every lane eight pieces in flight, fetched with
// non-temporal loads; a piece is eight f16 or four f32 weights, widened exactly and multiplied in f32; the L partial
// sums meet in a DPP reduction.
#include <hip/hip_fp16.h>

#include <type_traits>

#include "gemv_pieces.h"
#include "hq_internal.h"

namespace hq {
namespace {

struct DenseGemvArgs {
    const void* x;
    const uint8_t* w;
    float* y;
    uint32_t n, k, log_l;
};

constexpr int DG_WAVES = 16, DG_INFLIGHT = 8;

// NT: the weights are fetched with non-temporal loads (large matrices: 1.24 GB in 192 instead of 215 us; a matrix of a
// megabyte or two is the faster for staying in the caches: 2.7 against 3.3 us).
template <bool W_F16, bool X_BF16, bool NT>
__global__ __launch_bounds__(64 * DG_WAVES) void dense_gemv_kernel(DenseGemvArgs a) {
    extern __shared__ float4 lds_x4[];  // k floats
    float* lds_x = reinterpret_cast<float*>(lds_x4);
    constexpr uint32_t EPC = W_F16 ? 8u : 4u;  // weights per 16-byte piece
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    // x: four values per thread and pass (k % 4 == 0)
    for (uint32_t i = tid; i < a.k / 4u; i += 64u * DG_WAVES) {
        float4 v;
        if constexpr (X_BF16) {
            const uint2 r = static_cast<const uint2*>(a.x)[i];
            v = make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                            __uint_as_float(r.y & 0xffff0000u));
        } else {
            v = static_cast<const float4*>(a.x)[i];
        }
        lds_x4[i] = v;
    }
    __syncthreads();
    const uint32_t cpr = a.k / EPC;  // pieces per row
    const uint32_t L = 1u << a.log_l, li = lane & (L - 1u), sub = lane >> a.log_l, rps = 64u >> a.log_l;
    const uint32_t steps = (a.n + rps - 1u) / rps, n_waves = gridDim.x * DG_WAVES;
    const size_t row_bytes = (size_t)cpr * 16u;
    for (uint32_t step = blockIdx.x + gridDim.x * wv; step < steps; step += n_waves) {
        const uint32_t row = step * rps + sub, rowc = row < a.n ? row : a.n - 1u;
        const uint4* wr = reinterpret_cast<const uint4*>(a.w + (size_t)rowc * row_bytes);
        float acc = 0.f;
        for (uint32_t c0 = 0; c0 < cpr; c0 += L * DG_INFLIGHT) {
            uint4 q[DG_INFLIGHT];
#pragma unroll
            for (int u = 0; u < DG_INFLIGHT; ++u) {
                const uint32_t c = c0 + (uint32_t)u * L + li;
                // (no branch around the load; a piece past the row's end adds nothing)  Non-temporal loads suit this
                // pattern: an instruction of the wave covers whole 128-byte lines (64 consecutive pieces of a row)
                const uint4* src = wr + (c < cpr ? c : cpr - 1u);
                q[u] = NT ? ldnt16(reinterpret_cast<const uint8_t*>(src)) : *src;
            }
#pragma unroll
            for (int u = 0; u < DG_INFLIGHT; ++u) {
                const uint32_t c = c0 + (uint32_t)u * L + li;
                const bool live = c < cpr;
                const float4* xp = reinterpret_cast<const float4*>(lds_x + (size_t)(live ? c : 0u) * EPC);
                float part = 0.f;
                if constexpr (W_F16) {
                    const float4 x0 = xp[0], x1 = xp[1];
                    const uint32_t w[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
                    const float xs[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        part = fmaf(f16_bits_to_f32(w[e] & 0xffffu), xs[2 * e], part);
                        part = fmaf(f16_bits_to_f32(w[e] >> 16), xs[2 * e + 1], part);
                    }
                } else {
                    const float4 x0 = xp[0];
                    part = fmaf(__uint_as_float(q[u].x), x0.x, part);
                    part = fmaf(__uint_as_float(q[u].y), x0.y, part);
                    part = fmaf(__uint_as_float(q[u].z), x0.z, part);
                    part = fmaf(__uint_as_float(q[u].w), x0.w, part);
                }
                acc += live ? part : 0.f;
            }
        }
        acc = group_sum(acc, a.log_l);
        if (li == 0u && row < a.n) a.y[row] = acc;
    }
}

}  // namespace

// k floats of LDS for x: rows of up to 40,000 values.
bool dense_gemv_takes(uint32_t k, hq_act_dtype wdt) { return k % (wdt == HQ_F16 ? 8u : 4u) == 0 && (size_t)k * 4 <= 160 * 1024 - 512; }

int launch_dense_gemv(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, hq_act_dtype wdt, float* y, uint32_t m, uint32_t n,
                      uint32_t k) {
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    const uint32_t cpr = k / (wdt == HQ_F16 ? 8u : 4u);
    uint32_t log_l = 0;
    while (log_l < 6u && (1u << log_l) < cpr) ++log_l;
    const uint32_t rps = 64u >> log_l, steps = (n + rps - 1u) / rps;
    const uint32_t grid = steps < cus ? steps : cus;
    const bool nt = (uint64_t)n * cpr * 16u >= (8ull << 20);
    auto pick = [&](auto w16, auto xbf) -> void (*)(DenseGemvArgs) {
        constexpr bool W16 = decltype(w16)::value, XBF = decltype(xbf)::value;
        return nt ? dense_gemv_kernel<W16, XBF, true> : dense_gemv_kernel<W16, XBF, false>;
    };
    void (*kern)(DenseGemvArgs) = wdt == HQ_F16 ? (xdt == HQ_BF16 ? pick(std::true_type{}, std::true_type{}) : pick(std::true_type{}, std::false_type{}))
                                                : (xdt == HQ_BF16 ? pick(std::false_type{}, std::true_type{}) : pick(std::false_type{}, std::false_type{}));
    const size_t lds = (size_t)k * 4;
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, "hipFuncSetAttribute(dense gemv LDS)")) return rc;
    const size_t xrow = (size_t)k * (xdt == HQ_BF16 ? 2 : 4);
    for (uint32_t r = 0; r < m; ++r) {
        const DenseGemvArgs a{static_cast<const uint8_t*>(x) + r * xrow, static_cast<const uint8_t*>(w), y + (size_t)r * n, n, k, log_l};
        hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * DG_WAVES), lds, s, a);
        if (int rc = check_launch("dense gemv kernel launch")) return rc;
    }
    return HQ_OK;
}

}  // namespace hq

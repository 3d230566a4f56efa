// Glue kernels around mul_mat_id for the MoE FFN block: router projection over
// bf16 weights, softmax + top-k + renormalise, SwiGLU gating, and the weighted
// reduction of expert outputs with the sigmoid-gated shared expert.  Semantics
// follow hf2q's CPU specification moe_ffn_cpu_ref
// (src/inference/models/qwen35/ffn.rs:179-336) and softmax_topk_renorm_cpu
// (src/inference/models/qwen35/gpu_ffn.rs:1879-1924).  All are small
// bandwidth-bound kernels; they exist so that a decode token's MoE layer runs
// without a host round trip between the router and the expert GEMVs.
#include <math.h>

#include "hq_internal.h"
#include "moe_topk.h"

namespace hq {
namespace {

// y[m, n] = x[m, k] . W[n, k]^T, W bf16 row-major, x f32 or bf16, fp32 accumulate.
// One wave per output row; grid (ceil((n_a + n_b)/4), m).  Two matrices over the same
// activations share the launch: rows below n_a belong to the first, the rest to the second.
template <bool X_BF16>
__global__ __launch_bounds__(256) void dense_gemv_bf16_kernel(const void* __restrict__ x, const uint16_t* __restrict__ w_a,
                                                              float* __restrict__ y_a, uint32_t n_a,
                                                              const uint16_t* __restrict__ w_b, float* __restrict__ y_b,
                                                              uint32_t n_b, uint32_t k) {
    const uint32_t lane = threadIdx.x & 63u, m = blockIdx.y;
    uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_a + n_b) return;
    const bool second = row >= n_a;
    if (second) row -= n_a;
    const uint16_t* w = second ? w_b : w_a;
    float* y = second ? y_b : y_a;
    const uint32_t n = second ? n_b : n_a;
    const uint4* wr = reinterpret_cast<const uint4*>(w + (size_t)row * k);
    float acc = 0.f;
    for (uint32_t c = lane; c < k / 8; c += 64) {  // 8 weights per step
        const uint4 wv = wr[c];
        const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
        float xv[8];
        if constexpr (X_BF16) {
            const uint4 t = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(x) + (size_t)m * k)[c];
            const uint32_t tw[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                xv[2 * i] = bf16_bits_to_f32(tw[i] & 0xffffu);
                xv[2 * i + 1] = bf16_bits_to_f32(tw[i] >> 16);
            }
        } else {
            const float4* xp = reinterpret_cast<const float4*>(static_cast<const float*>(x) + (size_t)m * k) + 2 * c;
            const float4 t0 = xp[0], t1 = xp[1];
            xv[0] = t0.x, xv[1] = t0.y, xv[2] = t0.z, xv[3] = t0.w, xv[4] = t1.x, xv[5] = t1.y, xv[6] = t1.z, xv[7] = t1.w;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc = fmaf(bf16_bits_to_f32(ww[i] & 0xffffu), xv[2 * i], acc);
            acc = fmaf(bf16_bits_to_f32(ww[i] >> 16), xv[2 * i + 1], acc);
        }
    }
    acc = wave_sum(acc);
    if (lane == 0) y[(size_t)m * n + row] = acc;
}

template <int PL>
__global__ __launch_bounds__(64) void moe_softmax_topk_kernel(const float* __restrict__ logits, uint32_t* __restrict__ ids,
                                                              float* __restrict__ weights, uint32_t n_experts,
                                                              uint32_t top_k) {
    const uint32_t t = blockIdx.x, lane = threadIdx.x;
    uint32_t id;
    float w;
    softmax_topk_lane<PL>(logits + (size_t)t * n_experts, n_experts, top_k, lane, id, w);
    if (lane < top_k) {
        ids[(size_t)t * top_k + lane] = id;
        weights[(size_t)t * top_k + lane] = w;
    }
}

__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                       float* __restrict__ out, uint64_t n4) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const float4 g = reinterpret_cast<const float4*>(gate)[i], u = reinterpret_cast<const float4*>(up)[i];
    float4 o;
    o.x = silu_mul_f32(g.x, u.x);
    o.y = silu_mul_f32(g.y, u.y);
    o.z = silu_mul_f32(g.z, u.z);
    o.w = silu_mul_f32(g.w, u.w);
    reinterpret_cast<float4*>(out)[i] = o;
}

// out[t, :] = sum_s w[t, s] * y[t, s, :]  (+ sigmoid(shared_logit[t]) * shared[t, :])  (+ residual[t, :])
__global__ __launch_bounds__(256) void moe_weighted_reduce_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                                  const float* __restrict__ shared,
                                                                  const float* __restrict__ shared_logit,
                                                                  const float* __restrict__ residual, float* __restrict__ out,
                                                                  uint32_t top_k, uint32_t hidden) {
    const uint32_t t = blockIdx.y, i = blockIdx.x * 256 + threadIdx.x;  // i indexes float4 columns
    if (i >= hidden / 4) return;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t s = 0; s < top_k; ++s) {
        const float ws = w[(size_t)t * top_k + s];
        const float4 v = reinterpret_cast<const float4*>(y + ((size_t)t * top_k + s) * hidden)[i];
        acc.x = fmaf(ws, v.x, acc.x);
        acc.y = fmaf(ws, v.y, acc.y);
        acc.z = fmaf(ws, v.z, acc.z);
        acc.w = fmaf(ws, v.w, acc.w);
    }
    if (shared) {
        const float g = shared_logit ? 1.f / (1.f + expf(-shared_logit[t])) : 1.f;  // ffn.rs:28-30 sigmoid
        const float4 v = reinterpret_cast<const float4*>(shared + (size_t)t * hidden)[i];
        acc.x = fmaf(g, v.x, acc.x);
        acc.y = fmaf(g, v.y, acc.y);
        acc.z = fmaf(g, v.z, acc.z);
        acc.w = fmaf(g, v.w, acc.w);
    }
    if (residual) {
        const float4 v = reinterpret_cast<const float4*>(residual + (size_t)t * hidden)[i];
        acc.x += v.x;
        acc.y += v.y;
        acc.z += v.z;
        acc.w += v.w;
    }
    reinterpret_cast<float4*>(out + (size_t)t * hidden)[i] = acc;
}

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

// The same product for many activation rows (the router of a prefill chunk: 2048 tokens x 256 experts), bf16
// activations: both operands go from memory straight into the matrix cores.  One workgroup per tile of 32 token rows x
// 64 weight rows, its four waves a quarter of k each; a wave reads one activation fragment and two weight fragments per
// k-step (eight k-steps of loads in flight) for two MFMAs -- the loads are row-strided, a cache line per lane, and their
// line look-ups are what bounds the kernel, so fewer of them per MFMA is what counts.  The partial tiles are added in
// wave order through LDS.  The bf16 products are exact and the sums f32.  The weights are the MFMA's first operand, so
// a lane ends up with sixteen outputs of ONE token (lane % 32) per weight tile, four runs of four consecutive n.  Rows
// past m or n repeat the last one and are not stored.  k % 16 == 0.
// f32 activations are split into three bf16 terms each (truncations of x, of x - hi and of the rest: every step exact, 24
// significant bits in all), so an activation fragment costs three MFMAs per weight tile and the products stay exact.
template <bool X_BF16>
__global__ __launch_bounds__(256) void dense_gemm_bf16_kernel(const void* __restrict__ xv, const uint16_t* __restrict__ w,
                                                              float* __restrict__ y, uint32_t m, uint32_t n, uint32_t k) {
    __shared__ float part[3][2][16][64];
    const uint32_t lane = threadIdx.x & 63u, l32 = lane & 31u, lg = lane >> 5, wave = threadIdx.x >> 6;
    const uint32_t tiles_n = (n + 63u) / 64u;
    const uint32_t m0 = (blockIdx.x / tiles_n) * 32u, n0 = (blockIdx.x % tiles_n) * 64u;
    const uint32_t xr = m0 + l32 < m ? m0 + l32 : m - 1u;
    // this lane's k-group of eight values: one uint4 of bf16, or two of f32
    const uint4* xp = X_BF16 ? reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(xv) + (size_t)xr * k) + lg
                             : reinterpret_cast<const uint4*>(static_cast<const float*>(xv) + (size_t)xr * k) + 2u * lg;
    // k-step st of the activations: 1 (bf16) or 3 (f32) fragments
    constexpr int XT = X_BF16 ? 1 : 3;
    auto x_frags = [&](uint32_t st, bf16x8_t* f) {
        if constexpr (X_BF16) {
            f[0] = __builtin_bit_cast(bf16x8_t, xp[2u * st]);
        } else {
            const uint4 v0 = xp[4u * st], v1 = xp[4u * st + 1u];
            const uint32_t u[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
            uint32_t t[3][8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t hi = u[i] & 0xffff0000u;
                // (inf / nan stay in the first term alone: inf - inf would turn an infinite product into nan)
                const float r1 = (hi & 0x7f800000u) == 0x7f800000u ? 0.f : __uint_as_float(u[i]) - __uint_as_float(hi);
                const uint32_t mid = __float_as_uint(r1) & 0xffff0000u;
                const float r2 = r1 - __uint_as_float(mid);
                t[0][i] = hi, t[1][i] = mid, t[2][i] = __float_as_uint(r2) & 0xffff0000u;
            }
#pragma unroll
            for (int j = 0; j < 3; ++j)
                f[j] = __builtin_bit_cast(bf16x8_t, make_uint4((t[j][0] >> 16) | t[j][1], (t[j][2] >> 16) | t[j][3],
                                                               (t[j][4] >> 16) | t[j][5], (t[j][6] >> 16) | t[j][7]));
        }
    };
    const uint4* wp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const uint32_t wr = n0 + 32u * t + l32 < n ? n0 + 32u * t + l32 : n - 1u;
        wp[t] = reinterpret_cast<const uint4*>(w + (size_t)wr * k) + lg;
    }
    f32x16_t acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
    const uint32_t steps = k / 16u, per = (steps + 3u) / 4u;
    uint32_t st = wave * per;
    const uint32_t end = st + per < steps ? st + per : steps;
    constexpr uint32_t UN = X_BF16 ? 8u : 4u;  // k-steps of loads in flight
    for (; st + UN <= end; st += UN) {
        uint4 a0[UN], a1[UN];
        bf16x8_t b[UN][XT];
#pragma unroll
        for (uint32_t u = 0; u < UN; ++u) a0[u] = wp[0][2u * (st + u)], a1[u] = wp[1][2u * (st + u)], x_frags(st + u, b[u]);
#pragma unroll
        for (uint32_t u = 0; u < UN; ++u)
#pragma unroll
            for (int j = XT - 1; j >= 0; --j) {  // the smallest term first
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a0[u]), b[u][j], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a1[u]), b[u][j], acc[1], 0, 0, 0);
            }
    }
    for (; st < end; ++st) {
        bf16x8_t b[XT];
        x_frags(st, b);
#pragma unroll
        for (int j = XT - 1; j >= 0; --j) {
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wp[0][2u * st]), b[j], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wp[1][2u * st]), b[j], acc[1], 0, 0, 0);
        }
    }
    if (wave) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) part[wave - 1][t][v][lane] = acc[t][v];
    }
    __syncthreads();
    if (wave || m0 + l32 >= m) return;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = ((acc[t][v] + part[0][t][v][lane]) + part[1][t][v][lane]) + part[2][t][v][lane];
        float* yp = y + (size_t)(m0 + l32) * n + n0 + 32u * t + 4u * lg;
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n0 + 32u * t + 4u * lg + 8u * g + i < n) yp[8 * g + i] = acc[t][4 * g + i];
    }
}

}  // namespace

int launch_dense_gemv_bf16_pair(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_a, float* y_a, uint32_t n_a,
                                const void* w_b, float* y_b, uint32_t n_b, uint32_t m, uint32_t k) {
    const uint16_t* wa = static_cast<const uint16_t*>(w_a);
    const uint16_t* wb = static_cast<const uint16_t*>(w_b);
    // Many activation rows (a prefill chunk) and a matrix of at least 32 rows: the matrix-core form for it (2048
    // tokens x 256 experts x 2048: one wave per (token, expert) over the whole row took 175 us); a second matrix of a few
    // rows (the shared expert's gate) keeps the one-wave-per-output form in a launch of its own.
    if (m >= 32 && n_a >= 32 && k % 16 == 0) {
        const uint32_t tiles_a = ((m + 31u) / 32u) * ((n_a + 63u) / 64u);
        if (xdt == HQ_BF16)
            hipLaunchKernelGGL(dense_gemm_bf16_kernel<true>, dim3(tiles_a), dim3(256), 0, s, x, wa, y_a, m, n_a, k);
        else
            hipLaunchKernelGGL(dense_gemm_bf16_kernel<false>, dim3(tiles_a), dim3(256), 0, s, x, wa, y_a, m, n_a, k);
        if (int rc = check_launch("dense bf16 gemm launch")) return rc;
        if (!n_b) return HQ_OK;
        return launch_dense_gemv_bf16_pair(s, x, xdt, w_b, y_b, n_b, nullptr, nullptr, 0, m, k);
    }
    const dim3 grid((n_a + n_b + 3) / 4, m);
    if (xdt == HQ_BF16)
        hipLaunchKernelGGL(dense_gemv_bf16_kernel<true>, grid, dim3(256), 0, s, x, wa, y_a, n_a, wb, y_b, n_b, k);
    else
        hipLaunchKernelGGL(dense_gemv_bf16_kernel<false>, grid, dim3(256), 0, s, x, wa, y_a, n_a, wb, y_b, n_b, k);
    return check_launch("dense bf16 gemv launch");
}

int launch_dense_gemv_bf16(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m,
                           uint32_t n, uint32_t k) {
    return launch_dense_gemv_bf16_pair(s, x, xdt, w, y, n, nullptr, nullptr, 0, m, k);
}

int launch_moe_softmax_topk(hipStream_t s, const float* logits, uint32_t* ids, float* weights, uint32_t n_tokens,
                            uint32_t n_experts, uint32_t top_k) {
    // experts per lane: 4 (<= 256 experts), 8 or 16 (<= 1024, the entry point's limit)
    if (n_experts <= 256)
        hipLaunchKernelGGL(moe_softmax_topk_kernel<4>, dim3(n_tokens), dim3(64), 0, s, logits, ids, weights, n_experts, top_k);
    else if (n_experts <= 512)
        hipLaunchKernelGGL(moe_softmax_topk_kernel<8>, dim3(n_tokens), dim3(64), 0, s, logits, ids, weights, n_experts, top_k);
    else
        hipLaunchKernelGGL(moe_softmax_topk_kernel<16>, dim3(n_tokens), dim3(64), 0, s, logits, ids, weights, n_experts, top_k);
    return check_launch("moe softmax_topk launch");
}

// One 16-byte piece per thread: dst row r, bytes [16 p, 16 p + 16) <- head (16 p) / head_bytes of the head-major source.
__global__ __launch_bounds__(256) void unpermute021_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, uint32_t m,
                                                           uint32_t row_pieces, uint32_t head_pieces) {
    const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (uint64_t)m * row_pieces) return;
    const uint32_t r = (uint32_t)(idx / row_pieces), p = (uint32_t)(idx % row_pieces);
    dst[idx] = src[((uint64_t)(p / head_pieces) * m + r) * head_pieces + p % head_pieces];
}

int launch_unpermute021(hipStream_t s, const void* src, void* dst, uint32_t m, uint32_t k, uint32_t head_dim, uint32_t elem_bytes) {
    const uint32_t row_pieces = k * elem_bytes / 16u, head_pieces = head_dim * elem_bytes / 16u;
    const uint64_t total = (uint64_t)m * row_pieces;
    hipLaunchKernelGGL(unpermute021_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, static_cast<const uint4*>(src),
                       static_cast<uint4*>(dst), m, row_pieces, head_pieces);
    return check_launch("unpermute kernel launch");
}

int launch_silu_mul(hipStream_t s, const float* gate, const float* up, float* out, uint64_t n) {
    const uint64_t n4 = n / 4;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, gate, up, out, n4);
    return check_launch("silu_mul launch");
}

int launch_moe_weighted_reduce(hipStream_t s, const float* y, const float* w, const float* shared, const float* shared_logit,
                               const float* residual, float* out, uint32_t n_tokens, uint32_t top_k, uint32_t hidden) {
    const dim3 grid((hidden / 4 + 255) / 256, n_tokens);
    hipLaunchKernelGGL(moe_weighted_reduce_kernel, grid, dim3(256), 0, s, y, w, shared, shared_logit, residual, out, top_k,
                       hidden);
    return check_launch("moe weighted_reduce launch");
}

}  // namespace hq

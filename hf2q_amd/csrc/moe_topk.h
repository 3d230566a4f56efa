// Softmax + top-k + renormalise over one token's router logits by one wave, shared by the stand-alone kernel
// (moe.hip) and by the routed GEMV launch that computes its own routing (gemv.hip).  softmax_topk_renorm_cpu
// (src/inference/models/qwen35/gpu_ffn.rs:1879-1924) is the specification.
#pragma once
#include <math.h>

#include "hq_internal.h"

namespace hq {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// Wave-wide maximum of a 64-bit key with DPP moves only (no LDS traffic); every lane gets the result.  Two passes over
// 32-bit halves: the largest high word, then the largest low word among the lanes that hold it (a key's low word is
// never 0 unless the key is absent), which is the 64-bit maximum with half the moves of a 64-bit exchange.  Quad
// permutes and row mirrors cover a row of 16 lanes, row_bcast 15 / 31 carry the row maxima upwards, lane 63 then holds
// the maximum and is read back as a scalar.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, ROW_MASK, 0xf, false);
    return o > v ? o : v;
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = dpp_max_u32<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
    v = dpp_max_u32<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
    v = dpp_max_u32<0x141, 0xf>(v);  // row_half_mirror
    v = dpp_max_u32<0x140, 0xf>(v);  // row_mirror
    v = dpp_max_u32<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_max_u32<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
    const uint32_t hi = wave_max_u32((uint32_t)(v >> 32));
    const uint32_t lo = wave_max_u32((uint32_t)(v >> 32) == hi ? (uint32_t)v : 0u);
    return ((uint64_t)hi << 32) | lo;
}

// One wave per token, lane s < top_k receives slot s (expert id and renormalised weight): probabilities over all experts, the top_k largest (ties -> lower expert id,
// as a stable descending sort gives), renormalised over the selection (uniform if it sums to ~0).
// PL = experts per lane (n_experts <= 64 * PL).  A candidate is the key (probability bits,
// ~expert id): probabilities are >= 0, so their bit patterns order like the values, and the
// complemented id makes the lower expert win a tie; 0 marks a taken or absent candidate.
template <int PL>
__device__ __forceinline__ void softmax_topk_lane(const float* __restrict__ row, uint32_t n_experts, uint32_t top_k, uint32_t lane,
                                                  uint32_t& out_id, float& out_w) {
    float p[PL];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PL; ++i) {
        const uint32_t e = lane + 64u * i;
        p[i] = e < n_experts ? row[e] : -INFINITY;
        mx = fmaxf(mx, p[i]);
    }
    mx = wave_max(mx);
    float denom = 0.f;
#pragma unroll
    for (int i = 0; i < PL; ++i) {
        const uint32_t e = lane + 64u * i;
        p[i] = e < n_experts ? expf(p[i] - mx) : 0.f;
        denom += p[i];
    }
    denom = wave_sum(denom);
    const float inv_d = denom > 1e-20f ? 1.f / denom : 1.f;
    uint64_t key[PL];
#pragma unroll
    for (int i = 0; i < PL; ++i) {
        const uint32_t e = lane + 64u * i;
        key[i] = e < n_experts ? ((uint64_t)__float_as_uint(p[i] * inv_d) << 32) | (0xffffffffu - e) : 0ull;
    }

    float sum_sel = 0.f, my_w = 0.f;
    uint32_t my_id = 0;
    for (uint32_t s = 0; s < top_k; ++s) {
        uint64_t best = 0ull;
#pragma unroll
        for (int i = 0; i < PL; ++i) best = key[i] > best ? key[i] : best;
        best = wave_max_u64(best);  // uniform
#pragma unroll
        for (int i = 0; i < PL; ++i) key[i] = key[i] == best ? 0ull : key[i];  // keys are unique: only the owner matches
        const float bv = __uint_as_float((uint32_t)(best >> 32));
        const uint32_t be = 0xffffffffu - (uint32_t)best;
        sum_sel += bv;
        if (lane == s) {  // lane s keeps slot s (top_k <= 64)
            my_w = bv;
            my_id = be;
        }
    }
    const float inv_sum = sum_sel > 1e-20f ? 1.f / sum_sel : 1.f / (float)top_k;
    out_id = my_id;
    out_w = my_w * inv_sum;
}

}  // namespace hq

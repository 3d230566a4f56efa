// Softmax + top-k + renormalise over one token's router logits by one wave, shared by the stand-alone kernel
// (moe.hip) and by the routed GEMV launch that computes its own routing (gemv.hip).  softmax_topk_renorm_cpu
// (src/inference/models/qwen35/gpu_ffn.rs:1879-1924) is the specification.
#pragma once
#include <math.h>

#include "hq_internal.h"

namespace hq {

// Butterfly reductions over the 64 lanes, every lane gets the result: quad permutes and row mirrors inside a row of 16
// lanes, permlane swaps across the rows; no LDS traffic.  The sum adds the same pairs as an xor butterfly.
template <int CTRL>
__device__ __forceinline__ float dpp_partner(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_partner<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_partner<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_partner<0x141>(v);  // row_half_mirror
    v += dpp_partner<0x140>(v);  // row_mirror
    return xor32_add(xor16_add(v));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_partner<0xB1>(v));
    v = fmaxf(v, dpp_partner<0x4E>(v));
    v = fmaxf(v, dpp_partner<0x141>(v));
    v = fmaxf(v, dpp_partner<0x140>(v));
    return xor32_max(xor16_max(v));
}

// Wave-wide maximum of a signed 32-bit value, uniform: DPP inside the rows, row_bcast 15 / 31 carry the row maxima
// upwards, lane 63 then holds the maximum and is read back as a scalar.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_max_i32(int v) {
    const int o = __builtin_amdgcn_update_dpp(v, v, CTRL, ROW_MASK, 0xf, false);
    return o > v ? o : v;
}
__device__ __forceinline__ int wave_max_i32(int v) {
    v = dpp_max_i32<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
    v = dpp_max_i32<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
    v = dpp_max_i32<0x141, 0xf>(v);  // row_half_mirror
    v = dpp_max_i32<0x140, 0xf>(v);  // row_mirror
    v = dpp_max_i32<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_max_i32<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
    return __builtin_amdgcn_readlane(v, 63);
}

// One wave per token, lane s < top_k receives slot s (expert id and renormalised weight): probabilities over all
// experts, the top_k largest (ties -> lower expert id, as a stable descending sort gives), renormalised over the
// selection (uniform if it sums to ~0).  PL = experts per lane (n_experts <= 64 * PL), lane l holds the experts
// l, l + 64, ...
// Selection: probabilities are >= 0, so their bit patterns order like the values as signed integers, and -1 marks a
// taken or absent candidate.  A round takes the wave-wide maximum of the lanes' best candidates; nearly always one
// lane holds it and the round is done, otherwise (equal probabilities) the lowest expert id among the holders wins.
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
    int cand[PL];
#pragma unroll
    for (int i = 0; i < PL; ++i) cand[i] = lane + 64u * i < n_experts ? __float_as_int(p[i] * inv_d) : -1;

    float sum_sel = 0.f, my_w = 0.f;
    uint32_t my_id = 0;
    for (uint32_t s = 0; s < top_k; ++s) {
        // the lane's best candidate, the lower expert on equal probabilities
        int lb = cand[0];
        uint32_t li = 0;
#pragma unroll
        for (int i = 1; i < PL; ++i) {
            li = cand[i] > lb ? (uint32_t)i : li;
            lb = cand[i] > lb ? cand[i] : lb;
        }
        const int hi = wave_max_i32(lb);  // uniform; >= 0 while candidates are left (top_k <= n_experts)
        const uint64_t holders = __ballot(lb == hi);
        uint32_t be;
        if (__builtin_popcountll(holders) == 1) {  // uniform branch
            const uint32_t l = (uint32_t)__builtin_ctzll(holders);
            be = l + 64u * (uint32_t)__builtin_amdgcn_readlane((int)li, (int)l);
        } else {
            // several lanes hold equal probabilities: the lowest expert id among their best candidates
            const int inv = lb == hi ? (int)(0x7fffffffu - (lane + 64u * li)) : -1;
            be = 0x7fffffffu - (uint32_t)wave_max_i32(inv);
        }
#pragma unroll
        for (int i = 0; i < PL; ++i) cand[i] = lane + 64u * i == be ? -1 : cand[i];
        const float bv = __int_as_float(hi);
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

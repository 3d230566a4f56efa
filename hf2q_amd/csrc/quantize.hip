// Device-side GGML quantizers for Q4_K / Q5_K / Q6_K / Q8_0 / Q4_0, byte-identical to hf2q's
// CPU quantizers, without an importance matrix
// (src/quantize/ggml_quants/q4_k.rs:89-217, q6_k.rs:40-151, q8_0.rs:31-72 and the
// search helpers common.rs:61-167, 174-286) and with one (q4_k.rs:220-324, q5_k.rs:246-311,
// q6_k.rs:40-151 with weights, q4_0.rs:52-87; helpers common.rs:294-408 make_qkx3_quants and
// common.rs:415-518 make_qp_quants).  hf2q quantizes on the host at
// conversion / load time (in_memory_loader.rs:70-139); here the same bytes are
// produced on the GPU so that weights never have to cross PCIe as f32.
//
// Byte equality needs the same sequence of f32 roundings, so this file is built
// with -ffp-contract=off and uses fmaf exactly where the reference writes
// mul_add; divisions and sqrt are the correctly rounded ones (the HIP default).
// The scale search over a sub-block is an inherently sequential f32
// accumulation, so the parallelism is across sub-blocks: one thread per
// 32-element (Q4_K) or 16-element (Q6_K) sub-block, the super-block level
// decisions (max scale, 6-bit / int8 scale codes, f16 d) are combined through
// LDS, and the threads of a super-block then pack its bytes cooperatively.
#include <math.h>

#include "hq_internal.h"

namespace hq {
namespace {

constexpr float kGroupMaxEps = 1e-15f;  // common.rs:15

// common.rs:23-28: round-half-even through the 1.5*2^23 magic add.
__device__ __forceinline__ int nearest_int(float f) {
    const float v = f + 12582912.f;
    return (__float_as_int(v) & 0x007fffff) - 0x00400000;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));  // v_cvt_f16_f32, RNE
}

// ------------------------------------------------------------------ Q8_0
// q8_0.rs:31-72.  One thread per 32-element block.
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float* __restrict__ src, uint8_t* __restrict__ out,
                                                            uint64_t n_blocks) {
    const uint64_t b = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= n_blocks) return;
    float x[32];
    const float4* s4 = reinterpret_cast<const float4*>(src + b * 32);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float4 t = s4[i];
        x[4 * i] = t.x;
        x[4 * i + 1] = t.y;
        x[4 * i + 2] = t.z;
        x[4 * i + 3] = t.w;
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const float a = fabsf(x[i]);
        if (a > amax) amax = a;
    }
    const float d = amax / 127.f;
    const float id = d != 0.f ? 1.f / d : 0.f;
    uint8_t* o = out + b * Q8_0_BYTES;
    *reinterpret_cast<uint16_t*>(o) = (uint16_t)f32_to_f16_bits(d);
#pragma unroll
    for (int i = 0; i < 32; i += 2) {
        // Rust's f32::round is half-away-from-zero == roundf; `as i8` saturates.
        float r0 = roundf(x[i] * id), r1 = roundf(x[i + 1] * id);
        r0 = fminf(fmaxf(r0, -128.f), 127.f);
        r1 = fminf(fmaxf(r1, -128.f), 127.f);
        const uint32_t q0 = (uint32_t)(int)r0 & 0xffu, q1 = (uint32_t)(int)r1 & 0xffu;
        *reinterpret_cast<uint16_t*>(o + 2 + i) = (uint16_t)(q0 | (q1 << 8));
    }
}

// ------------------------------------------------------------------ Q4_K, Q5_K
// common.rs:174-286 make_qkx2_quants with n = 32, use_mad = false and
// nmax = 15, rmin = -1, rdelta = 0.1, nstep = 20 (Q4_K, the arguments of q4_k.rs:120-132) or
// nmax = 31, rmin = -0.5, rdelta = 0.1, nstep = 15 (Q5_K, q5_k.rs).
// L comes back packed four codes per word.
// V3 = true is common.rs:294-408 make_qkx3_quants as the importance-matrix paths call it (q4_k.rs:262-274,
// q5_k.rs:283-295): rmin = -0.9, rdelta = 0.05, nstep = 36, and the early return on max <= min.
template <int nmax, bool V3 = false>
__device__ float qkx2_search_32(const float (&x)[32], const float (&wt)[32], uint32_t (&Lp)[8], float& the_min) {
    constexpr int nstep = V3 ? 36 : nmax == 15 ? 20 : 15;
    constexpr float rmin = V3 ? -0.9f : nmax == 15 ? -1.f : -0.5f;
    constexpr float rdelta = V3 ? 0.05f : 0.1f;
    float mn = x[0], mx = x[0];
    float sum_w = wt[0];
    float sum_x = sum_w * x[0];
#pragma unroll
    for (int i = 1; i < 32; ++i) {
        if (x[i] < mn) mn = x[i];
        if (x[i] > mx) mx = x[i];
        sum_w += wt[i];
        sum_x = fmaf(wt[i], x[i], sum_x);
    }
    if (mn > 0.f) mn = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) Lp[i] = 0;
    if (V3 ? (mx <= mn) : (mx == mn)) {
        the_min = -mn;
        return 0.f;
    }
    float iscale = (float)nmax / (mx - mn);
    float scale = 1.f / iscale;
    float best_error = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        int l = nearest_int(iscale * (x[i] - mn));
        l = max(0, min(nmax, l));
        Lp[i >> 2] |= (uint32_t)l << (8 * (i & 3));
        float diff = fmaf(scale, (float)l, mn) - x[i];
        diff = diff * diff;
        best_error = fmaf(wt[i], diff, best_error);
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * (float)is + (float)nmax) / (mx - mn);
        float sum_l = 0.f, sum_l2 = 0.f, sum_xl = 0.f;
        uint32_t La[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) La[i] = 0;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            int l = nearest_int(iscale * (x[i] - mn));
            l = max(0, min(nmax, l));
            La[i >> 2] |= (uint32_t)l << (8 * (i & 3));
            const float lf = (float)l, w = wt[i];
            sum_l = fmaf(w, lf, sum_l);
            sum_l2 = fmaf(w * lf, lf, sum_l2);
            sum_xl = fmaf(w * lf, x[i], sum_xl);
        }
        const float D = fmaf(sum_w, sum_l2, -sum_l * sum_l);
        if (D > 0.f) {
            float this_scale = fmaf(sum_w, sum_xl, -sum_x * sum_l) / D;
            float this_min = fmaf(sum_l2, sum_x, -sum_l * sum_xl) / D;
            if (this_min > 0.f) {
                this_min = 0.f;
                this_scale = sum_xl / sum_l2;
            }
            float cur_error = 0.f;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const float lf = (float)((La[i >> 2] >> (8 * (i & 3))) & 0xffu);
                float diff = fmaf(this_scale, lf, this_min) - x[i];
                diff = diff * diff;
                cur_error = fmaf(wt[i], diff, cur_error);
            }
            if (cur_error < best_error) {
#pragma unroll
                for (int i = 0; i < 8; ++i) Lp[i] = La[i];
                best_error = cur_error;
                scale = this_scale;
                mn = this_min;
            }
        }
    }
    the_min = -mn;
    return scale;
}

// common.rs:415-518 make_qp_quants with n = 8, nmax = 63: the eight sub-block scales (or mins) of a super-block against
// their weights; the codes come back in L, the return value is the super-block's d (or dmin).
__device__ float qp_quants_8(const float* x, const float* qw, uint32_t* L) {
    constexpr int n = 8, nmax = 63;
    float mx = 0.f;
    for (int i = 0; i < n; ++i)
        if (x[i] > mx) mx = x[i];
    if (mx < kGroupMaxEps) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        return 0.f;
    }
    float iscale = (float)nmax / mx;
    for (int i = 0; i < n; ++i) L[i] = (uint32_t)nearest_int(iscale * x[i]) & 0xffu;
    const float scale = 1.f / iscale;
    float best_mse = 0.f;
    for (int i = 0; i < n; ++i) {
        const float diff = fmaf(scale, -(float)L[i], x[i]);
        best_mse = fmaf(qw[i] * diff, diff, best_mse);
    }
    for (int is = -4; is <= 4; ++is) {
        if (is == 0) continue;
        const float iscale_is = (0.1f * (float)is + (float)nmax) / mx;
        const float scale_is = 1.f / iscale_is;
        float mse = 0.f;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale_is * x[i]);
            if (l > nmax) l = nmax;
            const float diff = fmaf(scale_is, -(float)l, x[i]);
            mse = fmaf(qw[i] * diff, diff, mse);
        }
        if (mse < best_mse) {
            best_mse = mse;
            iscale = iscale_is;
        }
    }
    float sumlx = 0.f, suml2 = 0.f;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * x[i]);
        if (l > nmax) l = nmax;
        L[i] = (uint32_t)l & 0xffu;
        const float w = qw[i];
        sumlx = fmaf(w * x[i], (float)l, sumlx);
        suml2 = fmaf(w * (float)l, (float)l, suml2);
    }
    for (int itry = 0; itry < 5; ++itry) {
        int n_changed = 0;
        for (int i = 0; i < n; ++i) {
            const float w = qw[i];
            const float cur_l = (float)L[i];
            float slx = fmaf(w * x[i], -cur_l, sumlx);
            float sl2 = fmaf(w * cur_l, -cur_l, suml2);
            if (slx > 0.f && sl2 > 0.f) {
                int new_l = nearest_int(x[i] * sl2 / slx);
                if (new_l > nmax) new_l = nmax;
                if (((uint32_t)new_l & 0xffu) != L[i]) {
                    slx = fmaf(w * x[i], (float)new_l, slx);
                    sl2 = fmaf(w * (float)new_l, (float)new_l, sl2);
                    if (slx * slx * suml2 > sumlx * sumlx * sl2) {
                        L[i] = (uint32_t)new_l & 0xffu;
                        sumlx = slx;
                        suml2 = sl2;
                        ++n_changed;
                    }
                }
            }
        }
        if (!n_changed) break;
    }
    return suml2 > 0.f ? sumlx / suml2 : 0.f;
}

// q4_k.rs:89-217 (Q5 = false) and its five-bit twin q5_k.rs (Q5 = true: codes 0..31, the fifth bit of every code
// in qh, bit 2c for sub-block 2c and 2c + 1 for sub-block 2c + 1).  256 threads = 32 super-blocks x 8 sub-block
// threads.  IM: the importance-matrix paths q4_k.rs:220-324 / q5_k.rs:246-311: `imatrix` holds one weight per column of
// a row (n_per_row = 256 * blocks_per_row values); a sub-block's search weights are qw * sqrt(sigma2 + x^2) with sigma2
// from the whole super-block, and the super-block's scale and min codes come from make_qp_quants over the eight
// sub-blocks (one thread per super-block) instead of from the maxima.
template <bool Q5, bool IM = false>
__global__ __launch_bounds__(256) void quantize_q4_k_kernel(const float* __restrict__ src, uint8_t* __restrict__ out,
                                                            uint64_t n_blocks, const float* __restrict__ imatrix = nullptr,
                                                            uint32_t blocks_per_row = 1) {
    constexpr int NMAX = Q5 ? 31 : 15;
    __shared__ float s_scale[256], s_min[256];
    __shared__ float s_sw[IM ? 256 : 1], s_d[IM ? 64 : 1];  // IM: sub-block weight sums; d and dmin per super-block
    __shared__ uint32_t s_code[256];   // ls | lm << 8 per sub-block
    __shared__ uint32_t s_L[256 * 8];  // packed codes of every sub-block (32 bytes each)

    const uint32_t tid = threadIdx.x, j = tid & 7u, lb = tid >> 3;
    uint64_t blk = (uint64_t)blockIdx.x * 32 + lb;
    const bool live = blk < n_blocks;
    if (!live) blk = n_blocks - 1;  // keep every thread in the barriers; its result is discarded

    float x[32], wt[32];
    const float4* s4 = reinterpret_cast<const float4*>(src + blk * 256 + 32 * j);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float4 t = s4[i];
        x[4 * i] = t.x;
        x[4 * i + 1] = t.y;
        x[4 * i + 2] = t.z;
        x[4 * i + 3] = t.w;
    }
    uint32_t Lp[8];
    float the_min, scale;
    uint32_t ls, lm, d16, dmin16;
    if constexpr (IM) {
        // sigma2 from the sum of squares of the whole super-block, in element order (q4_k.rs:240-241): every thread
        // adds up all 256 for itself
        float sum_x2 = 0.f;
        const float4* b4 = reinterpret_cast<const float4*>(src + blk * 256);
        for (int i = 0; i < 64; ++i) {
            const float4 t = b4[i];
            sum_x2 = fmaf(t.x, t.x, sum_x2);
            sum_x2 = fmaf(t.y, t.y, sum_x2);
            sum_x2 = fmaf(t.z, t.z, sum_x2);
            sum_x2 = fmaf(t.w, t.w, sum_x2);
        }
        const float sigma2 = 2.f * sum_x2 / 256.f;
        const float* qw = imatrix + (size_t)(blk % blocks_per_row) * 256 + 32 * j;
        float sumw = 0.f;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            wt[i] = qw[i] * sqrtf(sigma2 + x[i] * x[i]);
            sumw += wt[i];
        }
        scale = qkx2_search_32<NMAX, true>(x, wt, Lp, the_min);
        s_scale[tid] = scale;
        s_min[tid] = the_min;
        s_sw[tid] = sumw;
        __syncthreads();
        if (j == 0) {  // the super-block's codes and d / dmin: make_qp_quants over its eight sub-blocks (q4_k.rs:277-278)
            uint32_t Ls[8], Lm[8];
            const float d_blk = qp_quants_8(&s_scale[lb * 8], &s_sw[lb * 8], Ls);
            const float dmin_blk = qp_quants_8(&s_min[lb * 8], &s_sw[lb * 8], Lm);
            for (int t = 0; t < 8; ++t) {
                const uint32_t a = Ls[t] > 63u ? 63u : Ls[t], b = Lm[t] > 63u ? 63u : Lm[t];
                s_code[lb * 8 + t] = a | (b << 8);
            }
            s_d[lb * 2] = d_blk;
            s_d[lb * 2 + 1] = dmin_blk;
        }
        __syncthreads();
        ls = s_code[tid] & 0xffu;
        lm = s_code[tid] >> 8;
        d16 = f32_to_f16_bits(s_d[lb * 2]);
        dmin16 = f32_to_f16_bits(s_d[lb * 2 + 1]);
    } else {
        float sum_x2 = 0.f;
#pragma unroll
        for (int i = 0; i < 32; ++i) sum_x2 = fmaf(x[i], x[i], sum_x2);
        const float av_x = sqrtf(sum_x2 / 32.f);
#pragma unroll
        for (int i = 0; i < 32; ++i) wt[i] = av_x + fabsf(x[i]);

        scale = qkx2_search_32<NMAX>(x, wt, Lp, the_min);
        s_scale[tid] = scale;
        s_min[tid] = the_min;
        __syncthreads();

        // Super-block maxima in sub-block order (strict > like the reference's scan).
        float max_scale = 0.f, max_min = 0.f;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float sc = s_scale[lb * 8 + t], mi = s_min[lb * 8 + t];
            if (sc > max_scale) max_scale = sc;
            if (mi > max_min) max_min = mi;
        }
        const float inv_scale = max_scale > 0.f ? 63.f / max_scale : 0.f;
        const float inv_min = max_min > 0.f ? 63.f / max_min : 0.f;
        ls = (uint32_t)nearest_int(inv_scale * scale) & 0xffu;  // `as u8` truncation
        lm = (uint32_t)nearest_int(inv_min * the_min) & 0xffu;
        ls = ls > 63u ? 63u : ls;
        lm = lm > 63u ? 63u : lm;
        s_code[tid] = ls | (lm << 8);
        d16 = f32_to_f16_bits(max_scale / 63.f);
        dmin16 = f32_to_f16_bits(max_min / 63.f);
    }

    // Second stage with the f16-rounded d / dmin (q4_k.rs:181-197).
    const float d = f16_bits_to_f32(d16) * (float)ls;
    if (d != 0.f) {
        const float dm = f16_bits_to_f32(dmin16) * (float)lm;
#pragma unroll
        for (int i = 0; i < 8; ++i) Lp[i] = 0;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            int l = nearest_int((x[i] + dm) / d);
            l = max(0, min(NMAX, l));
            Lp[i >> 2] |= (uint32_t)l << (8 * (i & 3));
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) s_L[tid * 8 + i] = Lp[i];
    __syncthreads();
    if (!live) return;

    // Pack: thread j writes the header (j == 0) and 16 bytes of qs.  Chunk c = j/2,
    // half h = j%2: bytes 16h..16h+15 of the chunk combine code l of sub-block 2c
    // (low nibble) with code l of sub-block 2c+1 (high nibble), l = 16h + i.
    uint8_t* o = out + blk * (Q5 ? Q5K_BYTES : Q4K_BYTES);
    if (j == 0) {
        uint32_t sc[8], mi[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            sc[t] = s_code[lb * 8 + t] & 0xffu;
            mi[t] = s_code[lb * 8 + t] >> 8;
        }
        uint32_t q[12];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            q[t] = sc[t] | ((sc[t + 4] >> 4) << 6);
            q[t + 4] = mi[t] | ((mi[t + 4] >> 4) << 6);
            q[t + 8] = (sc[t + 4] & 0xFu) | ((mi[t + 4] & 0xFu) << 4);
        }
        uint4 hdr;
        hdr.x = d16 | (dmin16 << 16);
        hdr.y = q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24);
        hdr.z = q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24);
        hdr.w = q[8] | (q[9] << 8) | (q[10] << 16) | (q[11] << 24);
        *reinterpret_cast<uint4*>(o) = hdr;
    }
    const uint32_t c = j >> 1, h = j & 1u;
    const uint32_t* lo = &s_L[(lb * 8 + 2 * c) * 8 + 4 * h];
    const uint32_t* hi = &s_L[(lb * 8 + 2 * c + 1) * 8 + 4 * h];
    constexpr uint32_t N4 = 0x0f0f0f0fu;  // (a no-op for Q4_K, whose codes have four bits)
    uint4 qs;
    qs.x = (lo[0] & N4) | ((hi[0] & N4) << 4);
    qs.y = (lo[1] & N4) | ((hi[1] & N4) << 4);
    qs.z = (lo[2] & N4) | ((hi[2] & N4) << 4);
    qs.w = (lo[3] & N4) | ((hi[3] & N4) << 4);
    *reinterpret_cast<uint4*>(o + (Q5 ? 48 : 16) + 32 * c + 16 * h) = qs;
    if constexpr (Q5) {
        // threads 0 and 1 of the super-block: qh bytes 16 j .. 16 j + 15, bit sb = the fifth bit of sub-block sb's code
        if (j < 2) {
            uint32_t qh[4] = {0, 0, 0, 0};
#pragma unroll
            for (int sb = 0; sb < 8; ++sb)
#pragma unroll
                for (int w = 0; w < 4; ++w) qh[w] |= ((s_L[(lb * 8 + sb) * 8 + 4 * j + w] >> 4) & 0x01010101u) << sb;
            *reinterpret_cast<uint4*>(o + 16 + 16 * j) = make_uint4(qh[0], qh[1], qh[2], qh[3]);
        }
    }
}

// ------------------------------------------------------------------ Q4_0
// q4_0.rs quantize_row (no imatrix): d = (the element of largest magnitude) / -8, codes trunc(x / d + 8.5) capped at
// 15; elements 0..15 in the low nibbles, 16..31 in the high ones.  One thread per block.
__global__ __launch_bounds__(256) void quantize_q4_0_kernel(const float* __restrict__ src, uint8_t* __restrict__ out,
                                                            uint64_t n_blocks) {
    const uint64_t b = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= n_blocks) return;
    float x[32];
    const float4* s4 = reinterpret_cast<const float4*>(src + b * 32);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float4 t = s4[i];
        x[4 * i] = t.x;
        x[4 * i + 1] = t.y;
        x[4 * i + 2] = t.z;
        x[4 * i + 3] = t.w;
    }
    float amax = 0.f, mx = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const float a = fabsf(x[i]);
        if (amax < a) {
            amax = a;
            mx = x[i];
        }
    }
    float d = mx / -8.f;
    // Opaque: otherwise the division and the conversion below become one v_fma_mixlo_f16 (mx * -0.125 + 0), and
    // the + 0 turns the -0.0 of an all-zero block into +0.0 (the reference stores 0x8000 there).
    asm volatile("" : "+v"(d));
    const float id = d != 0.f ? 1.f / d : 0.f;
    uint8_t* o = out + b * Q4_0_BYTES;
    *reinterpret_cast<uint16_t*>(o) = (uint16_t)f32_to_f16_bits(d);
#pragma unroll
    for (int i = 0; i < 16; i += 2) {
        uint32_t v = 0;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            // the reference casts to i8 (truncation towards zero; the values lie in [0.5, 16.5]) and caps at 15
            const int a = (int)(x[i + e] * id + 8.5f), c = (int)(x[16 + i + e] * id + 8.5f);
            v |= (uint32_t)((a < 15 ? a : 15) | ((c < 15 ? c : 15) << 4)) << (8 * e);
        }
        *reinterpret_cast<uint16_t*>(o + 2 + i) = (uint16_t)v;
    }
}

// ------------------------------------------------------------------ Q6_K
// common.rs:61-167 make_qx_quants with rmse_type = 1: n = 16, nmax = 32 for Q6_K (q6_k.rs:58; W: the sub-block's slice
// of the importance matrix as the weights, else x^2), n = 32, nmax = 8 with weights for Q4_0's importance-matrix path
// (q4_0.rs:75).  Codes come back as L = l + nmax, one per byte.
template <int N, int nmax, bool W>
__device__ float qx_search(const float (&x)[N], const float* qw, uint32_t (&Lp)[N / 4]) {
    float mx = 0.f, amax = 0.f;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            mx = x[i];
        }
    }
#pragma unroll
    for (int i = 0; i < N / 4; ++i) Lp[i] = 0;
    if (amax < kGroupMaxEps) return 0.f;
    float iscale = -(float)nmax / mx;
    float sumlx = 0.f, suml2 = 0.f;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        int l = nearest_int(iscale * x[i]);
        l = max(-nmax, min(nmax - 1, l));
        Lp[i >> 2] |= (uint32_t)(l + nmax) << (8 * (i & 3));
        const float w = W ? qw[i] : x[i] * x[i];
        sumlx = fmaf(w * x[i], (float)l, sumlx);
        suml2 = fmaf(w * (float)l, (float)l, suml2);
    }
    float scale = suml2 != 0.f ? sumlx / suml2 : 0.f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) continue;
        iscale = -((float)nmax + 0.1f * (float)is) / mx;
        sumlx = 0.f;
        suml2 = 0.f;
        uint32_t La[N / 4];
#pragma unroll
        for (int i = 0; i < N / 4; ++i) La[i] = 0;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            int l = nearest_int(iscale * x[i]);
            l = max(-nmax, min(nmax - 1, l));
            La[i >> 2] |= (uint32_t)(l + nmax) << (8 * (i & 3));
            const float w = W ? qw[i] : x[i] * x[i];
            sumlx = fmaf(w * x[i], (float)l, sumlx);
            suml2 = fmaf(w * (float)l, (float)l, suml2);
        }
        if (suml2 > 0.f && sumlx * sumlx > best * suml2) {
#pragma unroll
            for (int i = 0; i < N / 4; ++i) Lp[i] = La[i];
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

// Q4_0 with an importance matrix (q4_0.rs:52-87): sigma2 of a ROW = (sum of its squares, added in element order) / n_per_row,
// one thread per row; then per block weights qw * sqrt(sigma2 + x^2) and make_qx_quants(32, 8, rmse_type 1).
__global__ __launch_bounds__(64) void row_mean_square_kernel(const float* __restrict__ src, float* __restrict__ sigma2, uint64_t n_rows,
                                                             uint64_t n_per_row) {
    const uint64_t r = (uint64_t)blockIdx.x * 64 + threadIdx.x;
    if (r >= n_rows) return;
    const float* row = src + r * n_per_row;
    float sum = 0.f;
    for (uint64_t i = 0; i < n_per_row; ++i) sum += row[i] * row[i];
    sigma2[r] = sum / (float)n_per_row;
}
__global__ __launch_bounds__(256) void quantize_q4_0_im_kernel(const float* __restrict__ src, uint8_t* __restrict__ out, uint64_t n_blocks,
                                                               const float* __restrict__ imatrix, const float* __restrict__ sigma2,
                                                               uint32_t blocks_per_row) {
    const uint64_t b = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= n_blocks) return;
    float x[32], wt[32];
    const float4* s4 = reinterpret_cast<const float4*>(src + b * 32);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float4 t = s4[i];
        x[4 * i] = t.x;
        x[4 * i + 1] = t.y;
        x[4 * i + 2] = t.z;
        x[4 * i + 3] = t.w;
    }
    const float s2 = sigma2[b / blocks_per_row];
    const float* qw = imatrix + (size_t)(b % blocks_per_row) * 32;
#pragma unroll
    for (int i = 0; i < 32; ++i) wt[i] = qw[i] * sqrtf(s2 + x[i] * x[i]);
    uint32_t Lp[8];
    const float d = qx_search<32, 8, true>(x, wt, Lp);
    uint8_t* o = out + b * Q4_0_BYTES;
    *reinterpret_cast<uint16_t*>(o) = (uint16_t)f32_to_f16_bits(d);
    // byte j = code j | code (j + 16) << 4: words 0..3 hold codes 0..15, words 4..7 codes 16..31
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t v = (Lp[w] & 0x0f0f0f0fu) | ((Lp[w + 4] & 0x0f0f0f0fu) << 4);
        *reinterpret_cast<uint16_t*>(o + 2 + 4 * w) = (uint16_t)v;
        *reinterpret_cast<uint16_t*>(o + 4 + 4 * w) = (uint16_t)(v >> 16);
    }
}

// q6_k.rs:40-151.  256 threads = 16 super-blocks x 16 sub-block threads.
// IM: the sub-block's sixteen importance-matrix values are the search weights (q6_k.rs:58-64).
template <bool IM>
__global__ __launch_bounds__(256) void quantize_q6_k_kernel(const float* __restrict__ src, uint8_t* __restrict__ out,
                                                            uint64_t n_blocks, const float* __restrict__ imatrix = nullptr,
                                                            uint32_t blocks_per_row = 1) {
    __shared__ float s_scale[256];
    __shared__ uint32_t s_L[256 * 4];  // 16 code bytes per sub-block = the 256 codes of a super-block in order
    __shared__ int s_sc[256];

    const uint32_t tid = threadIdx.x, ib = tid & 15u, lb = tid >> 4;
    uint64_t blk = (uint64_t)blockIdx.x * 16 + lb;
    const bool live = blk < n_blocks;
    if (!live) blk = n_blocks - 1;

    float x[16];
    const float4* s4 = reinterpret_cast<const float4*>(src + blk * 256 + 16 * ib);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float4 t = s4[i];
        x[4 * i] = t.x;
        x[4 * i + 1] = t.y;
        x[4 * i + 2] = t.z;
        x[4 * i + 3] = t.w;
    }
    uint32_t Lp[4];
    const float scale = qx_search<16, 32, IM>(x, IM ? imatrix + (size_t)(blk % blocks_per_row) * 256 + 16 * ib : nullptr, Lp);
    s_scale[tid] = scale;
    __syncthreads();

    // First sub-block with the largest |scale| (strict > in sub-block order).
    float max_scale = 0.f, max_abs = 0.f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        const float sc = s_scale[lb * 16 + t];
        if (fabsf(sc) > max_abs) {
            max_abs = fabsf(sc);
            max_scale = sc;
        }
    }
    const bool zero_block = max_abs < kGroupMaxEps;
    uint32_t d16 = 0;
    int sc8 = 0;
    if (!zero_block) {
        const float iscale = -128.f / max_scale;
        d16 = f32_to_f16_bits(1.f / iscale);
        sc8 = min(127, nearest_int(iscale * scale));
        sc8 = (int)(int8_t)sc8;  // stored as int8
        const float d = f16_bits_to_f32(d16) * (float)sc8;
        if (d != 0.f) {
#pragma unroll
            for (int i = 0; i < 4; ++i) Lp[i] = 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                int l = nearest_int(x[i] / d);
                l = max(-32, min(31, l));
                Lp[i >> 2] |= (uint32_t)(l + 32) << (8 * (i & 3));
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) Lp[i] = 0;  // memset block (q6_k.rs:67-74)
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) s_L[tid * 4 + i] = Lp[i];
    s_sc[tid] = sc8;
    __syncthreads();
    if (!live) return;

    // Pack (q6_k.rs:112-150): thread ib covers half h = ib/8 and the four columns
    // l = 4*(ib%8) .. +3 of that half: 4 bytes of ql[l], 4 of ql[l+32], 4 of qh[l].
    uint8_t* o = out + blk * Q6K_BYTES;
    const uint32_t h = ib >> 3, l0 = 4 * (ib & 7u);
    const uint8_t* Lb = reinterpret_cast<const uint8_t*>(&s_L[lb * 64]) + 128 * h + l0;
    uint32_t ql_a = 0, ql_b = 0, qh = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t a = Lb[i], b = Lb[i + 32], c = Lb[i + 64], e = Lb[i + 96];
        ql_a |= ((a & 0xFu) | ((c & 0xFu) << 4)) << (8 * i);
        ql_b |= ((b & 0xFu) | ((e & 0xFu) << 4)) << (8 * i);
        qh |= ((a >> 4) | ((b >> 4) << 2) | ((c >> 4) << 4) | ((e >> 4) << 6)) << (8 * i);
    }
    // 210-byte blocks are only 2-byte aligned: store as 16-bit halves.
    uint16_t* p;
    p = reinterpret_cast<uint16_t*>(o + 64 * h + l0);
    p[0] = (uint16_t)ql_a;
    p[1] = (uint16_t)(ql_a >> 16);
    p = reinterpret_cast<uint16_t*>(o + 64 * h + 32 + l0);
    p[0] = (uint16_t)ql_b;
    p[1] = (uint16_t)(ql_b >> 16);
    p = reinterpret_cast<uint16_t*>(o + 128 + 32 * h + l0);
    p[0] = (uint16_t)qh;
    p[1] = (uint16_t)(qh >> 16);
    o[192 + ib] = zero_block ? 0 : (uint8_t)s_sc[lb * 16 + ib];
    if (ib == 0) *reinterpret_cast<uint16_t*>(o + 208) = (uint16_t)d16;
}

}  // namespace

int launch_quantize(hipStream_t s, const float* src, uint64_t n_elems, uint64_t n_per_row, hq_ggml_type t,
                    void* out, const float* imatrix, float* row_scratch) {
    uint8_t* o = static_cast<uint8_t*>(out);
    const bool im = imatrix != nullptr;
    if (t == HQ_Q8_0) {  // (q8_0.rs:31-72 takes the importance matrix and does not use it)
        const uint64_t nb = n_elems / 32;
        if ((nb + 255) / 256 > 0x7fffffffu) return fail(HQ_ERR_INVALID_ARGUMENT, "quantize: too many blocks");
        hipLaunchKernelGGL(quantize_q8_0_kernel, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, s, src, o, nb);
    } else if (t == HQ_Q4_K || t == HQ_Q5_K) {
        const uint64_t nb = n_elems / 256;
        const uint32_t bpr = (uint32_t)(n_per_row / 256);
        if ((nb + 31) / 32 > 0x7fffffffu) return fail(HQ_ERR_INVALID_ARGUMENT, "quantize: too many blocks");
        const dim3 grid((unsigned)((nb + 31) / 32));
        if (t == HQ_Q4_K) {
            if (im) hipLaunchKernelGGL((quantize_q4_k_kernel<false, true>), grid, dim3(256), 0, s, src, o, nb, imatrix, bpr);
            else hipLaunchKernelGGL((quantize_q4_k_kernel<false, false>), grid, dim3(256), 0, s, src, o, nb, nullptr, 1u);
        } else {
            if (im) hipLaunchKernelGGL((quantize_q4_k_kernel<true, true>), grid, dim3(256), 0, s, src, o, nb, imatrix, bpr);
            else hipLaunchKernelGGL((quantize_q4_k_kernel<true, false>), grid, dim3(256), 0, s, src, o, nb, nullptr, 1u);
        }
    } else if (t == HQ_Q4_0) {
        const uint64_t nb = n_elems / 32;
        if ((nb + 255) / 256 > 0x7fffffffu) return fail(HQ_ERR_INVALID_ARGUMENT, "quantize: too many blocks");
        if (im) {
            const uint64_t n_rows = n_elems / n_per_row;
            hipLaunchKernelGGL(row_mean_square_kernel, dim3((unsigned)((n_rows + 63) / 64)), dim3(64), 0, s, src, row_scratch, n_rows, n_per_row);
            if (int rc = check_launch("quantize row sums launch")) return rc;
            hipLaunchKernelGGL(quantize_q4_0_im_kernel, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, s, src, o, nb, imatrix, row_scratch,
                               (uint32_t)(n_per_row / 32));
        } else {
            hipLaunchKernelGGL(quantize_q4_0_kernel, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, s, src, o, nb);
        }
    } else if (t == HQ_Q6_K) {
        const uint64_t nb = n_elems / 256;
        if ((nb + 15) / 16 > 0x7fffffffu) return fail(HQ_ERR_INVALID_ARGUMENT, "quantize: too many blocks");
        if (im) hipLaunchKernelGGL(quantize_q6_k_kernel<true>, dim3((unsigned)((nb + 15) / 16)), dim3(256), 0, s, src, o, nb, imatrix, (uint32_t)(n_per_row / 256));
        else hipLaunchKernelGGL(quantize_q6_k_kernel<false>, dim3((unsigned)((nb + 15) / 16)), dim3(256), 0, s, src, o, nb, nullptr, 1u);
    } else {
        return fail(HQ_ERR_UNSUPPORTED, "quantize: ggml type %d", (int)t);
    }
    return check_launch("quantize kernel launch");
}

}  // namespace hq

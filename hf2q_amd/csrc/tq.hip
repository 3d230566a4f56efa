// TurboQuant-style 8-bit KV cache: sign x FWHT rotation, write-side encode, and
// single-query decode attention that dequantises the cache in-kernel.
//
// Cache layout (src/inference/models/qwen35/kv_cache.rs:1982-2113): codes
// [n_kv_heads, capacity, head_dim] u8, norms [n_kv_heads, capacity, head_dim/256]
// f32.  A cached element is  norm * int8(code)  (linear map), or
// lut[code] * norm / 16 / scale_factor  when a 256-entry table is supplied.
//
// Decode attention is HBM-bound: 2*(head_dim+4) bytes per (kv head, position),
// read once.  The sequence is split over workgroups (flash-decoding); every
// wave walks 16-position tiles of its split:
//   * scores: K codes are turned into bf16 (an int8 is exact in bf16) and
//     multiplied with the up-to-8 query heads of the GQA group on the matrix
//     cores (v_mfma_f32_16x16x32_bf16; the queries are an exact hi+lo bf16 split
//     of the f32 input), then scaled by scale * norm_k in fp32;
//   * online softmax in fp32 on the MFMA result layout;
//   * P.V on the VALU: a lane owns 8 output coordinates for all heads, reads 8
//     V codes per position (v_cvt) and does fp32 FMAs with p * norm_v broadcast
//     from LDS, so no transposed V operand is needed.
// Partial (max, sum, unnormalised output) per split go to `tmp`; a second kernel
// merges the splits.
#include <math.h>

#include "hq_internal.h"

namespace hq {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// kv_cache.rs:3871-3876: bit j of byte j>>3 set => element j is negated.
__constant__ uint8_t kSigns256[32] = {0xa7, 0x3b, 0x91, 0xf4, 0x6d, 0xc2, 0x58, 0x0e, 0xb3, 0x7f, 0x24,
                                      0xd6, 0x89, 0x45, 0xea, 0x1c, 0x63, 0xaf, 0xd8, 0x52, 0x97, 0x0b,
                                      0xe1, 0x3d, 0x76, 0xc4, 0x19, 0xfe, 0x4a, 0x85, 0x2c, 0xdb};

// Lane l of a wave holds elements 4l..4l+3 of a 256-vector.
__device__ __forceinline__ void apply_signs(float (&v)[4], uint32_t lane) {
    const uint32_t bits = kSigns256[lane >> 1] >> (4 * (lane & 1u));  // elements 4l..4l+3
#pragma unroll
    for (int e = 0; e < 4; ++e)
        if ((bits >> e) & 1u) v[e] = -v[e];
}

// Normalised Walsh-Hadamard transform of 256 elements held 4 per lane.  Stages
// run in the order h = 1, 2, 4, ... 128 with (a, b) -> (a+b, a-b) on the pair
// (j, j+h), the same operations in the same order as the plain iterative form,
// so the result is bit-identical to it; the final 1/16 is exact.
__device__ __forceinline__ void fwht256(float (&v)[4], uint32_t lane) {
    float a = v[0], b = v[1], c = v[2], d = v[3];
    v[0] = a + b;  // h = 1
    v[1] = a - b;
    v[2] = c + d;
    v[3] = c - d;
    a = v[0], b = v[1], c = v[2], d = v[3];
    v[0] = a + c;  // h = 2
    v[2] = a - c;
    v[1] = b + d;
    v[3] = b - d;
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {  // h = 4m: partner lane differs in bit m
        const bool upper = lane & m;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float o = __shfl_xor(v[e], m);
            v[e] = upper ? o - v[e] : v[e] + o;
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] *= 0.0625f;
}

// buf[n_heads][head_dim] f32, in place; one wave per 256-block.
template <bool UNDO>
__global__ __launch_bounds__(64) void fwht_sign_kernel(float* __restrict__ buf) {
    float4* p = reinterpret_cast<float4*>(buf + (size_t)blockIdx.x * 256) + threadIdx.x;
    const float4 t = *p;
    float v[4] = {t.x, t.y, t.z, t.w};
    if (!UNDO) apply_signs(v, threadIdx.x);
    fwht256(v, threadIdx.x);
    if (UNDO) apply_signs(v, threadIdx.x);
    *p = make_float4(v[0], v[1], v[2], v[3]);
}

// Write-side encode: rotate, then per 256-block scale = amax/127,
// code = round_half_away(x/scale) as int8 (the Q8_0 rule, q8_0.rs:59-67).
// src [n_tokens][n_kv_heads][head_dim]; token t goes to slot (write_pos + t) % capacity.
__global__ __launch_bounds__(64) void tq_encode_kernel(const float* __restrict__ src, uint8_t* __restrict__ codes,
                                                       float* __restrict__ norms, uint32_t n_kv_heads,
                                                       uint32_t head_dim, uint32_t capacity, uint32_t write_pos) {
    const uint32_t npp = head_dim / 256;
    const uint32_t blk = blockIdx.x % npp, h = (blockIdx.x / npp) % n_kv_heads, t = blockIdx.x / (npp * n_kv_heads);
    const uint32_t lane = threadIdx.x;
    const float4 in = reinterpret_cast<const float4*>(src + ((size_t)t * n_kv_heads + h) * head_dim + 256 * blk)[lane];
    float v[4] = {in.x, in.y, in.z, in.w};
    apply_signs(v, lane);
    fwht256(v, lane);
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) amax = fmaxf(amax, __shfl_xor(amax, m));
    const float d = amax / 127.f;
    const float id = d != 0.f ? 1.f / d : 0.f;
    uint32_t packed = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float r = roundf(v[e] * id);
        packed |= ((uint32_t)(int)r & 0xffu) << (8 * e);
    }
    const size_t slot = ((size_t)write_pos + t) % capacity;
    const size_t row = (size_t)h * capacity + slot;
    reinterpret_cast<uint32_t*>(codes + row * head_dim + 256 * blk)[lane] = packed;
    if (lane == 0) norms[row * npp + blk] = d;
}

struct AttnArgs {
    const float* q;
    const uint8_t* k_codes;
    const float* k_norms;
    const uint8_t* v_codes;
    const float* v_norms;
    const float* lut;
    float* tmp;
    uint32_t num_heads, num_kv_heads, group;  // group = num_heads / num_kv_heads
    uint32_t kv_capacity, first, last;         // visible logical positions [first, last)
    uint32_t ring_start, n_splits, tiles_per_wave;
    float scale, softcap, lut_mul;             // lut_mul = 1 / (16 * scale_factor)
    uint32_t fuse_fwht_pre;
};

constexpr int HD = 256;           // head_dim handled by the attention kernels
constexpr int TMP_STRIDE = HD + 2;  // per (head, split): unnormalised output, running max, running sum

__device__ __forceinline__ float wave_max4(float v) {  // over the 4 lane groups that share lane%16
    v = fmaxf(v, __shfl_xor(v, 16));
    return fmaxf(v, __shfl_xor(v, 32));
}

// 8 int8 (two words) -> 8 bf16 as an MFMA fragment.
__device__ __forceinline__ bf16x8_t codes_to_frag(uint32_t w0, uint32_t w1) {
    uint4 o;
    o.x = (__float_as_uint(sbyte(w0, 0)) >> 16) | (__float_as_uint(sbyte(w0, 1)) & 0xffff0000u);
    o.y = (__float_as_uint(sbyte(w0, 2)) >> 16) | (__float_as_uint(sbyte(w0, 3)) & 0xffff0000u);
    o.z = (__float_as_uint(sbyte(w1, 0)) >> 16) | (__float_as_uint(sbyte(w1, 1)) & 0xffff0000u);
    o.w = (__float_as_uint(sbyte(w1, 2)) >> 16) | (__float_as_uint(sbyte(w1, 3)) & 0xffff0000u);
    return __builtin_bit_cast(bf16x8_t, o);
}

__device__ __forceinline__ uint32_t bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// Orders a wave's own LDS accesses for the compiler; the hardware serves one wave's LDS
// instructions in issue order, so data a lane wrote is there when another lane of the same wave
// reads it afterwards.
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One workgroup: one kv head, one chunk of <= 8 query heads of its group, one split of the sequence.
template <bool LUT>
__global__ __launch_bounds__(256) void tq_attn_split_kernel(AttnArgs a) {
    __shared__ float s_q[8][HD];          // the chunk's queries (rotated here when fuse_fwht_pre)
    __shared__ uint4 s_qh[8][33], s_ql[8][33];  // their bf16 hi / lo halves, 8 values per entry
    __shared__ float s_p[4][16][8];       // per wave: p * norm_v of the current tile, [position][head]
    __shared__ float s_alpha[4][8];       // per wave: rescale factor of the running output
    __shared__ float s_o[4][8][HD];       // per wave outputs for the final merge
    __shared__ float s_m[4][8], s_l[4][8];
    __shared__ float s_lut[LUT ? 256 : 1];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t n_chunks = (a.group + 7u) / 8u;
    const uint32_t kvh = blockIdx.y / n_chunks, hc = blockIdx.y % n_chunks;
    const uint32_t h0 = kvh * a.group + hc * 8u;
    const uint32_t nh = min(8u, a.group - hc * 8u);
    const uint32_t split = blockIdx.x;

    const uint32_t j = lane & 15u, g = lane >> 4;
    const uint32_t half = lane >> 5, dg = lane & 31u;
    const size_t head_base = (size_t)kvh * a.kv_capacity;
    const uint32_t split_first = a.first + split * (a.tiles_per_wave * 64u);

    // Operands of one 16-position tile of this wave.  K: lane (position j, quarter g) holds 64
    // contiguous code bytes; V: lane (half, dg) holds coordinates 8*dg..+7 of positions 2t + half.
    struct Tile {
        uint4 k0, k1, k2, k3;
        uint2 v[8];
        float kn, vn;
        bool ok;
    };
    // physical slot of logical position idx (ring buffer); ring_start, idx < kv_capacity
    auto slot_of = [&](uint32_t idx) -> uint32_t {
        const uint32_t s = a.ring_start + idx;
        return s >= a.kv_capacity ? s - a.kv_capacity : s;
    };
    auto load_tile = [&](uint32_t it, Tile& t) {
        const uint32_t tile0 = split_first + (it * 4u + wave) * 16u;  // first logical position of this wave's tile
        const uint32_t idx = tile0 + j;
        t.ok = idx < a.last;
        const uint32_t slot = slot_of(t.ok ? idx : a.first);  // positions past the end read a valid slot, weight 0
        const uint4* kp = reinterpret_cast<const uint4*>(a.k_codes + (head_base + slot) * HD + 64 * g);
        t.k0 = kp[0], t.k1 = kp[1], t.k2 = kp[2], t.k3 = kp[3];
        t.kn = a.k_norms[head_base + slot];
        t.vn = t.ok ? a.v_norms[head_base + slot] : 0.f;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const uint32_t vi = tile0 + 2 * q + half;
            const uint32_t vs = slot_of(vi < a.last ? vi : a.first);
            t.v[q] = *reinterpret_cast<const uint2*>(a.v_codes + (head_base + vs) * HD + 8 * dg);
        }
    };

    // s_p / s_alpha are private to the wave and LDS serves a wave's accesses in order, so the tile
    // loop needs no workgroup barrier.
    // The first tile is requested before anything else so that its trip from HBM overlaps the
    // staging of the queries; inside the loop the next tile is requested before the current one is
    // worked on.  With one or two waves per SIMD nothing else hides the latency.
    Tile cur, nxt;
    load_tile(0, cur);

    // ---- queries -> LDS (zero rows for absent heads), optional sign x FWHT ----
    for (uint32_t i = tid; i < 8 * HD / 4; i += 256) {
        const uint32_t h = i / (HD / 4), c = i % (HD / 4);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (h < nh) v = reinterpret_cast<const float4*>(a.q + (size_t)(h0 + h) * HD)[c];
        reinterpret_cast<float4*>(&s_q[h][0])[c] = v;
    }
    if constexpr (LUT) s_lut[tid] = a.lut[tid] * a.lut_mul;
    __syncthreads();
    if (a.fuse_fwht_pre) {
        for (uint32_t h = wave; h < 8; h += 4) {
            float4* p = reinterpret_cast<float4*>(&s_q[h][0]) + lane;
            const float4 t = *p;
            float v[4] = {t.x, t.y, t.z, t.w};
            apply_signs(v, lane);
            fwht256(v, lane);
            *p = make_float4(v[0], v[1], v[2], v[3]);
        }
        __syncthreads();
    }

    // ---- query fragments: lane (j = lane%16: head, g = lane/16) holds q[j][64g + 8kk + e] as an exact
    // bf16 hi + lo pair.  The split is done once per workgroup (thread = head tid/32, chunk tid%32 of 8
    // values) and every wave reads its fragments back; rows are padded to 33 chunks against bank conflicts.
    {
        const uint32_t h = tid >> 5, ch = tid & 31u;
        uint32_t hi[8], lo[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = s_q[h][8 * ch + e];
            hi[e] = bf16_rne(x);
            lo[e] = bf16_rne(x - bf16_bits_to_f32(hi[e]));
        }
        s_qh[h][ch] = make_uint4(hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16), hi[4] | (hi[5] << 16), hi[6] | (hi[7] << 16));
        s_ql[h][ch] = make_uint4(lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16), lo[4] | (lo[5] << 16), lo[6] | (lo[7] << 16));
    }
    __syncthreads();
    uint4 qhi[8], qlo[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
        qhi[kk] = j < 8 ? s_qh[j][8 * g + kk] : make_uint4(0, 0, 0, 0);
        qlo[kk] = j < 8 ? s_ql[j][8 * g + kk] : make_uint4(0, 0, 0, 0);
    }

    // ---- running state ----
    float m_run = -INFINITY, l_run = 0.f;  // for head j (identical in the 4 lane groups for m; partial for l)
    float acc[8][8];                        // [head][coordinate]: lane owns d = 8*(lane%32)..+7, positions of its half
#pragma unroll
    for (int h = 0; h < 8; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] = 0.f;


    for (uint32_t it = 0; it < a.tiles_per_wave; ++it) {
        if (it + 1 < a.tiles_per_wave) load_tile(it + 1, nxt);
        const uint4 k0 = cur.k0, k1 = cur.k1, k2 = cur.k2, k3 = cur.k3;
        const float kn = cur.kn, vn = cur.vn;
        const bool ok = cur.ok;
        uint2 vraw[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) vraw[q] = cur.v[q];
        // -------- scores on the matrix cores --------
        f32x4_t c = {0.f, 0.f, 0.f, 0.f};
        const uint32_t kw[16] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w,
                                 k2.x, k2.y, k2.z, k2.w, k3.x, k3.y, k3.z, k3.w};
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            if constexpr (!LUT) {
                const bf16x8_t af = codes_to_frag(kw[2 * kk], kw[2 * kk + 1]);
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8_t, qhi[kk]), c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8_t, qlo[kk]), c, 0, 0, 0);
            } else {
                // table values are arbitrary f32: hi+lo split of K as well, three products
                uint32_t hi[8], lo[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float x = s_lut[(kw[2 * kk + (e >> 2)] >> (8 * (e & 3))) & 0xffu];
                    hi[e] = bf16_rne(x);
                    lo[e] = bf16_rne(x - bf16_bits_to_f32(hi[e]));
                }
                const bf16x8_t ah = __builtin_bit_cast(bf16x8_t, make_uint4(hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16),
                                                                            hi[4] | (hi[5] << 16), hi[6] | (hi[7] << 16)));
                const bf16x8_t al = __builtin_bit_cast(bf16x8_t, make_uint4(lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16),
                                                                            lo[4] | (lo[5] << 16), lo[6] | (lo[7] << 16)));
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, __builtin_bit_cast(bf16x8_t, qhi[kk]), c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, __builtin_bit_cast(bf16x8_t, qlo[kk]), c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, __builtin_bit_cast(bf16x8_t, qhi[kk]), c, 0, 0, 0);
            }
        }
        // c[v] = dot(q[head j], K[position 4g+v]); norms / validity of those positions sit in lanes 4g+v
        float s[4], pv_norm[4];
        float tmax = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int src = 4 * g + v;
            const float nk = __shfl(kn, src);
            pv_norm[v] = __shfl(vn, src);
            const bool okv = __shfl((int)ok, src) != 0;
            float x = c[v] * (a.scale * nk);
            if (a.softcap != 0.f) x = a.softcap * tanhf(x / a.softcap);
            s[v] = okv ? x : -INFINITY;
            tmax = fmaxf(tmax, s[v]);
        }
        tmax = wave_max4(tmax);
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = m_new == -INFINITY ? 1.f : __expf(m_run - m_new);  // exp(-inf) = 0 on the first tile
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float p = s[v] == -INFINITY ? 0.f : __expf(s[v] - m_new);
            psum += p;
            if (j < 8) s_p[wave][4 * g + v][j] = p * pv_norm[v];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (g == 0 && j < 8) s_alpha[wave][j] = alpha;
        wave_lds_fence();  // the wave's own writes of s_p / s_alpha before its reads below
        // -------- P.V on the VALU --------
        {
            const float4 a0 = *reinterpret_cast<const float4*>(&s_alpha[wave][0]);
            const float4 a1 = *reinterpret_cast<const float4*>(&s_alpha[wave][4]);
            const float al[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
            for (int h = 0; h < 8; ++h)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[h][e] *= al[h];
        }
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float4 p0 = *reinterpret_cast<const float4*>(&s_p[wave][2 * t + half][0]);
            const float4 p1 = *reinterpret_cast<const float4*>(&s_p[wave][2 * t + half][4]);
            const float pp[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
            float vv[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t w = e < 4 ? vraw[t].x : vraw[t].y;
                if constexpr (LUT)
                    vv[e] = s_lut[(w >> (8 * (e & 3))) & 0xffu];
                else
                    vv[e] = sbyte(w, e & 3);
            }
#pragma unroll
            for (int h = 0; h < 8; ++h)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[h][e] = fmaf(pp[h], vv[e], acc[h][e]);
        }
        wave_lds_fence();  // reads of s_p / s_alpha before the next tile overwrites them
        cur = nxt;
    }

    // ---- merge the two position-halves of the wave, then the four waves, and emit the split's partial ----
#pragma unroll
    for (int h = 0; h < 8; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] += __shfl_xor(acc[h][e], 32);
    l_run += __shfl_xor(l_run, 16);
    l_run += __shfl_xor(l_run, 32);
    __syncthreads();
    if (half == 0) {
#pragma unroll
        for (int h = 0; h < 8; ++h) {
            float4* o = reinterpret_cast<float4*>(&s_o[wave][h][8 * dg]);
            o[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
            o[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
        }
    }
    if (g == 0 && j < 8) {
        s_m[wave][j] = m_run;
        s_l[wave][j] = l_run;
    }
    __syncthreads();
    for (uint32_t h = 0; h < nh; ++h) {
        const float m = fmaxf(fmaxf(s_m[0][h], s_m[1][h]), fmaxf(s_m[2][h], s_m[3][h]));
        float o = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float f = s_m[w][h] == -INFINITY ? 0.f : __expf(s_m[w][h] - m);
            o += f * s_o[w][h][tid];
            l += f * s_l[w][h];
        }
        float* out = a.tmp + ((size_t)(h0 + h) * a.n_splits + split) * TMP_STRIDE;
        out[tid] = o;
        if (tid == 0) {
            out[HD] = m;
            out[HD + 1] = l;
        }
    }
}

// out[h][d] = sum_s e^{m_s - m} O_s[d] / sum_s e^{m_s - m} l_s.  Grid (num_heads, 4): a workgroup
// owns 64 output coordinates of one head; its 4 waves take a quarter of the splits each, with
// the loads of 8 splits in flight at a time.
__global__ __launch_bounds__(256) void tq_attn_reduce_kernel(const float* __restrict__ tmp, float* __restrict__ out,
                                                             uint32_t n_splits) {
    __shared__ float s_w[256];  // e^{m_s - m}
    __shared__ float s_part[4][64];
    __shared__ float s_red[4];
    const uint32_t h = blockIdx.x, tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t d = blockIdx.y * 64u + lane;
    const float* base = tmp + (size_t)h * n_splits * TMP_STRIDE;
    // n_splits <= 256 = the workgroup size: one thread per split fetches its running maximum and sum
    float ms = -INFINITY, ls = 0.f;
    if (tid < n_splits) {
        ms = base[(size_t)tid * TMP_STRIDE + HD];
        ls = base[(size_t)tid * TMP_STRIDE + HD + 1];
    }
    float m = ms;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    const float w = ms == -INFINITY ? 0.f : __expf(ms - m);
    s_w[tid] = w;
    float lw = w * ls;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) lw += __shfl_xor(lw, o);
    __syncthreads();  // s_red read by everyone before it is reused; s_w visible
    if (lane == 0) s_red[wave] = lw;
    float o = 0.f;
    const uint32_t per = (n_splits + 3u) / 4u, s0 = wave * per, s1 = min(n_splits, s0 + per);
    for (uint32_t s = s0; s < s1; s += 8) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = s + i < s1 ? base[(size_t)(s + i) * TMP_STRIDE + d] : 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) o = fmaf(s + i < s1 ? s_w[s + i] : 0.f, v[i], o);
    }
    s_part[wave][lane] = o;
    __syncthreads();
    if (wave == 0) {
        const float l = s_red[0] + s_red[1] + s_red[2] + s_red[3];
        const float t = s_part[0][lane] + s_part[1][lane] + s_part[2][lane] + s_part[3][lane];
        out[(size_t)h * HD + d] = l > 0.f ? t / l : 0.f;
    }
}

}  // namespace

int launch_fwht_sign(hipStream_t s, float* buf, uint32_t n_heads, uint32_t head_dim, bool undo) {
    const unsigned blocks = n_heads * (head_dim / 256);
    if (undo)
        hipLaunchKernelGGL(fwht_sign_kernel<true>, dim3(blocks), dim3(64), 0, s, buf);
    else
        hipLaunchKernelGGL(fwht_sign_kernel<false>, dim3(blocks), dim3(64), 0, s, buf);
    return check_launch("fwht kernel launch");
}

int launch_tq_encode(hipStream_t s, const float* src, uint8_t* codes, float* norms, uint32_t n_tokens,
                     uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t write_pos) {
    const unsigned blocks = n_tokens * n_kv_heads * (head_dim / 256);
    hipLaunchKernelGGL(tq_encode_kernel, dim3(blocks), dim3(64), 0, s, src, codes, norms, n_kv_heads, head_dim, capacity,
                       write_pos);
    return check_launch("tq encode kernel launch");
}

// Visible logical range of a single query at the end of the sequence.
static void visible_range(const hq_tq_attn_params& p, uint32_t& first, uint32_t& last) {
    last = p.kv_seq_len;
    first = 0;
    if (p.mask_type == 2 && p.sliding_window > 0 && p.kv_seq_len > p.sliding_window) first = p.kv_seq_len - p.sliding_window;
}

uint32_t tq_attn_splits(uint32_t n_positions) {
    // 64 positions (one 16-position tile per wave) is the least a workgroup takes; at most 256 splits
    // (two workgroups per CU at two kv heads).
    const uint32_t groups = (n_positions + 63u) / 64u;
    return groups < 128u ? (groups ? groups : 1u) : 128u;
}

size_t tq_attn_tmp_bytes(uint32_t num_heads, uint32_t head_dim, uint32_t kv_seq_len) {
    (void)head_dim;
    return (size_t)num_heads * tq_attn_splits(kv_seq_len) * TMP_STRIDE * sizeof(float);
}

int launch_tq_attention(hipStream_t s, const float* q, const uint8_t* k_codes, const float* k_norms,
                        const uint8_t* v_codes, const float* v_norms, const float* lut, float* out, float* tmp,
                        const hq_tq_attn_params& p) {
    AttnArgs a{};
    a.q = q;
    a.k_codes = k_codes;
    a.k_norms = k_norms;
    a.v_codes = v_codes;
    a.v_norms = v_norms;
    a.lut = lut;
    a.tmp = tmp;
    a.num_heads = p.num_heads;
    a.num_kv_heads = p.num_kv_heads;
    a.group = p.num_heads / p.num_kv_heads;
    a.kv_capacity = p.kv_capacity;
    visible_range(p, a.first, a.last);
    a.ring_start = p.ring_start;
    // the split count is a function of kv_seq_len alone so that it matches the tmp size the caller was told
    a.n_splits = tq_attn_splits(p.kv_seq_len);
    const uint32_t n_pos = a.last - a.first;
    const uint32_t groups = (n_pos + 63u) / 64u;
    a.tiles_per_wave = (groups + a.n_splits - 1u) / a.n_splits;
    a.scale = p.scale;
    a.softcap = p.softcap;
    a.lut_mul = 1.f / (16.f * (p.head_dim == 512 ? p.scale_factor_d512 : 1.f));
    a.fuse_fwht_pre = p.fuse_fwht_pre;
    const dim3 grid(a.n_splits, p.num_kv_heads * ((a.group + 7u) / 8u));
    if (lut)
        hipLaunchKernelGGL(tq_attn_split_kernel<true>, grid, dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL(tq_attn_split_kernel<false>, grid, dim3(256), 0, s, a);
    if (int rc = check_launch("tq attention kernel launch")) return rc;
    hipLaunchKernelGGL(tq_attn_reduce_kernel, dim3(p.num_heads, HD / 64), dim3(256), 0, s, tmp, out, a.n_splits);
    return check_launch("tq attention reduce launch");
}

}  // namespace hq

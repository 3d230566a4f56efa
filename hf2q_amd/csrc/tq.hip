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

#include <type_traits>

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

// The same from literals instead of a table in memory, for kernels that have many loads in flight when they reach the
// rotation (a wave's loads return in order: a table fetch would wait for all of them).  Word w holds bytes 4w..4w+3.
__device__ __forceinline__ void apply_signs_inline(float (&v)[4], uint32_t lane) {
    const uint32_t w = lane >> 3;
    const uint32_t lo = w & 2u ? (w & 1u ? 0x1cea4589u : 0xd6247fb3u) : (w & 1u ? 0x0e58c26du : 0xf4913ba7u);
    const uint32_t hi = w & 2u ? (w & 1u ? 0xdb2c854au : 0xfe19c476u) : (w & 1u ? 0x3de10b97u : 0x52d8af63u);
    const uint32_t bits = (w & 4u ? hi : lo) >> (4u * (lane & 7u));  // elements 4l..4l+3
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
    // h = 4m: the partner lane differs in bit m; the upper lane's o - v is formed as (-v) + o, the same number
    auto stage = [&](auto mm) {
        constexpr int m = decltype(mm)::value;
        const uint32_t flip = lane & (uint32_t)m ? 0x80000000u : 0u;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = __uint_as_float(__float_as_uint(v[e]) ^ flip) + lane_xor<m>(v[e], lane);
    };
    stage(std::integral_constant<int, 1>{});
    stage(std::integral_constant<int, 2>{});
    stage(std::integral_constant<int, 4>{});
    stage(std::integral_constant<int, 8>{});
    stage(std::integral_constant<int, 16>{});
    stage(std::integral_constant<int, 32>{});
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
    amax = xor_max<1, 2, 4, 8, 16, 32>(amax, lane);
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

// Bulk dequantisation of positions start .. start + n_tokens - 1 of every kv head into
// dst[n_kv_heads][n_tokens][head_dim] f32; one wave per 256-block.  Linear codes: norm * int8(code);
// table codes: lut[code] * norm * lut_mul.  UNROT adds the inverse rotation of the block.
template <bool LUT, bool UNROT>
__global__ __launch_bounds__(64) void tq_dequant_kernel(const uint8_t* __restrict__ codes, const float* __restrict__ norms,
                                                        const float* __restrict__ lut, float lut_mul, float* __restrict__ dst,
                                                        uint32_t n_tokens, uint32_t head_dim, uint32_t capacity,
                                                        uint32_t start) {
    const uint32_t npp = head_dim / 256;
    const uint32_t blk = blockIdx.x % npp, t = (blockIdx.x / npp) % n_tokens, h = blockIdx.x / (npp * n_tokens);
    const uint32_t lane = threadIdx.x;
    const size_t row = (size_t)h * capacity + start + t;
    const uint32_t w = reinterpret_cast<const uint32_t*>(codes + row * head_dim + 256 * blk)[lane];
    const float norm = norms[row * npp + blk];
    float v[4];
    {
        // every product is rounded on its own: no fusion with the first additions of the rotation
#pragma clang fp contract(off)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (LUT)
                v[e] = lut[(w >> (8 * e)) & 0xffu] * norm * lut_mul;
            else
                v[e] = norm * sbyte(w, e);
        }
    }
    if constexpr (UNROT) {
        fwht256(v, lane);
        apply_signs(v, lane);
    }
    reinterpret_cast<float4*>(dst + ((size_t)h * n_tokens + t) * head_dim + 256 * blk)[lane] = make_float4(v[0], v[1], v[2], v[3]);
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
    return xor32_max(xor16_max(v));
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

// One workgroup: one kv head, one chunk of <= 8 query heads of its group, one split of the sequence
// and, for head_dim = NB * 256, one 256-block of the output (blockIdx.z): the scores run over all NB
// blocks of K, each with its own norm, the P.V product over the workgroup's block of V.
template <bool LUT, int NB>
__global__ __launch_bounds__(256) void tq_attn_split_kernel(AttnArgs a) {
    constexpr uint32_t ROW = NB * HD;        // bytes of a cache row, floats of a query
    __shared__ float s_q[8][ROW];         // the chunk's queries (rotated here when fuse_fwht_pre)
    __shared__ uint4 s_qh[NB][8][33], s_ql[NB][8][33];  // their bf16 hi / lo halves, 8 values per entry
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
    const uint32_t ob = NB > 1 ? blockIdx.z : 0u;

    const uint32_t j = lane & 15u, g = lane >> 4;
    const uint32_t half = lane >> 5, dg = lane & 31u;
    const size_t head_base = (size_t)kvh * a.kv_capacity;
    const uint32_t split_first = a.first + split * (a.tiles_per_wave * 64u);

    // Operands of one 16-position tile of this wave.  K: lane (position j, quarter g) holds 64
    // contiguous code bytes; V: lane (half, dg) holds coordinates 8*dg..+7 of positions 2t + half.
    struct Tile {
        uint4 k[NB][4];
        uint2 v[8];
        float kn[NB], vn;
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
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint4* kp = reinterpret_cast<const uint4*>(a.k_codes + (head_base + slot) * ROW + HD * b + 64 * g);
            t.k[b][0] = kp[0], t.k[b][1] = kp[1], t.k[b][2] = kp[2], t.k[b][3] = kp[3];
            t.kn[b] = a.k_norms[(head_base + slot) * NB + b];
        }
        t.vn = t.ok ? a.v_norms[(head_base + slot) * NB + ob] : 0.f;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const uint32_t vi = tile0 + 2 * q + half;
            const uint32_t vs = slot_of(vi < a.last ? vi : a.first);
            t.v[q] = *reinterpret_cast<const uint2*>(a.v_codes + (head_base + vs) * ROW + HD * ob + 8 * dg);
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
    for (uint32_t i = tid; i < 8 * ROW / 4; i += 256) {
        const uint32_t h = i / (ROW / 4), c = i % (ROW / 4);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (h < nh) v = reinterpret_cast<const float4*>(a.q + (size_t)(h0 + h) * ROW)[c];
        reinterpret_cast<float4*>(&s_q[h][0])[c] = v;
    }
    if constexpr (LUT) s_lut[tid] = a.lut[tid] * a.lut_mul;
    __syncthreads();
    if (a.fuse_fwht_pre) {
        for (uint32_t hb = wave; hb < 8 * NB; hb += 4) {  // every 256-block is rotated on its own
            float4* p = reinterpret_cast<float4*>(&s_q[hb / NB][HD * (hb % NB)]) + lane;
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
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const uint32_t h = tid >> 5, ch = tid & 31u;
        uint32_t hi[8], lo[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = s_q[h][HD * b + 8 * ch + e];
            hi[e] = bf16_rne(x);
            lo[e] = bf16_rne(x - bf16_bits_to_f32(hi[e]));
        }
        s_qh[b][h][ch] = make_uint4(hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16), hi[4] | (hi[5] << 16), hi[6] | (hi[7] << 16));
        s_ql[b][h][ch] = make_uint4(lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16), lo[4] | (lo[5] << 16), lo[6] | (lo[7] << 16));
    }
    __syncthreads();
    uint4 qhi[NB][8], qlo[NB][8];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            qhi[b][kk] = j < 8 ? s_qh[b][j][8 * g + kk] : make_uint4(0, 0, 0, 0);
            qlo[b][kk] = j < 8 ? s_ql[b][j][8 * g + kk] : make_uint4(0, 0, 0, 0);
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
        const float vn = cur.vn;
        const bool ok = cur.ok;
        uint2 vraw[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) vraw[q] = cur.v[q];
        // -------- scores on the matrix cores, one accumulator per 256-block (each has its own norm) --------
        f32x4_t c[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            c[b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            const uint32_t kw[16] = {cur.k[b][0].x, cur.k[b][0].y, cur.k[b][0].z, cur.k[b][0].w, cur.k[b][1].x, cur.k[b][1].y,
                                     cur.k[b][1].z, cur.k[b][1].w, cur.k[b][2].x, cur.k[b][2].y, cur.k[b][2].z, cur.k[b][2].w,
                                     cur.k[b][3].x, cur.k[b][3].y, cur.k[b][3].z, cur.k[b][3].w};
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                if constexpr (!LUT) {
                    const bf16x8_t af = codes_to_frag(kw[2 * kk], kw[2 * kk + 1]);
                    c[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8_t, qhi[b][kk]), c[b], 0, 0, 0);
                    c[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8_t, qlo[b][kk]), c[b], 0, 0, 0);
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
                    c[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, __builtin_bit_cast(bf16x8_t, qhi[b][kk]), c[b], 0, 0, 0);
                    c[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, __builtin_bit_cast(bf16x8_t, qlo[b][kk]), c[b], 0, 0, 0);
                    c[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, __builtin_bit_cast(bf16x8_t, qhi[b][kk]), c[b], 0, 0, 0);
                }
            }
        }
        // c[b][v] = dot(q[head j], K[position 4g+v]) over block b; norms / validity of those positions sit in lanes 4g+v
        float s[4], pv_norm[4];
        float tmax = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int src = 4 * g + v;
            pv_norm[v] = __shfl(vn, src);
            const bool okv = __shfl((int)ok, src) != 0;
            float x = 0.f;
#pragma unroll
            for (int b = 0; b < NB; ++b) x += c[b][v] * (a.scale * __shfl(cur.kn[b], src));
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
        for (int e = 0; e < 8; ++e) acc[h][e] = xor32_add(acc[h][e]);
    l_run = xor32_add(xor16_add(l_run));
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
        float* out = a.tmp + (((size_t)(h0 + h) * NB + ob) * a.n_splits + split) * TMP_STRIDE;
        out[tid] = o;
        if (tid == 0) {
            out[HD] = m;
            out[HD + 1] = l;
        }
    }
}

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;

// x of the lane eight places round its row of 16 (lanes j and j ^ 8 exchange).
__device__ __forceinline__ float row_xor8(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
}

// The same split for linear int8 codes with BOTH products on the f16 matrix cores.
//
// A code byte c becomes the f16 number 1152 + c without arithmetic: the byte with its sign bit flipped
// (c + 128, unsigned) placed under the f16 bit pattern of 1024 (0x6400 | u = 1024 + u, exact for
// u < 1024) by one v_perm_b32 against a register that holds the 0x64.  Odd elements of the reduction
// dimension take the opposite sign instead: the byte xor 0x7f is 127 - c, and under 0xe4 that is
// -(1024 + 127 - c) = c - 1151.  The constants are taken out again as a correction,
// q . (k + off) - sum(off_i q_i) for the scores and sum p (v + off) - sum(off_t p_t) for the output
// with off = +1152, -1151, +1152, ...; because the signs alternate, the constant part of the running
// sums stays near zero for smooth operands (a query with a large mean, evenly spread attention)
// instead of eating accumulator bits.
//
// Queries and weights enter as f16 hi + lo pairs (22 bits); products are exact in the MFMA and
// accumulate in fp32.  A chunk has at most 8 heads and the MFMA has 16 rows / columns, so the hi
// parts take rows / columns 0..7 and the lo parts 8..15 of the SAME instruction: lane j < 8 stands
// for the hi part of head j, lane j >= 8 for the lo part of head j - 8.
//
// f16 has a narrow exponent range, so both are normalised first: a head's query by the power of two
// that brings its largest magnitude into [512, 1024); the weights p * norm_v by their own running
// maximum, i.e. the kernel keeps two running maxima per head, m of the scores s (for the denominator
// l = sum e^(s - m)) and mv of s + ln norm_v (for the numerator, whose weights e^(s + ln norm_v - mv)
// * 2^14 then lie in [0, 2^14]).
//
// Tiles are 32 positions per wave.  Scores: two 16-position halves, MFMA 16x16x32 with the K codes
// as rows (lane (j, g): position j, 16 code bytes at 64i + 16g for i = 0..3) and the queries as
// columns, so lane (j, g) receives, after adding its partner j ^ 8, the scores of head j % 8 for
// positions 4g..4g+3 of each half: eight positions, which are exactly one k-group of the second
// product.  P.V: the weights of those eight positions are the lane's A fragment as they stand; the B
// fragment of output coordinate 16n + 4i + e is byte 4i + e of the eight V rows that lane (n, g)
// fetched for the same eight positions (16 bytes each), gathered two at a time by v_perm_b32.  16
// accumulators (i, e) of 4 registers hold row 4g + v (head (4g + v) % 8, hi or lo part), coordinate
// 16n + 4i + e.
//
// head_dim = NB * 256: blockIdx.z is the 256-block of the output this workgroup produces; the scores
// run over all NB blocks of K (each block has its own norm and its own query scaling), the P.V
// product over the workgroup's block of V.
//
// Cache offsets are 32-bit here: the launcher takes this kernel only below 4 GiB per code tensor.
template <bool RING, int NB>
__global__ __launch_bounds__(256) void tq_attn_split_f16_kernel(AttnArgs a) {
    constexpr uint32_t ROW = NB * HD;  // bytes of a cache row, floats of a query
    // s_o: per wave and row, the 256 coordinates in the order [i][j][e] (coordinate 16j + 4i + e), so
    // that a wave's stores are contiguous.  The fused rotation stages the queries in the same memory.
    __shared__ __align__(16) float s_o[4][16][HD];
    __shared__ uint4 s_qf[NB][16][33];             // scaled queries as f16, 8 values per entry; rows 0..7 hi, 8..15 lo
    __shared__ float s_corr[NB][16], s_unscale[NB][8];  // sum(off_i q_i) of a row; 2^e that undoes a head's scaling
    __shared__ float s_m[4][8], s_l[4][8];
    float(*s_q)[ROW] = reinterpret_cast<float(*)[ROW]>(&s_o[0][0][0]);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t n_chunks = (a.group + 7u) / 8u;
    const uint32_t kvh = blockIdx.y / n_chunks, hc = blockIdx.y % n_chunks;
    const uint32_t h0 = kvh * a.group + hc * 8u;
    const uint32_t nh = min(8u, a.group - hc * 8u);
    const uint32_t split = blockIdx.x;
    const uint32_t ob = NB > 1 ? blockIdx.z : 0u;
    const uint32_t j = lane & 15u, g = lane >> 4;
    const uint32_t head_base = kvh * a.kv_capacity;
    const uint32_t split_first = a.first + split * (a.tiles_per_wave * 64u);
    const uint32_t split_end = min(a.last, split_first + a.tiles_per_wave * 64u);
    const uint32_t n_iter = (a.tiles_per_wave + 1u) / 2u;  // 128 positions per workgroup and iteration

    struct Tile {
        uint4 k[NB][2][4];  // block, half, i: code bytes 64i + 16g .. +15 of position j
        uint4 v[8];         // positions 4g..4g+3 of half 0, then of half 1; coordinates 16j.. of block ob
        float kn[NB][2];    // norm_k of position j
        float vn[2];        // norm_v of block ob
        uint32_t keep[2];   // all ones, or 0 where the position is past the end (the norms then read as -1 and 0)
    };
    // Cache row of logical position idx; positions past the end of the split read a valid row and get
    // weight 0.  RING: rows start at ring_start and wrap (ring_start, idx < kv_capacity); otherwise
    // row = position.
    const uint32_t last_row = max(split_end, a.first + 1u) - 1u;
    auto row_of = [&](uint32_t idx) -> uint32_t {
        const uint32_t i = min(idx, last_row);
        if constexpr (!RING) return i;
        const uint32_t sl = a.ring_start + i;
        return sl >= a.kv_capacity ? sl - a.kv_capacity : sl;
    };
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto load_tile = [&](uint32_t it, Tile& t) {
        const uint32_t tile0 = split_first + (it * 4u + wave_u) * 32u;  // wave-uniform
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const uint32_t idx = tile0 + 16u * hf + j;
            const uint32_t keep = idx < split_end ? 0xffffffffu : 0u;
            const uint32_t row = head_base + row_of(idx);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint4* kp = reinterpret_cast<const uint4*>(a.k_codes + (row * ROW + (uint32_t)(HD * b) + 16u * g));
                t.k[b][hf][0] = kp[0], t.k[b][hf][1] = kp[4], t.k[b][hf][2] = kp[8], t.k[b][hf][3] = kp[12];
                // (no select here: it lets the compiler put the load under a branch, and it then waits for every
                // load in flight where the branch ends; the row is a valid one either way, attend() masks it)
                t.kn[b][hf] = a.k_norms[row * NB + b];
            }
            t.vn[hf] = a.v_norms[row * NB + ob];
            t.keep[hf] = keep;
        }
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const uint32_t vi = tile0 + (q < 4 ? 4u * g + q : 16u + 4u * g + (q - 4));
            const uint32_t row = head_base + row_of(vi);
            t.v[q] = *reinterpret_cast<const uint4*>(a.v_codes + (row * ROW + HD * ob + 16u * j));
        }
    };

    // The queries are requested first and the cache rows of the first iteration right after them: a wave's loads
    // return in the order they were issued, so the queries arrive ahead of the rows and their staging overlaps the
    // rows' trip from HBM.
    // Fused rotation: thread tid takes float4 chunks tid, tid + 256, ... of the 8 x ROW staged values; otherwise
    // head tid / 32, values 8 (tid % 32) .. +7 of every block.
    constexpr int QV = 2 * NB;
    float4 qv[QV];
#pragma unroll
    for (int r = 0; r < QV; ++r) {
        // No branch around the loads (the compiler would wait for them where the branches join, before the cache
        // rows are requested): heads past the chunk's last read that one and are zeroed by an AND.
        const uint32_t i = tid + 256u * r;
        const uint32_t hh = a.fuse_fwht_pre ? i / (ROW / 4) : tid >> 5;
        const uint32_t off = a.fuse_fwht_pre ? 4u * (i % (ROW / 4)) : (uint32_t)HD * (r >> 1) + 8u * (tid & 31u) + 4u * (r & 1);
        const uint4 raw = *reinterpret_cast<const uint4*>(a.q + (size_t)(h0 + min(hh, nh - 1u)) * ROW + off);
        const uint32_t keep = hh < nh ? 0xffffffffu : 0u;
        qv[r] = make_float4(__uint_as_float(raw.x & keep), __uint_as_float(raw.y & keep), __uint_as_float(raw.z & keep),
                            __uint_as_float(raw.w & keep));
    }
    // The second iteration's rows are requested after the queries have been staged: a wave stalls in the issue of a
    // load while the memory pipeline is full, and the first iteration's rows of the four waves fill it on their own
    // (80 KB per CU), so asking for more up front only delays the staging.
    Tile tile_a, tile_b;
    load_tile(0, tile_a);

    // ---- queries: every 256-block of a head scaled on its own and split into f16 hi + lo; thread =
    // head tid/32, chunk tid%32 of 8 values; rows are padded to 33 chunks against bank conflicts ----
    if (a.fuse_fwht_pre) {  // sign x FWHT of every block in LDS first
#pragma unroll
        for (int r = 0; r < QV; ++r) {
            const uint32_t i = tid + 256u * r;
            reinterpret_cast<float4*>(&s_q[i / (ROW / 4)][0])[i % (ROW / 4)] = qv[r];
        }
        __syncthreads();
        for (uint32_t hb = wave; hb < 8 * NB; hb += 4) {
            float4* p = reinterpret_cast<float4*>(&s_q[hb / NB][HD * (hb % NB)]) + lane;
            const float4 t = *p;
            float v[4] = {t.x, t.y, t.z, t.w};
            apply_signs_inline(v, lane);
            fwht256(v, lane);
            *p = make_float4(v[0], v[1], v[2], v[3]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const uint32_t h = tid >> 5, ch = tid & 31u;
        float4 v0 = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
        if (a.fuse_fwht_pre) {
            v0 = *reinterpret_cast<const float4*>(&s_q[h][HD * b + 8 * ch]), v1 = *reinterpret_cast<const float4*>(&s_q[h][HD * b + 8 * ch + 4]);
        } else {
            v0 = qv[2 * b], v1 = qv[2 * b + 1];
        }
        const float x[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
        float amax = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float ax = fabsf(x[e]);
            amax = ax <= 3.0e38f ? fmaxf(amax, ax) : amax;
        }
        amax = xor_max<16, 8, 4, 2, 1>(amax, lane);  // the 32 threads of a head
        // amax = f * 2^ex with f in [0.5, 1): scaling by 2^(10 - ex) brings it into [512, 1024)
        int sh = amax > 0.f ? 10 - __builtin_amdgcn_frexp_expf(amax) : 0;
        sh = sh < -100 ? -100 : sh > 100 ? 100 : sh;
        const float scl = __builtin_amdgcn_ldexpf(1.f, sh);
        uint32_t hi[8], lo[8];
        float sum_hi = 0.f, sum_lo = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float xs = x[e] * scl;
            const _Float16 fh = (_Float16)xs;
            const _Float16 fl = (_Float16)(xs - (float)fh);
            hi[e] = __builtin_bit_cast(unsigned short, fh);
            lo[e] = __builtin_bit_cast(unsigned short, fl);
            sum_hi += ((e & 1) ? -1151.f : 1152.f) * (float)fh;
            sum_lo += ((e & 1) ? -1151.f : 1152.f) * (float)fl;
        }
        sum_hi = xor_sum<16, 8, 4, 2, 1>(sum_hi, lane);
        sum_lo = xor_sum<16, 8, 4, 2, 1>(sum_lo, lane);
        s_qf[b][h][ch] = make_uint4(hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16), hi[4] | (hi[5] << 16), hi[6] | (hi[7] << 16));
        s_qf[b][8 + h][ch] = make_uint4(lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16), lo[4] | (lo[5] << 16), lo[6] | (lo[7] << 16));
        if (ch == 0) {
            s_corr[b][h] = sum_hi;
            s_corr[b][8 + h] = sum_lo;
            s_unscale[b][h] = __builtin_amdgcn_ldexpf(1.f, -sh);
        }
    }
    __syncthreads();  // also: s_q has been read, its memory (s_o) may be written again
    // MFMA step kk = 2i + w takes words 2w, 2w + 1 of K load i: coordinates 64i + 16g + 8w .. +7
    uint4 qf[NB][8];
    float corr[NB], sscale[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) qf[b][kk] = s_qf[b][j][8u * (kk >> 1) + 2u * g + (kk & 1)];
        corr[b] = s_corr[b][j];
        sscale[b] = s_unscale[b][j & 7u] * a.scale;
    }
    const bool lo_lane = j >= 8u;
    if (n_iter > 1) load_tile(1, tile_b);

    const uint32_t magic = 0x0000e464u;
    // two bytes of one word -> two f16 (1024 + byte, -(1024 + byte)): bytes 0, 1 with sel 0x05010400; 2, 3 with 0x05030402
    auto pair_of = [&](uint32_t w, uint32_t sel) -> uint32_t { return __builtin_amdgcn_perm(magic, w, sel); };
    // byte e of two words -> two f16 (1024 + byte of wa, -(1024 + byte of wb))
    auto gather2 = [&](uint32_t wa, uint32_t wb, int e) -> uint32_t {
        return __builtin_amdgcn_perm(wb, wa, 0x0c000c00u | (uint32_t)e | ((uint32_t)(4 + e) << 16)) | 0xe4006400u;
    };

    // of head j % 8: m, mv running maxima; l partial over this lane's positions; of row j: lp = sum(off_t p_t)
    // over the row's weights (hi or lo parts), partial likewise
    float m_run = -INFINITY, mv_run = -INFINITY, l_run = 0.f, lp_run = 0.f;
    f32x4_t acc[4][4];  // [i][e][v]: row 4g + v, coordinate 16j + 4i + e
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    constexpr float LOG2E = 1.4426950408889634f;

    auto attend = [&](const Tile& cur) {
        // positions past the end: norm_k = -1 (score -inf), norm_v = 0 (no weight)
        float kn[NB][2], vn[2];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
                kn[b][hf] = __uint_as_float((__float_as_uint(cur.kn[b][hf]) & cur.keep[hf]) | (0xbf800000u & ~cur.keep[hf]));
            vn[hf] = __uint_as_float(__float_as_uint(cur.vn[hf]) & cur.keep[hf]);
        }
        // -------- scores: two independent accumulation chains per half --------
        float s[8], lv[8];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            float dot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                f32x4_t c0 = {0.f, 0.f, 0.f, 0.f}, c1 = c0;
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) {
                    const uint4 kq = cur.k[b][hf][kk >> 1];
                    const uint32_t u0 = ((kk & 1) ? kq.z : kq.x) ^ 0x7f807f80u, u1 = ((kk & 1) ? kq.w : kq.y) ^ 0x7f807f80u;
                    const uint4 fr = make_uint4(pair_of(u0, 0x05010400u), pair_of(u0, 0x05030402u), pair_of(u1, 0x05010400u),
                                                pair_of(u1, 0x05030402u));
                    const f16x8_t af = __builtin_bit_cast(f16x8_t, fr);
                    if (kk & 1)
                        c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, __builtin_bit_cast(f16x8_t, qf[b][kk]), c1, 0, 0, 0);
                    else
                        c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, __builtin_bit_cast(f16x8_t, qf[b][kk]), c0, 0, 0, 0);
                }
                // c0 + c1 = (hi or lo part of q[head j % 8]) . (K[position 4g + v] + off) over block b; the
                // norms of those positions sit in lanes 4g + v
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float part = (c0[v] + c1[v]) - corr[b];
                    dot[v] += (part + row_xor8(part)) * (sscale[b] * __shfl(kn[b][hf], 4 * g + v));
                }
            }
            const float lvn_own = __log2f(vn[hf]);  // log 0 = -inf: no weight in the numerator
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int src = 4 * g + v;
                lv[4 * hf + v] = __shfl(lvn_own, src);
                s[4 * hf + v] = __shfl(kn[0][hf], src) >= 0.f ? dot[v] : -INFINITY;
            }
        }
        if (a.softcap != 0.f) {
            // cap * tanh(x / cap), tanh y = 1 - 2 / (e^2y + 1)
            const float inv = 2.f * LOG2E / a.softcap;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const float e2 = __builtin_amdgcn_exp2f(fminf(s[v] * inv, 80.f));
                s[v] = s[v] == -INFINITY ? -INFINITY : a.softcap * (1.f - __fdividef(2.f, e2 + 1.f));
            }
        }
        // the exponent domain is base 2 from here: s2 = s log2 e, t2 = s2 + log2 norm_v
        float t[8], smax = -INFINITY, tmax = -INFINITY;
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            s[v] *= LOG2E;
            t[v] = s[v] + lv[v];
            smax = fmaxf(smax, s[v]);
            tmax = fmaxf(tmax, t[v]);
        }
        smax = wave_max4(smax);
        tmax = wave_max4(tmax);
        const float m_new = fmaxf(m_run, smax), mv_new = fmaxf(mv_run, tmax);
        // nothing accumulated yet (running maximum -inf): any factor will do, 1 spares the rescaling below
        const float alpha = m_run == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m_run - m_new);
        const float alpha_v = mv_run == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(mv_run - mv_new);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;           // -inf - (-inf) would be NaN
        const float mv_use = (mv_new == -INFINITY ? 0.f : mv_new) - 14.f;  // weights scaled by 2^14
        float psum = 0.f, ppsum = 0.f;
        uint32_t pb[8];
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            psum += __builtin_amdgcn_exp2f(s[v] - m_use);
            const float pp = __builtin_amdgcn_exp2f(t[v] - mv_use);
            const _Float16 fh = (_Float16)pp;
            const _Float16 mine = (_Float16)(lo_lane ? pp - (float)fh : pp);
            pb[v] = __builtin_bit_cast(unsigned short, mine);
            ppsum += ((v & 1) ? -1151.f : 1152.f) * (float)mine;
        }
        l_run = l_run * alpha + psum;
        lp_run = lp_run * alpha_v + ppsum;
        m_run = m_new;
        mv_run = mv_new;
        const f16x8_t pf = __builtin_bit_cast(f16x8_t, make_uint4(pb[0] | (pb[1] << 16), pb[2] | (pb[3] << 16), pb[4] | (pb[5] << 16), pb[6] | (pb[7] << 16)));
        // -------- P.V --------
        if (__builtin_amdgcn_ballot_w64(alpha_v != 1.f) != 0) {  // rare once the maximum has settled
            float al[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) al[v] = __shfl(alpha_v, 4 * g + v);  // lane 4g + v stands for row 4g + v
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[i][e][v] *= al[v];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t vw[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const uint4 vq = cur.v[q];
                vw[q] = (i == 0 ? vq.x : i == 1 ? vq.y : i == 2 ? vq.z : vq.w) ^ ((q & 1) ? 0x7f7f7f7fu : 0x80808080u);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint4 fr = make_uint4(gather2(vw[0], vw[1], e), gather2(vw[2], vw[3], e), gather2(vw[4], vw[5], e),
                                            gather2(vw[6], vw[7], e));
                acc[i][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pf, __builtin_bit_cast(f16x8_t, fr), acc[i][e], 0, 0, 0);
            }
        }
    };
    // the two tiles swap roles from iteration to iteration (copying one into the other costs a move per register)
    for (uint32_t it = 0; it < n_iter; it += 2) {
        attend(tile_a);
        if (it + 2 < n_iter) load_tile(it + 2, tile_a);
        if (it + 1 < n_iter) {
            attend(tile_b);
            if (it + 3 < n_iter) load_tile(it + 3, tile_b);
        }
    }

    // ---- merge of the four waves.  First the maxima, so that every wave can bring its own numbers to
    // the workgroup's scale before they meet: O_row = (acc - lp) * 2^(mv - m_wg) / 2^14, l * 2^(m - m_wg).
    l_run = xor32_add(xor16_add(l_run));
    lp_run = xor32_add(xor16_add(lp_run));
    if (lane < 8u) s_m[wave][lane] = m_run;
    __syncthreads();
    const uint32_t hj = j & 7u;
    const float m_wg = fmaxf(fmaxf(s_m[0][hj], s_m[1][hj]), fmaxf(s_m[2][hj], s_m[3][hj]));
    const float fo_own = mv_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mv_run - m_wg - 14.f);
    if (lane < 8u) s_l[wave][lane] = m_run == -INFINITY ? 0.f : l_run * __builtin_amdgcn_exp2f(m_run - m_wg);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const float lpv = __shfl(lp_run, 4 * g + v), fo = __shfl(fo_own, 4 * g + v);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 o = make_float4((acc[i][0][v] - lpv) * fo, (acc[i][1][v] - lpv) * fo, (acc[i][2][v] - lpv) * fo,
                                         (acc[i][3][v] - lpv) * fo);
            *reinterpret_cast<float4*>(&s_o[wave][4 * g + v][64 * i + 4 * j]) = o;
        }
    }
    __syncthreads();
    {
        // thread = head tid / 32, eight consecutive stored values: i = c8 / 8, j = 2 (c8 % 8) and the next, e = 0..3
        const uint32_t h = tid >> 5, c8 = tid & 31u;
        if (h < nh) {
            float4 o0 = make_float4(0.f, 0.f, 0.f, 0.f), o1 = o0;
#pragma unroll
            for (int w = 0; w < 4; ++w)
#pragma unroll
                for (int part = 0; part < 2; ++part) {
                    const float4 x0 = *reinterpret_cast<const float4*>(&s_o[w][h + 8 * part][8 * c8]);
                    const float4 x1 = *reinterpret_cast<const float4*>(&s_o[w][h + 8 * part][8 * c8 + 4]);
                    o0.x += x0.x, o0.y += x0.y, o0.z += x0.z, o0.w += x0.w;
                    o1.x += x1.x, o1.y += x1.y, o1.z += x1.z, o1.w += x1.w;
                }
            float* out = a.tmp + (((size_t)(h0 + h) * NB + ob) * a.n_splits + split) * TMP_STRIDE;
            const uint32_t ci = c8 >> 3, cj = 2u * (c8 & 7u);
            float* o_at = out + 16u * cj + 4u * ci;  // TMP_STRIDE is even, not a multiple of 4: 8-byte stores
            reinterpret_cast<float2*>(o_at)[0] = make_float2(o0.x, o0.y);
            reinterpret_cast<float2*>(o_at)[1] = make_float2(o0.z, o0.w);
            reinterpret_cast<float2*>(o_at + 16)[0] = make_float2(o1.x, o1.y);
            reinterpret_cast<float2*>(o_at + 16)[1] = make_float2(o1.z, o1.w);
            if (c8 == 0) {
                const float m = fmaxf(fmaxf(s_m[0][h], s_m[1][h]), fmaxf(s_m[2][h], s_m[3][h]));
                out[HD] = m * (1.f / LOG2E);  // the merge kernel works with natural exponents
                out[HD + 1] = (s_l[0][h] + s_l[1][h]) + (s_l[2][h] + s_l[3][h]);
            }
        }
    }
}

// out[h][d] = sum_s e^{m_s - m} O_s[d] / sum_s e^{m_s - m} l_s, optionally followed by the inverse
// rotation (FWHT, then signs) of the head's 256 coordinates.  One workgroup of 16 waves per head: a
// wave takes a sixteenth of the splits, a lane four consecutive coordinates, so that at up to 128
// splits every load of the kernel is in flight at once; wave 0 adds the partial sums, divides and
// rotates.
constexpr int MERGE_WAVES = 16;
template <bool UNDO>
__global__ __launch_bounds__(64 * MERGE_WAVES) void tq_attn_merge_kernel(const float* __restrict__ tmp, float* __restrict__ out,
                                                                         uint32_t n_splits) {
    __shared__ float s_w[256];  // e^{m_s - m}
    __shared__ __align__(16) float s_part[MERGE_WAVES][HD];
    __shared__ float s_red[MERGE_WAVES];
    const uint32_t h = blockIdx.x, tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const float* base = tmp + (size_t)h * n_splits * TMP_STRIDE;
    const uint32_t per = (n_splits + MERGE_WAVES - 1u) / MERGE_WAVES, s0 = min(n_splits, wave * per), s1 = min(n_splits, s0 + per);
    constexpr int CH = 8;
    // rows of tmp are 8-byte aligned (TMP_STRIDE is even): two float2 per lane and split
    auto fetch = [&](uint32_t s, float2 (&v)[CH][2]) {
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            const float2* row = reinterpret_cast<const float2*>(base + (size_t)min(s + i, n_splits - 1u) * TMP_STRIDE) + 2u * lane;
            v[i][0] = row[0];
            v[i][1] = row[1];
        }
    };
    float2 v[CH][2];
    fetch(s0, v);  // on their way while the weights are worked out
    // n_splits <= 256: one thread per split fetches its running maximum and sum
    float ms = -INFINITY, ls = 0.f;
    if (tid < n_splits) {
        ms = base[(size_t)tid * TMP_STRIDE + HD];
        ls = base[(size_t)tid * TMP_STRIDE + HD + 1];
    }
    float m = ms;
    m = xor_max<32, 16, 8, 4, 2, 1>(m, lane);
    if (lane == 0) s_red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));  // splits live in the first 256 threads
    const float w = ms == -INFINITY ? 0.f : __expf(ms - m);
    if (tid < 256u) s_w[tid] = w;
    float lw = w * ls;
    lw = xor_sum<32, 16, 8, 4, 2, 1>(lw, lane);
    __syncthreads();  // s_red read by everyone before it is reused; s_w visible
    if (lane == 0) s_red[wave] = lw;
    float o[4] = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t s = s0; s < s1; s += CH) {
        if (s != s0) fetch(s, v);
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            const float ws = s + i < s1 ? s_w[s + i] : 0.f;
            o[0] = fmaf(ws, v[i][0].x, o[0]);
            o[1] = fmaf(ws, v[i][0].y, o[1]);
            o[2] = fmaf(ws, v[i][1].x, o[2]);
            o[3] = fmaf(ws, v[i][1].y, o[3]);
        }
    }
    *reinterpret_cast<float4*>(&s_part[wave][4 * lane]) = make_float4(o[0], o[1], o[2], o[3]);
    __syncthreads();
    if (wave == 0) {
        const float l = (s_red[0] + s_red[1]) + (s_red[2] + s_red[3]);
        float r[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w2 = 0; w2 < MERGE_WAVES; ++w2) {
            const float4 t = *reinterpret_cast<const float4*>(&s_part[w2][4 * lane]);
            r[0] += t.x, r[1] += t.y, r[2] += t.z, r[3] += t.w;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = l > 0.f ? r[e] / l : 0.f;
        if constexpr (UNDO) {
            fwht256(r, lane);
            apply_signs(r, lane);
        }
        reinterpret_cast<float4*>(out + (size_t)h * HD)[lane] = make_float4(r[0], r[1], r[2], r[3]);
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

int launch_tq_dequantize(hipStream_t s, const uint8_t* codes, const float* norms, const float* lut, float* dst,
                         uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t start_pos, uint32_t n_tokens,
                         float scale_factor_d512, bool unrotate) {
    const unsigned blocks = n_kv_heads * n_tokens * (head_dim / 256);
    const float lut_mul = 1.f / (16.f * (head_dim == 512 ? scale_factor_d512 : 1.f));
    void (*kern)(const uint8_t*, const float*, const float*, float, float*, uint32_t, uint32_t, uint32_t, uint32_t) =
        lut ? (unrotate ? tq_dequant_kernel<true, true> : tq_dequant_kernel<true, false>)
            : (unrotate ? tq_dequant_kernel<false, true> : tq_dequant_kernel<false, false>);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(64), 0, s, codes, norms, lut, lut_mul, dst, n_tokens, head_dim, capacity,
                       start_pos);
    return check_launch("tq dequantize kernel launch");
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
    return (size_t)num_heads * (head_dim / HD) * tq_attn_splits(kv_seq_len) * TMP_STRIDE * sizeof(float);
}

int launch_tq_attention(hipStream_t s, const float* q, const uint8_t* k_codes, const float* k_norms,
                        const uint8_t* v_codes, const float* v_norms, const float* lut, float* out, float* tmp,
                        const hq_tq_attn_params& p, bool undo_rotation) {
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
    const uint32_t nb = p.head_dim / HD;
    const dim3 grid(a.n_splits, p.num_kv_heads * ((a.group + 7u) / 8u), nb);
    // the f16 kernel indexes the code tensors with 32-bit byte offsets
    const bool small = (uint64_t)p.num_kv_heads * p.kv_capacity * p.head_dim <= 0xffffffffull;
    const bool ring = p.ring_start != 0;
    void (*kern)(AttnArgs);
    if (nb == 1)
        kern = lut ? tq_attn_split_kernel<true, 1>
               : !small ? tq_attn_split_kernel<false, 1>
               : ring ? tq_attn_split_f16_kernel<true, 1> : tq_attn_split_f16_kernel<false, 1>;
    else
        kern = lut ? tq_attn_split_kernel<true, 2>
               : !small ? tq_attn_split_kernel<false, 2>
               : ring ? tq_attn_split_f16_kernel<true, 2> : tq_attn_split_f16_kernel<false, 2>;
    hipLaunchKernelGGL(kern, grid, dim3(256), 0, s, a);
    if (int rc = check_launch("tq attention kernel launch")) return rc;
    // every 256-block of a head is a row of its own in tmp and in out
    if (undo_rotation)
        hipLaunchKernelGGL(tq_attn_merge_kernel<true>, dim3(p.num_heads * nb), dim3(64 * MERGE_WAVES), 0, s, tmp, out, a.n_splits);
    else
        hipLaunchKernelGGL(tq_attn_merge_kernel<false>, dim3(p.num_heads * nb), dim3(64 * MERGE_WAVES), 0, s, tmp, out, a.n_splits);
    return check_launch("tq attention merge launch");
}

}  // namespace hq

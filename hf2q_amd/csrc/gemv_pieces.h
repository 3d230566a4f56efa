// Device helpers shared by the dequant-fused GEMV kernels (gemv.hip) and the fused MoE decode layer (moe_fused.hip):
// the per-lane piece of a GGML block row, its dot product with staged activations, activation staging into LDS, and
// the DPP reductions.  Everything here is __device__ __forceinline__ or constexpr; each translation unit gets its own
// copy (anonymous namespace).
#pragma once

#include "hq_internal.h"

namespace hq {
namespace {

constexpr uint32_t M4 = 0x000f000fu, M2 = 0x00300030u, M1 = 0x10101010u, MAGIC = 0x43004300u;
constexpr uint32_t N4 = 0x0f0f0f0fu, N2 = 0x30303030u;  // the Q6_K kernels work on four bytes at a time
// Pseudo types of the flat walk (gemv_walk.h), not GGML ids: kX2 + t is a lane's piece of type t twice over -- two
// consecutive blocks (Q8_0, Q4_0), or the lane's quarter of two consecutive super-blocks (K-quants) -- fetched together,
// so that a wave has twice the bytes of a window in flight: one piece per lane is 1.2 .. 3.4 KB per wave, less than the
// memory system needs from sixteen waves per CU to run at its rate.
constexpr int kX2 = 1000;
template <int TYPE>
constexpr bool kIsX2 = TYPE >= kX2;
template <int TYPE>
constexpr int kBaseType = TYPE >= kX2 ? TYPE - kX2 : TYPE;
constexpr int HQ_Q8_0_X2 = kX2 + HQ_Q8_0;
// Types whose block is one lane's piece of 32 weights (the K-quants give a lane 64 of a super-block's 256).
template <int TYPE>
constexpr bool kBlock32 = TYPE == HQ_Q8_0 || TYPE == HQ_Q4_0;
template <int TYPE>
constexpr uint32_t kBlockBytes1 = TYPE == HQ_Q4_K ? Q4K_BYTES : TYPE == HQ_Q5_K ? Q5K_BYTES : TYPE == HQ_Q6_K ? Q6K_BYTES
                                  : TYPE == HQ_Q4_0 ? Q4_0_BYTES : Q8_0_BYTES;
template <int TYPE>
constexpr uint32_t kBlockBytes = kIsX2<TYPE> ? 2u * kBlockBytes1<kBaseType<TYPE>> : kBlockBytes1<TYPE>;
template <int TYPE>
struct Lane {  // weights per lane and step
    static constexpr int kElems = kBlock32<TYPE> ? 32 : 64;
};

// Per-lane fetch of one piece of row data.  The primary template is the doubled piece of a base type (its
// specialisations below): the same quarter of the next super-block, or the next block.
template <int TYPE>
struct Piece {
    static_assert(kIsX2<TYPE>, "base types have their own pieces");
    Piece<kBaseType<TYPE>> a, b;
    __device__ __forceinline__ void load(const uint8_t* blk, int c) {
        a.load(blk, c);
        b.load(blk + kBlockBytes1<kBaseType<TYPE>>, c);
    }
};

template <>
struct Piece<HQ_Q4_K> {
    uint4 hdr, q0, q1;
    __device__ __forceinline__ void load(const uint8_t* blk, int c) {
        hdr = *reinterpret_cast<const uint4*>(blk);
        q0 = *reinterpret_cast<const uint4*>(blk + 16 + 32 * c);
        q1 = *reinterpret_cast<const uint4*>(blk + 32 + 32 * c);
    }
};
template <>
struct Piece<HQ_Q6_K> {
    uint4 qa, qb, qh;
    uint2 sc;
    uint32_t d;  // the block's last four bytes: two scale bytes, then d (f16) in the upper half
    __device__ __forceinline__ void load(const uint8_t* blk, int c) {
        const int h = c >> 1, lr = c & 1;
        qa = ld16_unaligned(blk + 64 * h + 16 * lr);
        qb = ld16_unaligned(blk + 64 * h + 32 + 16 * lr);
        qh = ld16_unaligned(blk + 128 + 32 * h + 16 * lr);
        sc = ld8_unaligned(blk + 192 + 8 * h);
        // (a full word and a shift where d is used, not a half-word load: the masking that the compiler attaches to a
        // half-word load sits where the load is issued, and in a pipelined loop its wait drains every fetch in flight)
        d = ld4_unaligned(blk + 206);
    }
};
template <>
struct Piece<HQ_Q5_K> {  // header, the chunk's 32 nibble bytes, all 32 high-bit bytes (bits 2c, 2c+1 are this chunk's)
    uint4 hdr, q0, q1, h0, h1;
    __device__ __forceinline__ void load(const uint8_t* blk, int c) {
        hdr = *reinterpret_cast<const uint4*>(blk);
        h0 = *reinterpret_cast<const uint4*>(blk + 16);
        h1 = *reinterpret_cast<const uint4*>(blk + 32);
        q0 = *reinterpret_cast<const uint4*>(blk + 48 + 32 * c);
        q1 = *reinterpret_cast<const uint4*>(blk + 64 + 32 * c);
    }
};
template <>
struct Piece<HQ_Q4_0> {
    uint4 q;
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t* blk, int) {
        d = ld2(blk);
        q = ld16_unaligned(blk + 2);
    }
};
template <>
struct Piece<HQ_Q8_0> {
    uint4 q0, q1;
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t* blk, int) {
        d = ld2(blk);
        q0 = ld16_unaligned(blk + 2);
        q1 = ld16_unaligned(blk + 18);
    }
};

template <>
struct Piece<HQ_Q8_0_X2> {  // [d0][32 int8][d1][32 int8] as seventeen words
    uint4 a, b, c, e;
    uint32_t t;
    __device__ __forceinline__ void load(const uint8_t* blk, int) {
        a = ld16_unaligned(blk);
        b = ld16_unaligned(blk + 16);
        c = ld16_unaligned(blk + 32);
        e = ld16_unaligned(blk + 48);
        t = ld4_unaligned(blk + 64);
    }
};

__device__ __forceinline__ uint32_t word(const uint4& v, int i) {
    return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
}

// ---- paired-bf16 activations (xp: 32 words = 64 activations of this lane, sx: 4 run sums) ----
__device__ __forceinline__ float dot_pair(const Piece<HQ_Q4_K>& p, int c, const uint32_t* xp, const float* sx,
                                          uint32_t m4, uint32_t, uint32_t magic) {
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t w = j < 4 ? word(p.q0, j) : word(p.q1, j - 4);
        lo = dot2_bf16((w & m4) | magic, xp[2 * j], lo);
        lo = dot2_bf16(((w >> 8) & m4) | magic, xp[2 * j + 1], lo);
        hi = dot2_bf16(((w >> 4) & m4) | magic, xp[16 + 2 * j], hi);
        hi = dot2_bf16(((w >> 12) & m4) | magic, xp[16 + 2 * j + 1], hi);
    }
    uint32_t sc0, sc1, m0, m1;
    q4k_scales(p.hdr.y, p.hdr.z, p.hdr.w, c, sc0, sc1, m0, m1);
    const float d = f16_bits_to_f32(p.hdr.x & 0xffffu), dmin = f16_bits_to_f32(p.hdr.x >> 16);
    const float d0 = d * (float)sc0, d1 = d * (float)sc1;
    const float sl = sx[0] + sx[1], sh = sx[2] + sx[3];
    float acc = d0 * lo - (128.f * d0 + dmin * (float)m0) * sl;
    acc += d1 * hi - (128.f * d1 + dmin * (float)m1) * sh;
    return acc;
}

// Q5_K: the fifth bit of element j of sub-blocks 2c / 2c+1 is bit 2c / 2c+1 of high-bit byte j.  Four 5-bit values at a
// time as the bytes of one word (m1 = 0x10101010 arrives in the second mask register), then two byte permutes put bytes
// (0, 2) and (1, 3) under the high byte 0x43 of `magic`: bf16 128 + q with q in 0..31, the pair order of the staged
// activations.
__device__ __forceinline__ float dot_pair(const Piece<HQ_Q5_K>& p, int c, const uint32_t* xp, const float* sx,
                                          uint32_t, uint32_t m1, uint32_t magic) {
    float lo = 0.f, hi = 0.f;
    constexpr uint32_t SEL02 = 0x07020500u, SEL13 = 0x07030501u;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t w = j < 4 ? word(p.q0, j) : word(p.q1, j - 4);
        const uint32_t hs = (j < 4 ? word(p.h0, j) : word(p.h1, j - 4)) >> (2 * c);
        const uint32_t ql = and_or(hs << 4, m1, w & 0x0f0f0f0fu);
        const uint32_t qh = and_or(hs << 3, m1, (w >> 4) & 0x0f0f0f0fu);
        lo = dot2_bf16(__builtin_amdgcn_perm(magic, ql, SEL02), xp[2 * j], lo);
        lo = dot2_bf16(__builtin_amdgcn_perm(magic, ql, SEL13), xp[2 * j + 1], lo);
        hi = dot2_bf16(__builtin_amdgcn_perm(magic, qh, SEL02), xp[16 + 2 * j], hi);
        hi = dot2_bf16(__builtin_amdgcn_perm(magic, qh, SEL13), xp[16 + 2 * j + 1], hi);
    }
    uint32_t sc0, sc1, m0, mn1;
    q4k_scales(p.hdr.y, p.hdr.z, p.hdr.w, c, sc0, sc1, m0, mn1);
    const float d = f16_bits_to_f32(p.hdr.x & 0xffffu), dmin = f16_bits_to_f32(p.hdr.x >> 16);
    const float d0 = d * (float)sc0, d1 = d * (float)sc1;
    const float sl = sx[0] + sx[1], sh = sx[2] + sx[3];
    float acc = d0 * lo - (128.f * d0 + dmin * (float)m0) * sl;
    acc += d1 * hi - (128.f * d1 + dmin * (float)mn1) * sh;
    return acc;
}

// Q6_K: the four runs' sums r[i] (of (q + off) * x) and activation sums sx[i] combined with the runs' scales (bytes lr,
// lr + 2, lr + 4, lr + 6 of this half's eight) and d.  Every operation is written out and nothing else is fused: the
// kernels that share this get the same bits whatever surrounds the call.
__device__ __forceinline__ float q6k_combine(const Piece<HQ_Q6_K>& p, int c, float off, float r0, float r1, float r2, float r3,
                                             const float* sx) {
#pragma clang fp contract(off)
    const int lr = c & 1;
    const uint32_t s01 = p.sc.x >> (8 * lr), s23 = p.sc.y >> (8 * lr);
    const float d = f16_bits_to_f32(p.d >> 16);
    float acc = (float)(int)(int8_t)(s01 & 0xff) * fmaf(-off, sx[0], r0);
    acc = fmaf((float)(int)(int8_t)((s01 >> 16) & 0xff), fmaf(-off, sx[1], r1), acc);
    acc = fmaf((float)(int)(int8_t)(s23 & 0xff), fmaf(-off, sx[2], r2), acc);
    acc = fmaf((float)(int)(int8_t)((s23 >> 16) & 0xff), fmaf(-off, sx[3], r3), acc);
    return d * acc;
}

// Q6_K: four 6-bit values at a time as the bytes of one word (nibbles of ql, two-bit fields of qh; n4 = 0x0f0f0f0f and
// n2 = 0x30303030 arrive in the mask registers), then two byte permutes put bytes (0, 2) and (1, 3) under the high
// byte 0x43 of `magic`: bf16 128 + q, the pair order of the staged activations.
__device__ __forceinline__ float dot_pair(const Piece<HQ_Q6_K>& p, int c, const uint32_t* xp, const float* sx,
                                          uint32_t n4, uint32_t n2, uint32_t magic) {
    float r0 = 0.f, r1 = 0.f, r2 = 0.f, r3 = 0.f;
    constexpr uint32_t SEL02 = 0x07020500u, SEL13 = 0x07030501u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t a = word(p.qa, j), b = word(p.qb, j), v = word(p.qh, j);
        const uint32_t q0 = and_or(v << 4, n2, a & n4);
        const uint32_t q1 = and_or(v << 2, n2, b & n4);
        const uint32_t q2 = and_or(v, n2, (a >> 4) & n4);
        const uint32_t q3 = and_or(v >> 2, n2, (b >> 4) & n4);
        r0 = dot2_bf16(__builtin_amdgcn_perm(magic, q0, SEL02), xp[2 * j], r0);
        r0 = dot2_bf16(__builtin_amdgcn_perm(magic, q0, SEL13), xp[2 * j + 1], r0);
        r1 = dot2_bf16(__builtin_amdgcn_perm(magic, q1, SEL02), xp[8 + 2 * j], r1);
        r1 = dot2_bf16(__builtin_amdgcn_perm(magic, q1, SEL13), xp[8 + 2 * j + 1], r1);
        r2 = dot2_bf16(__builtin_amdgcn_perm(magic, q2, SEL02), xp[16 + 2 * j], r2);
        r2 = dot2_bf16(__builtin_amdgcn_perm(magic, q2, SEL13), xp[16 + 2 * j + 1], r2);
        r3 = dot2_bf16(__builtin_amdgcn_perm(magic, q3, SEL02), xp[24 + 2 * j], r3);
        r3 = dot2_bf16(__builtin_amdgcn_perm(magic, q3, SEL13), xp[24 + 2 * j + 1], r3);
    }
    // values hold 128 + q with q in 0..63 and the format's own -32, hence the 160
    return q6k_combine(p, c, 160.f, r0, r1, r2, r3, sx);
}

// Q4_0: y = d * (q - 8); low nibbles are elements 0..15 of the block, high nibbles 16..31; values hold 128 + q.
// xp: 16 paired words = the block's 32 activations, sx: the sums of its two runs of sixteen.
__device__ __forceinline__ float dot_pair(const Piece<HQ_Q4_0>& p, int, const uint32_t* xp, const float* sx, uint32_t m4,
                                          uint32_t, uint32_t magic) {
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t w = word(p.q, j);
        lo = dot2_bf16((w & m4) | magic, xp[2 * j], lo);
        lo = dot2_bf16(((w >> 8) & m4) | magic, xp[2 * j + 1], lo);
        hi = dot2_bf16(((w >> 4) & m4) | magic, xp[8 + 2 * j], hi);
        hi = dot2_bf16(((w >> 12) & m4) | magic, xp[8 + 2 * j + 1], hi);
    }
    return f16_bits_to_f32(p.d) * ((lo + hi) - 136.f * (sx[0] + sx[1]));
}
// (Q8_0 has no paired form: 128 + q needs eight mantissa bits beside the leading one, bf16 has seven.)
__device__ __forceinline__ float dot_pair(const Piece<HQ_Q8_0>&, int, const uint32_t*, const float*, uint32_t, uint32_t, uint32_t) {
    return 0.f;
}

// ---- f32 activations (xf: this lane's 64 (32 for Q8_0) activations, sx: run sums) ----
__device__ __forceinline__ float dot4(uint32_t q, const float* x, float acc) {
    // q is a word of four masked bytes; hidden from the optimiser, which would otherwise fold the mask into a bit-field
    // extract per byte (v_bfe + v_cvt_f32_ubyte0) where v_cvt_f32_ubyte0..3 of the one masked word do
    asm("" : "+v"(q));
    acc = fmaf(ubyte0(q), x[0], acc);
    acc = fmaf(ubyte1(q), x[1], acc);
    acc = fmaf(ubyte2(q), x[2], acc);
    return fmaf(ubyte3(q), x[3], acc);
}

__device__ __forceinline__ float dot_f32(const Piece<HQ_Q4_K>& p, int c, const float* xf, const float* sx) {
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t w = j < 4 ? word(p.q0, j) : word(p.q1, j - 4);
        lo = dot4(w & 0x0f0f0f0fu, xf + 4 * j, lo);
        hi = dot4((w >> 4) & 0x0f0f0f0fu, xf + 32 + 4 * j, hi);
    }
    uint32_t sc0, sc1, m0, m1;
    q4k_scales(p.hdr.y, p.hdr.z, p.hdr.w, c, sc0, sc1, m0, m1);
    const float d = f16_bits_to_f32(p.hdr.x & 0xffffu), dmin = f16_bits_to_f32(p.hdr.x >> 16);
    float acc = d * (float)sc0 * lo - dmin * (float)m0 * (sx[0] + sx[1]);
    acc += d * (float)sc1 * hi - dmin * (float)m1 * (sx[2] + sx[3]);
    return acc;
}

__device__ __forceinline__ float dot_f32(const Piece<HQ_Q6_K>& p, int c, const float* xf, const float* sx) {
    float r0 = 0.f, r1 = 0.f, r2 = 0.f, r3 = 0.f;
    constexpr uint32_t N4 = 0x0f0f0f0fu, N2 = 0x30303030u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t a = word(p.qa, j), b = word(p.qb, j), v = word(p.qh, j);
        r0 = dot4((a & N4) | ((v << 4) & N2), xf + 4 * j, r0);
        r1 = dot4((b & N4) | ((v << 2) & N2), xf + 16 + 4 * j, r1);
        r2 = dot4(((a >> 4) & N4) | (v & N2), xf + 32 + 4 * j, r2);
        r3 = dot4(((b >> 4) & N4) | ((v >> 2) & N2), xf + 48 + 4 * j, r3);
    }
    return q6k_combine(p, c, 32.f, r0, r1, r2, r3, sx);
}

__device__ __forceinline__ float dot_f32(const Piece<HQ_Q5_K>& p, int c, const float* xf, const float* sx) {
    float lo = 0.f, hi = 0.f;
    constexpr uint32_t N4 = 0x0f0f0f0fu, N1 = 0x10101010u;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t w = j < 4 ? word(p.q0, j) : word(p.q1, j - 4);
        const uint32_t hs = (j < 4 ? word(p.h0, j) : word(p.h1, j - 4)) >> (2 * c);
        lo = dot4((w & N4) | ((hs << 4) & N1), xf + 4 * j, lo);
        hi = dot4(((w >> 4) & N4) | ((hs << 3) & N1), xf + 32 + 4 * j, hi);
    }
    uint32_t sc0, sc1, m0, m1;
    q4k_scales(p.hdr.y, p.hdr.z, p.hdr.w, c, sc0, sc1, m0, m1);
    const float d = f16_bits_to_f32(p.hdr.x & 0xffffu), dmin = f16_bits_to_f32(p.hdr.x >> 16);
    float acc = d * (float)sc0 * lo - dmin * (float)m0 * (sx[0] + sx[1]);
    acc += d * (float)sc1 * hi - dmin * (float)m1 * (sx[2] + sx[3]);
    return acc;
}

// The same dot products in two halves of 32 activations each (xh: the half's activations), for callers that cannot
// afford all 64 in registers: half h leaves its raw sums in out[], dot_f32_finish combines both halves' sums.  The
// operations and their order are those of dot_f32: the same bits.
__device__ __forceinline__ void dot_f32_half(const Piece<HQ_Q4_K>& p, int, int h, const float* xh, float* out) {
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t w = j < 4 ? word(p.q0, j) : word(p.q1, j - 4);
        acc = dot4((h ? w >> 4 : w) & 0x0f0f0f0fu, xh + 4 * j, acc);
    }
    out[0] = acc;
}
__device__ __forceinline__ float dot_f32_finish(const Piece<HQ_Q4_K>& p, int c, const float* lo, const float* hi, const float* sx) {
    uint32_t sc0, sc1, m0, m1;
    q4k_scales(p.hdr.y, p.hdr.z, p.hdr.w, c, sc0, sc1, m0, m1);
    const float d = f16_bits_to_f32(p.hdr.x & 0xffffu), dmin = f16_bits_to_f32(p.hdr.x >> 16);
    float acc = d * (float)sc0 * lo[0] - dmin * (float)m0 * (sx[0] + sx[1]);
    acc += d * (float)sc1 * hi[0] - dmin * (float)m1 * (sx[2] + sx[3]);
    return acc;
}
__device__ __forceinline__ void dot_f32_half(const Piece<HQ_Q5_K>& p, int c, int h, const float* xh, float* out) {
    float acc = 0.f;
    constexpr uint32_t N4 = 0x0f0f0f0fu, N1 = 0x10101010u;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t w = j < 4 ? word(p.q0, j) : word(p.q1, j - 4);
        const uint32_t hs = (j < 4 ? word(p.h0, j) : word(p.h1, j - 4)) >> (2 * c);
        acc = dot4(h ? ((w >> 4) & N4) | ((hs << 3) & N1) : (w & N4) | ((hs << 4) & N1), xh + 4 * j, acc);
    }
    out[0] = acc;
}
__device__ __forceinline__ float dot_f32_finish(const Piece<HQ_Q5_K>& p, int c, const float* lo, const float* hi, const float* sx) {
    uint32_t sc0, sc1, m0, m1;
    q4k_scales(p.hdr.y, p.hdr.z, p.hdr.w, c, sc0, sc1, m0, m1);
    const float d = f16_bits_to_f32(p.hdr.x & 0xffffu), dmin = f16_bits_to_f32(p.hdr.x >> 16);
    float acc = d * (float)sc0 * lo[0] - dmin * (float)m0 * (sx[0] + sx[1]);
    acc += d * (float)sc1 * hi[0] - dmin * (float)m1 * (sx[2] + sx[3]);
    return acc;
}
// Q6_K: half 0 = the runs of the low nibbles (r0, r1), half 1 = those of the high nibbles (r2, r3).
__device__ __forceinline__ void dot_f32_half(const Piece<HQ_Q6_K>& p, int, int h, const float* xh, float* out) {
    float ra = 0.f, rb = 0.f;
    constexpr uint32_t N4 = 0x0f0f0f0fu, N2 = 0x30303030u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t a = word(p.qa, j), b = word(p.qb, j), v = word(p.qh, j);
        if (h == 0) {
            ra = dot4((a & N4) | ((v << 4) & N2), xh + 4 * j, ra);
            rb = dot4((b & N4) | ((v << 2) & N2), xh + 16 + 4 * j, rb);
        } else {
            ra = dot4(((a >> 4) & N4) | (v & N2), xh + 4 * j, ra);
            rb = dot4(((b >> 4) & N4) | ((v >> 2) & N2), xh + 16 + 4 * j, rb);
        }
    }
    out[0] = ra;
    out[1] = rb;
}
__device__ __forceinline__ float dot_f32_finish(const Piece<HQ_Q6_K>& p, int c, const float* lo, const float* hi, const float* sx) {
    return q6k_combine(p, c, 32.f, lo[0], lo[1], hi[0], hi[1], sx);
}

// Q4_0: y = d * (q - 8); low nibbles are elements 0..15 of the block, high nibbles 16..31.
__device__ __forceinline__ float dot_f32(const Piece<HQ_Q4_0>& p, int, const float* xf, const float* sx) {
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t w = word(p.q, j);
        lo = dot4(w & 0x0f0f0f0fu, xf + 4 * j, lo);
        hi = dot4((w >> 4) & 0x0f0f0f0fu, xf + 16 + 4 * j, hi);
    }
    return f16_bits_to_f32(p.d) * ((lo + hi) - 8.f * (sx[0] + sx[1]));
}

__device__ __forceinline__ float dot_f32(const Piece<HQ_Q8_0>& p, int, const float* xf, const float*) {
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t w = j < 4 ? word(p.q0, j) : word(p.q1, j - 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = fmaf(sbyte(w, i), xf[4 * j + i], acc);
    }
    return f16_bits_to_f32(p.d) * acc;
}

// Two blocks: the first one's weights are bytes 2 .. 33 (each word spans two of the fetched ones), its scale the low half
// of word 0; the second one's scale is the high half of word 8, its weights words 9 .. 16.  Per block the operations of
// the one-block form; the lane adds the two.
__device__ __forceinline__ float dot_f32(const Piece<HQ_Q8_0_X2>& p, int, const float* xf, const float*) {
    const uint32_t w[17] = {p.a.x, p.a.y, p.a.z, p.a.w, p.b.x, p.b.y, p.b.z, p.b.w, p.c.x, p.c.y, p.c.z, p.c.w, p.e.x, p.e.y, p.e.z, p.e.w, p.t};
    float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t q = __builtin_amdgcn_alignbyte(w[j + 1], w[j], 2);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc0 = fmaf(sbyte(q, i), xf[4 * j + i], acc0);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc1 = fmaf(sbyte(w[9 + j], i), xf[32 + 4 * j + i], acc1);
    }
    // (the first product rounded on its own, the second fused into the sum: said here, so that every kernel that inlines this
    // gets the same bits whichever of the two the compiler would have fused)
    float first = f16_bits_to_f32(w[0] & 0xffffu) * acc0;
    asm volatile("" : "+v"(first));
    return fmaf(f16_bits_to_f32(w[8] >> 16), acc1, first);
}
__device__ __forceinline__ float dot_pair(const Piece<HQ_Q8_0_X2>&, int, const uint32_t*, const float*, uint32_t, uint32_t, uint32_t) {
    return 0.f;
}

// Doubled pieces: the base type's dot product of either half, each over its own activations (the second half's follow
// the first's in xp / xf and sx), added.
template <int TYPE>
__device__ __forceinline__ float dot_pair(const Piece<TYPE>& p, int c, const uint32_t* xp, const float* sx, uint32_t m4, uint32_t m2,
                                          uint32_t magic) {
    constexpr int B = kBaseType<TYPE>;
    // (the first half's value is final before the second is added: one way of fusing the last multiply, in every kernel)
    float first = dot_pair(p.a, c, xp, sx, m4, m2, magic);
    asm volatile("" : "+v"(first));
    return first + dot_pair(p.b, c, xp + (kBlock32<B> ? 16 : 32), sx + (kBlock32<B> ? 2 : 4), m4, m2, magic);
}
template <int TYPE>
__device__ __forceinline__ float dot_f32(const Piece<TYPE>& p, int c, const float* xf, const float* sx) {
    constexpr int B = kBaseType<TYPE>;
    float first = dot_f32(p.a, c, xf, sx);
    asm volatile("" : "+v"(first));
    return first + dot_f32(p.b, c, xf + (kBlock32<B> ? 32 : 64), sx + (kBlock32<B> ? 2 : 4));
}

// Staging of one activation row in LDS, 16 activations per thread and pass:
// PAIR -> pre-paired bf16 words + per-16 sums, otherwise f32 values + per-16 sums.
// The fetch and the conversion are separate so that the first pass can be fetched
// ahead of the first weight loads (vector loads return in order: activations
// issued behind a deep queue of weight fetches would hold the whole workgroup at
// its barrier until those have come back).
template <bool X_BF16>
struct XRaw {
    uint4 r[X_BF16 ? 2 : 4];
    __device__ __forceinline__ void fetch(const void* __restrict__ xrow, uint32_t i) {
        const uint4* src = reinterpret_cast<const uint4*>(static_cast<const uint8_t*>(xrow) +
                                                          (size_t)i * (X_BF16 ? 32 : 64));
#pragma unroll
        for (int j = 0; j < (X_BF16 ? 2 : 4); ++j) r[j] = src[j];
    }
};

template <bool X_BF16, bool PAIR>
__device__ __forceinline__ void stage_store(const XRaw<X_BF16>& raw, uint32_t i, uint32_t* lds_x, float* lds_s) {
    float v[16];
    if constexpr (X_BF16) {
        const uint4 a = raw.r[0], b = raw.r[1];
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            v[2 * j] = bf16_bits_to_f32(w[j] & 0xffffu);
            v[2 * j + 1] = bf16_bits_to_f32(w[j] >> 16);
        }
        if constexpr (PAIR) {
            uint4 o0, o1;
            o0.x = (w[0] & 0xffffu) | (w[1] << 16);
            o0.y = (w[0] >> 16) | (w[1] & 0xffff0000u);
            o0.z = (w[2] & 0xffffu) | (w[3] << 16);
            o0.w = (w[2] >> 16) | (w[3] & 0xffff0000u);
            o1.x = (w[4] & 0xffffu) | (w[5] << 16);
            o1.y = (w[4] >> 16) | (w[5] & 0xffff0000u);
            o1.z = (w[6] & 0xffffu) | (w[7] << 16);
            o1.w = (w[6] >> 16) | (w[7] & 0xffff0000u);
            reinterpret_cast<uint4*>(lds_x)[2 * i] = o0;
            reinterpret_cast<uint4*>(lds_x)[2 * i + 1] = o1;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[4 * j] = __uint_as_float(raw.r[j].x);
            v[4 * j + 1] = __uint_as_float(raw.r[j].y);
            v[4 * j + 2] = __uint_as_float(raw.r[j].z);
            v[4 * j + 3] = __uint_as_float(raw.r[j].w);
        }
    }
    if constexpr (!PAIR) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            reinterpret_cast<float4*>(lds_x)[4 * i + j] = make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) s += v[j];
    lds_s[i] = s;
}

// SwiGLU staging: activations silu(gate) * up (silu_mul_f32, the arithmetic of the
// stand-alone SwiGLU kernel) written to LDS as f32 with their per-16 sums.  The
// exponentials are the expensive part, so every thread takes four activations, not
// sixteen, and the sum of a run of sixteen is chained through the four lanes of a
// quad in the order a single thread would add them.
struct SwigluRaw {
    uint4 g, u;
    __device__ __forceinline__ void fetch(const uint8_t* grow, const uint8_t* urow, uint32_t i) {
        g = reinterpret_cast<const uint4*>(grow)[i];
        u = reinterpret_cast<const uint4*>(urow)[i];
    }
};

__device__ __forceinline__ float swiglu1(uint32_t g, uint32_t u) {
    return silu_mul_f32(__uint_as_float(g), __uint_as_float(u));
}

// Value of `v` in the previous lane of the quad (lane 0 of a quad receives its own).
__device__ __forceinline__ float quad_prev(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x90 /* quad_perm [0,0,1,2] */, 0xf, 0xf, false));
}

__device__ __forceinline__ void stage_swiglu(const SwigluRaw& raw, uint32_t i, uint32_t* lds_x, float* lds_s) {
#pragma clang fp contract(off)  // the sums add the rounded products, as a kernel reading them from memory would
    const float v0 = swiglu1(raw.g.x, raw.u.x), v1 = swiglu1(raw.g.y, raw.u.y);
    const float v2 = swiglu1(raw.g.z, raw.u.z), v3 = swiglu1(raw.g.w, raw.u.w);
    reinterpret_cast<float4*>(lds_x)[i] = make_float4(v0, v1, v2, v3);
    const uint32_t q = threadIdx.x & 3u;
    // lane q of the quad continues the running sum of lanes 0..q-1
    float s = 0.f;
#pragma unroll
    for (uint32_t step = 0; step < 4; ++step) {
        const float carry = quad_prev(s);
        if (q == step) s = (((step ? carry : 0.f) + v0) + v1) + v2 + v3;
    }
    if (q == 3) lds_s[i >> 2] = s;
}

// v + (v from the lane selected by a DPP control), one VALU op.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
    return v + __int_as_float(t);
}

// Sum over aligned groups of L = 2^log_l lanes; every lane of a group ends up with
// the group's sum.  Quad permutes and row mirrors cover 16 lanes, the last two
// levels cross 16-lane rows with permlane swaps.
__device__ __forceinline__ float group_sum(float v, uint32_t log_l) {
    if (log_l >= 1) v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    if (log_l >= 2) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    if (log_l >= 3) v = dpp_add<0x141>(v);  // row_half_mirror
    if (log_l >= 4) v = dpp_add<0x140>(v);  // row_mirror
    if (log_l >= 5) v = xor16_add(v);
    if (log_l >= 6) v = xor32_add(v);
    return v;
}

}  // namespace
}  // namespace hq

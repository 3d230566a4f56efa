// Dequant-fused GEMV over GGML Q4_K / Q6_K / Q8_0 blocks for decode (m <= 8) and
// for mul_mat_id expert dispatch (one GEMV per routed (token, slot) row).
// y[p, r] = sum_k x[xrow(p), k] * W_p[r, k],  W_p = w (dense) or w + ids[p]*stride.
//
// Bandwidth-bound: the algorithmic traffic is the packed weight bytes
// (0.5625 / 0.8203 / 1.0625 bytes per weight for Q4_K / Q6_K / Q8_0); the
// activation vector is staged once per workgroup in LDS.
//
// Mapping (64-lane wavefronts, 4 per workgroup):
//   * a lane owns one 64-weight piece of a K-quant super-block (Q4_K: one
//     64-element chunk = 32 bytes of nibbles; Q6_K: 16 bytes of ql, 16 of
//     ql+32, 16 of qh = four 16-element runs) or one 32-weight Q8_0 block, and
//     fetches it with 16-byte loads;
//   * L = the largest power of two <= 64 dividing the pieces of a row; L lanes
//     share a row, so a wave covers 64/L rows (a "slot") per step and takes
//     pieces/L steps over the row;
//   * a wave owns NR slots and keeps D weight fetches in flight while it walks
//     its (step, slot) tasks; the activations of a step are read from LDS once
//     and re-used for all NR slots;
//   * partial sums are reduced across the L lanes with DPP row operations.
//
// bf16 activations with K-quants use v_dot2c_f32_bf16: nibbles / 6-bit values
// are turned into bf16 pairs with one and-or against the magic 0x4300 (=128.0,
// ulp 1), i.e. the pair holds (128+q); the offset is removed afterwards with
// the per-16-element activation sums kept beside the activations in LDS:
//   sum (128+q) x = 128*sum x + sum q x.
// Products bf16*bf16 are exact in f32, accumulation is f32.  The activations
// are stored pre-paired, (x[4t], x[4t+2]) and (x[4t+1], x[4t+3]), which is the
// order in which one masked shift of a little-endian weight word yields values.
// f32 activations (the reference's dtype) and Q8_0 use exact v_cvt + v_fma.
#include <math.h>

#include "hq_internal.h"

namespace hq {

namespace {

constexpr uint32_t M4 = 0x000f000fu, M2 = 0x00300030u, MAGIC = 0x43004300u;

template <int TYPE>
struct Lane {  // weights per lane and step
    static constexpr int kElems = TYPE == HQ_Q8_0 ? 32 : 64;
};

// Per-lane fetch of one piece of row data.
template <int TYPE>
struct Piece;

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
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t* blk, int c) {
        const int h = c >> 1, lr = c & 1;
        qa = ld16_unaligned(blk + 64 * h + 16 * lr);
        qb = ld16_unaligned(blk + 64 * h + 32 + 16 * lr);
        qh = ld16_unaligned(blk + 128 + 32 * h + 16 * lr);
        sc = ld8_unaligned(blk + 192 + 8 * h);
        d = ld2(blk + 208);
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

__device__ __forceinline__ float dot_pair(const Piece<HQ_Q6_K>& p, int c, const uint32_t* xp, const float* sx,
                                          uint32_t m4, uint32_t m2, uint32_t magic) {
    float r0 = 0.f, r1 = 0.f, r2 = 0.f, r3 = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t a = word(p.qa, j), b = word(p.qb, j), v = word(p.qh, j);
        r0 = dot2_bf16(and_or((v << 4), m2, (a & m4) | magic), xp[2 * j], r0);
        r0 = dot2_bf16(and_or((v >> 4), m2, ((a >> 8) & m4) | magic), xp[2 * j + 1], r0);
        r1 = dot2_bf16(and_or((v << 2), m2, (b & m4) | magic), xp[8 + 2 * j], r1);
        r1 = dot2_bf16(and_or((v >> 6), m2, ((b >> 8) & m4) | magic), xp[8 + 2 * j + 1], r1);
        r2 = dot2_bf16(and_or(v, m2, ((a >> 4) & m4) | magic), xp[16 + 2 * j], r2);
        r2 = dot2_bf16(and_or((v >> 8), m2, ((a >> 12) & m4) | magic), xp[16 + 2 * j + 1], r2);
        r3 = dot2_bf16(and_or((v >> 2), m2, ((b >> 4) & m4) | magic), xp[24 + 2 * j], r3);
        r3 = dot2_bf16(and_or((v >> 10), m2, ((b >> 12) & m4) | magic), xp[24 + 2 * j + 1], r3);
    }
    // scale bytes lr, lr+2, lr+4, lr+6 of this half's eight; values hold 128 + q with q in 0..63
    // and the format's own -32, hence the 160.
    const int lr = c & 1;
    const uint32_t s01 = p.sc.x >> (8 * lr), s23 = p.sc.y >> (8 * lr);
    const float d = f16_bits_to_f32(p.d);
    float acc = (float)(int)(int8_t)(s01 & 0xff) * (r0 - 160.f * sx[0]);
    acc += (float)(int)(int8_t)((s01 >> 16) & 0xff) * (r1 - 160.f * sx[1]);
    acc += (float)(int)(int8_t)(s23 & 0xff) * (r2 - 160.f * sx[2]);
    acc += (float)(int)(int8_t)((s23 >> 16) & 0xff) * (r3 - 160.f * sx[3]);
    return d * acc;
}

// ---- f32 activations (xf: this lane's 64 (32 for Q8_0) activations, sx: run sums) ----
__device__ __forceinline__ float dot4(uint32_t q, const float* x, float acc) {
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
    const int lr = c & 1;
    const uint32_t s01 = p.sc.x >> (8 * lr), s23 = p.sc.y >> (8 * lr);
    const float d = f16_bits_to_f32(p.d);
    float acc = (float)(int)(int8_t)(s01 & 0xff) * (r0 - 32.f * sx[0]);
    acc += (float)(int)(int8_t)((s01 >> 16) & 0xff) * (r1 - 32.f * sx[1]);
    acc += (float)(int)(int8_t)(s23 & 0xff) * (r2 - 32.f * sx[2]);
    acc += (float)(int)(int8_t)((s23 >> 16) & 0xff) * (r3 - 32.f * sx[3]);
    return d * acc;
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

// Stage one activation row in LDS: PAIR -> pre-paired bf16 words + per-16 sums,
// otherwise f32 values + per-16 sums.  Each thread handles 16 activations.
template <bool X_BF16, bool PAIR>
__device__ __forceinline__ void stage_x(const void* __restrict__ xrow, uint32_t k, uint32_t* lds_x, float* lds_s) {
    for (uint32_t i = threadIdx.x; i < k / 16; i += blockDim.x) {
        float v[16];
        if constexpr (X_BF16) {
            const uint4* src = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(xrow) + 16 * i);
            const uint4 a = src[0], b = src[1];
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
            const float4* src = reinterpret_cast<const float4*>(static_cast<const float*>(xrow) + 16 * i);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 t = src[j];
                v[4 * j] = t.x;
                v[4 * j + 1] = t.y;
                v[4 * j + 2] = t.z;
                v[4 * j + 3] = t.w;
            }
        }
        if constexpr (!PAIR) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                reinterpret_cast<float4*>(lds_x)[4 * i + j] =
                    make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
        }
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) s += v[j];
        lds_s[i] = s;
    }
}

struct KArgs {
    const void* x;
    const uint8_t* w;
    const uint32_t* ids;
    float* y;
    uint32_t top_k, n, k, n_experts;
    uint64_t expert_stride;
    uint32_t log_l;  // log2 of the lanes that share one row
    // Bit masks of the nibble -> bf16 conversion.  They are passed as arguments and
    // not written as literals so that the compiler keeps them in registers and
    // forms the three-operand v_and_or_b32 (gfx9 VOP3 takes no literals; with
    // literals it emits v_and + v_or instead).
    uint32_t m4, m2, magic;
};

// v + (v from the lane selected by a DPP control), one VALU op.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
    return v + __int_as_float(t);
}

// Sum over aligned groups of L = 2^log_l lanes; every lane of a group ends up with
// the group's sum.  Quad permutes and row mirrors cover 16 lanes, the last two
// levels cross 16-lane rows and go through ds_bpermute.
__device__ __forceinline__ float group_sum(float v, uint32_t log_l) {
    if (log_l >= 1) v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    if (log_l >= 2) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    if (log_l >= 3) v = dpp_add<0x141>(v);  // row_half_mirror
    if (log_l >= 4) v = dpp_add<0x140>(v);  // row_mirror
    if (log_l >= 5) v += __shfl_xor(v, 16);
    if (log_l >= 6) v += __shfl_xor(v, 32);
    return v;
}

// Loads the activations of one piece from LDS into registers.
template <int TYPE, bool PAIR, int XW>
__device__ __forceinline__ void load_x_piece(const uint32_t* lds_x, const float* lds_s, uint32_t pc, int c,
                                             uint32_t* xr, float* sx) {
    constexpr int EPL = Lane<TYPE>::kElems;
    if constexpr (TYPE == HQ_Q6_K) {
        // four runs of 16 at stride 32 inside one 128-element half
        const uint32_t e0 = (pc >> 2) * 256u + (uint32_t)(c >> 1) * 128u + (uint32_t)(c & 1) * 16u;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t e = e0 + 32u * r;
            const uint4* src = reinterpret_cast<const uint4*>(lds_x + (PAIR ? e / 2 : e));
#pragma unroll
            for (int j = 0; j < XW / 16; ++j) {
                const uint4 t = src[j];
                xr[(XW / 4) * r + 4 * j] = t.x;
                xr[(XW / 4) * r + 4 * j + 1] = t.y;
                xr[(XW / 4) * r + 4 * j + 2] = t.z;
                xr[(XW / 4) * r + 4 * j + 3] = t.w;
            }
            sx[r] = lds_s[e / 16];
        }
    } else {
        // Q4_K: 64 consecutive activations; Q8_0: 32
        const uint32_t e0 = pc * EPL;
        const uint4* src = reinterpret_cast<const uint4*>(lds_x + (PAIR ? e0 / 2 : e0));
#pragma unroll
        for (int j = 0; j < XW / 4; ++j) {
            const uint4 t = src[j];
            xr[4 * j] = t.x;
            xr[4 * j + 1] = t.y;
            xr[4 * j + 2] = t.z;
            xr[4 * j + 3] = t.w;
        }
#pragma unroll
        for (int r = 0; r < EPL / 16; ++r) sx[r] = lds_s[e0 / 16 + r];
    }
}

// One workgroup = 4 waves sharing the staged activation row.  A wave owns NR
// "row slots" (a slot = the 64/L rows its lanes cover at once) and walks the
// (step, slot) tasks in step-major order with D weight fetches in flight:
// the fetch for task t+D is issued right after task t has consumed its
// registers, so HBM latency is covered by D-1 tasks of arithmetic per wave
// (times the waves resident on the SIMD).  The activations of a step stay in
// registers for all NR slots.  NR % D == 0 keeps every buffer index static.
template <int TYPE, bool X_BF16, bool PAIR, int NR, int D>
__global__ __launch_bounds__(256) void gemv_kernel(KArgs a) {
    static_assert(NR % D == 0, "buffer rotation must repeat per step");
    extern __shared__ uint4 smem[];
    constexpr int EPL = Lane<TYPE>::kElems;
    constexpr uint32_t BYTES = TYPE == HQ_Q4_K ? Q4K_BYTES : TYPE == HQ_Q6_K ? Q6K_BYTES : Q8_0_BYTES;
    constexpr int XW = PAIR ? EPL / 2 : EPL;  // LDS words per piece

    uint32_t* lds_x = reinterpret_cast<uint32_t*>(smem);
    float* lds_s = reinterpret_cast<float*>(lds_x + (PAIR ? a.k / 2 : a.k));

    const uint32_t p = blockIdx.y;
    const uint8_t* w = a.w;
    bool valid = true;
    if (a.ids) {
        const uint32_t e = a.ids[p];
        valid = e < a.n_experts;
        w += (size_t)(valid ? e : 0u) * a.expert_stride;
    }

    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t L = 1u << a.log_l;
    const uint32_t rpw = 64u >> a.log_l;  // rows per slot
    const uint32_t li = lane & (L - 1u);
    const uint32_t steps = (a.k / EPL) >> a.log_l;  // pieces per row / L (host guarantees divisibility)
    const uint32_t row0 = (blockIdx.x * 4u + wave) * rpw * NR + (lane >> a.log_l);
    const uint32_t row_bytes = (a.k / (TYPE == HQ_Q8_0 ? 32 : 256)) * BYTES;
    // L >= 4 for the K-quants (k >= 256), so a lane keeps the same sub-piece index c
    // on every step.
    const int c = TYPE == HQ_Q8_0 ? 0 : (int)(li & 3u);
    // byte offset of this lane's piece inside a row at step 0, and its advance per step
    const uint32_t boff0 = (TYPE == HQ_Q8_0 ? li : li >> 2) * BYTES;
    const uint32_t bstep = (TYPE == HQ_Q8_0 ? L : L >> 2) * BYTES;

    // Address of slot u's row (clamped to the last row: always a valid read).
    const uint8_t* wl = w + boff0;
    auto row_ptr = [&](int u) -> const uint8_t* {
        uint32_t r = row0 + (uint32_t)u * rpw;
        r = r < a.n ? r : a.n - 1u;
        return wl + (size_t)r * row_bytes;
    };

    // First D fetches go out before the activations are staged, so their latency
    // overlaps the staging and its barrier.
    Piece<TYPE> buf[D];
#pragma unroll
    for (int u = 0; u < D; ++u) buf[u].load(row_ptr(u), c);

    const size_t xbytes = X_BF16 ? 2 : 4;
    stage_x<X_BF16, PAIR>(static_cast<const uint8_t*>(a.x) + (size_t)(p / a.top_k) * a.k * xbytes, a.k, lds_x,
                          lds_s);

    // The conversion masks must sit in VGPRs for v_and_or_b32 (one scalar operand
    // at most per VALU op on gfx9); the copy is opaque so they stay there.
    uint32_t m4, m2, magic;
    asm volatile("v_mov_b32 %0, %3\n\tv_mov_b32 %1, %4\n\tv_mov_b32 %2, %5"
                 : "=v"(m4), "=v"(m2), "=v"(magic)
                 : "s"(a.m4), "s"(a.m2), "s"(a.magic));

    float acc[NR];
#pragma unroll
    for (int u = 0; u < NR; ++u) acc[u] = 0.f;

    __syncthreads();

    for (uint32_t s = 0; s < steps; ++s) {
        uint32_t xr[XW];
        float sx[4];
        load_x_piece<TYPE, PAIR, XW>(lds_x, lds_s, li + s * L, c, xr, sx);
        const bool more = s + 1 < steps;  // uniform
#pragma unroll
        for (int u = 0; u < NR; ++u) {
            Piece<TYPE>& b = buf[u % D];
            if constexpr (PAIR)
                acc[u] += dot_pair(b, c, xr, sx, m4, m2, magic);
            else
                acc[u] += dot_f32(b, c, reinterpret_cast<const float*>(xr), sx);
            // refill this buffer with the task D ahead: same step while slots remain,
            // else the first slots of the next step
            if (u + D < NR || more) {
                const uint8_t* nxt = u + D < NR ? row_ptr(u + D) + (size_t)s * bstep
                                                : row_ptr(u + D - NR) + (size_t)(s + 1) * bstep;
                // Tie the refill to this task's result: without the (empty) asm the
                // compiler hoists every refill above the arithmetic into fresh
                // registers, which doubles the buffers and halves occupancy.
                asm volatile("" : "+v"(nxt) : "v"(acc[u]));
                b.load(nxt, c);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

#pragma unroll
    for (int u = 0; u < NR; ++u) {
        const float v = group_sum(acc[u], a.log_l);
        const uint32_t r = row0 + (uint32_t)u * rpw;
        if (li == 0 && r < a.n) a.y[(size_t)p * a.n + r] = valid ? v : __builtin_nanf("");
    }
}

template <int TYPE, bool X_BF16, bool PAIR, int NR, int D>
int launch_r(hipStream_t s, const KArgs& ka, uint32_t pairs, uint32_t rpw, size_t lds) {
    auto kern = gemv_kernel<TYPE, X_BF16, PAIR, NR, D>;
    if (lds > 64 * 1024) {
        if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                               "hipFuncSetAttribute(gemv LDS)"))
            return rc;
    }
    const uint32_t rows_per_wg = 4 * rpw * NR;
    const dim3 grid((ka.n + rows_per_wg - 1) / rows_per_wg, pairs);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, ka);
    return check_launch("gemv kernel launch");
}

template <int TYPE, bool X_BF16>
int launch_t(hipStream_t s, const GemvArgs& a) {
    constexpr bool PAIR = X_BF16 && TYPE != HQ_Q8_0;
    constexpr int EPL = Lane<TYPE>::kElems;
    KArgs ka{a.x, a.w, a.ids, a.y, a.top_k, a.n, a.k, a.n_experts, a.expert_stride, 0, M4, M2, MAGIC};
    const uint32_t pieces = a.k / EPL;
    // L = largest power of two <= 64 that divides the pieces of a row
    uint32_t log_l = 0;
    while (log_l < 6 && pieces % (2u << log_l) == 0) ++log_l;
    ka.log_l = log_l;
    const uint32_t rpw = 64u >> log_l;
    const size_t lds = (size_t)(PAIR ? a.k * 2 : a.k * 4) + (size_t)(a.k / 16) * 4;
    if (lds > 160 * 1024 - 512)
        return fail(HQ_ERR_UNSUPPORTED, "gemv: k = %u needs %zu bytes of LDS (limit 160 KiB)", a.k, lds);
    // Tasks (row slot x step) one SIMD would get if the work were spread evenly over
    // 256 CUs x 4 SIMDs; more slots per wave amortise the per-wave set-up, fewer keep
    // every SIMD busy on small problems.
    const uint64_t slots = (uint64_t)((a.n + rpw - 1) / rpw) * a.pairs;
    const uint64_t per_simd = slots / 1024;
    if (per_simd >= 32) return launch_r<TYPE, X_BF16, PAIR, 8, 4>(s, ka, a.pairs, rpw, lds);
    if (per_simd >= 8) return launch_r<TYPE, X_BF16, PAIR, 4, 2>(s, ka, a.pairs, rpw, lds);
    if (per_simd >= 2) return launch_r<TYPE, X_BF16, PAIR, 2, 2>(s, ka, a.pairs, rpw, lds);
    return launch_r<TYPE, X_BF16, PAIR, 1, 1>(s, ka, a.pairs, rpw, lds);
}

}  // namespace

int launch_gemv(hipStream_t s, const GemvArgs& a, hq_act_dtype xdt, hq_ggml_type t) {
    const bool bf = xdt == HQ_BF16;
    switch (t) {
        case HQ_Q4_K: return bf ? launch_t<HQ_Q4_K, true>(s, a) : launch_t<HQ_Q4_K, false>(s, a);
        case HQ_Q6_K: return bf ? launch_t<HQ_Q6_K, true>(s, a) : launch_t<HQ_Q6_K, false>(s, a);
        case HQ_Q8_0: return bf ? launch_t<HQ_Q8_0, true>(s, a) : launch_t<HQ_Q8_0, false>(s, a);
    }
    return fail(HQ_ERR_UNSUPPORTED, "gemv: ggml type %d", (int)t);
}

}  // namespace hq

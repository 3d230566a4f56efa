// Dequant-fused product for 3..8 activation rows (small-batch decode) on the matrix cores:
// y[m, n] = sum_k x[m, k] * W[n, k] with every weight fetched once for all rows, where the GEMV
// kernel would fetch it once per row.  Q4_K, Q5_K and Q6_K weights, k a multiple of 1024 (the stage-once form at
// the end of the file: any k of whole super-blocks, and Q8_0 / Q4_0 under bf16 rows).
//
// Bandwidth-bound like the GEMV (0.5625 bytes per weight); the arithmetic that depends on the row
// count moves to v_mfma_f32_16x16x32_bf16, what is left on the VALU (nibbles -> bf16, scales) does
// not depend on it.
//
// Mapping.  A workgroup owns 16 weight rows, its four waves a quarter of k each (super-block
// 4*chunk + wave of every 1024-element chunk), summed through LDS at the end.  The MFMA takes the
// activations as its first operand and the weights as its second: lane (j, g) (j = lane % 16,
// g = lane / 16) supplies weights 8g..8g+7 of one 32-weight sub-block of row j -- the nibbles of
// eight bytes it fetched itself -- and receives the products of row j with activation rows
// 4g..4g+3.  So the lane that holds a row's outputs also holds that row's block header, and
// applies the sub-block scale to the four sums without any cross-lane traffic:
//   acc += d*sc * C - (128 * d*sc + dmin*m) * S,   S = sum of the activations of the sub-block,
// where C is the MFMA result over the values 128 + q (the nibble under the bit pattern of bf16
// 128.0, one v_and_or_b32 per pair, exact).  The second term is itself a small product over the
// sub-blocks, (activation row x sub-block) . (sub-block x weight row), and goes through
// v_mfma_f32_16x16x4_f32 in full f32, two instructions per super-block.
//
// Activations are staged per 1024-element chunk, double-buffered: bf16 rows as they are (rows
// 0..7 of the MFMA, 8..15 repeat them and are ignored), f32 rows as an exact bf16 hi + lo pair in
// rows m and m + 8 whose results are added at the end (16 bits of mantissa; the GEMV kernel works
// in full f32).  Words are stored pre-paired, (x0, x2), (x1, x3), the order in which a masked
// shift of a little-endian nibble word yields values.  The per-sub-block sums S sit beside them.
#include "hq_internal.h"

namespace hq {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

struct RowsArgs {
    const void* x;
    const uint8_t* w;
    float* y;
    uint32_t m, n, k;
};

constexpr uint32_t KC = 1024;            // activations staged per pass
constexpr uint32_t XROW = KC * 2 + 16;   // bytes of a staged row; the pad spreads the rows over the banks
constexpr uint32_t SBUF = 64 * 16 * 4;   // sums [32 sub-blocks of 32, or 64 groups of 16][16 rows]
// One of the two staging buffers: 8 (bf16) or 16 (f32 as hi + lo) staged rows, then the sums.
template <bool X_BF16>
constexpr uint32_t kXBuf = (X_BF16 ? 8 : 16) * XROW;
template <bool X_BF16>
constexpr uint32_t kStage = kXBuf<X_BF16> + SBUF;
constexpr uint32_t M4 = 0x000f000fu, MAGIC = 0x43004300u;
constexpr uint32_t WIDE_MIN_ROWS = 49152;  // 768 workgroups of 64 rows

typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2v_t;

// (x0, x1), (x2, x3) -> (x0, x2), (x1, x3): one byte permute each
__device__ __forceinline__ void pair_words(uint32_t a, uint32_t b, uint32_t& o0, uint32_t& o1) {
    o0 = __builtin_amdgcn_perm(b, a, 0x05040100u);
    o1 = __builtin_amdgcn_perm(b, a, 0x07060302u);
}
// Two floats -> one word of two bf16 (round to nearest even), low half first.
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2v_t));
}
constexpr uint32_t ONES = 0x3f803f80u;  // (1.0, 1.0) in bf16: a dot2 with it adds the two halves of a word

// A thread's share of a chunk: input row tid / 32 (of at most 8), sub-block tid % 32 = 32 activations.
// SUM16: the sums are kept per 16 activations (Q6_K's scale groups), two per thread, else per 32.
// HALF (f32 rows, four at most): the hi parts in rows 0 .. 3 and the lo parts in rows 4 .. 7 of a buffer of eight rows, the
// size of the bf16 staging, where the full form puts them in rows 0 .. 7 and 8 .. 15 of sixteen.
template <bool X_BF16, bool SUM16, bool HALF = false>
struct Staged {
    static_assert(!HALF || !X_BF16, "f32 rows");
    static constexpr uint32_t LO = HALF ? 4u : 8u;  // the lo parts' row offset
    uint4 r[X_BF16 ? 4 : 8];
    __device__ __forceinline__ void fetch(const RowsArgs& a, uint32_t chunk, uint32_t tid) {
        // No branch around the loads: with conditional loads in flight the compiler can no longer count how
        // many newer loads stand behind an older one and waits for all of them.  Threads of absent rows read
        // the last row and zero what they got (in store()).
        const uint32_t row = tid >> 5, sb = tid & 31u;
        constexpr int N = X_BF16 ? 4 : 8;
        const uint32_t src_row = row < a.m ? row : a.m - 1u;
        // (a last chunk of fewer than 1024 elements: the sub-blocks past the row's end read its last one; nothing uses them)
        const uint32_t col = chunk * KC + 32u * sb < a.k ? chunk * KC + 32u * sb : a.k - 32u;
        const uint4* src = reinterpret_cast<const uint4*>(static_cast<const uint8_t*>(a.x) + ((size_t)src_row * a.k + col) * (X_BF16 ? 2 : 4));
#pragma unroll
        for (int i = 0; i < N; ++i) r[i] = src[i];
    }
    // Zeroed by an AND, not by a select: a select lets the compiler move the load itself under the condition.
    __device__ __forceinline__ uint4 masked(int i, uint32_t keep) const {
        return make_uint4(r[i].x & keep, r[i].y & keep, r[i].z & keep, r[i].w & keep);
    }
    __device__ __forceinline__ void store(uint8_t* buf, uint32_t tid, uint32_t m) const {
        const uint32_t row = tid >> 5, sb = tid & 31u;
        const uint32_t present = row < m ? 0xffffffffu : 0u;
        float* sums = reinterpret_cast<float*>(buf + kXBuf<X_BF16 || HALF>);
        if constexpr (X_BF16) {
            float s[2] = {0.f, 0.f};
            uint4 o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4 t = masked(i, present);
                pair_words(t.x, t.y, o[i].x, o[i].y);
                pair_words(t.z, t.w, o[i].z, o[i].w);
                float& si = s[SUM16 ? i / 2 : 0];
                si = dot2_bf16(t.x, ONES, si);
                si = dot2_bf16(t.y, ONES, si);
                si = dot2_bf16(t.z, ONES, si);
                si = dot2_bf16(t.w, ONES, si);
            }
            uint4* dst = reinterpret_cast<uint4*>(buf + row * XROW + sb * 64u);
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[i] = o[i];
            if constexpr (SUM16) {
                sums[(2u * sb) * 16u + row] = s[0];
                sums[(2u * sb + 1u) * 16u + row] = s[1];
            } else {
                sums[sb * 16u + row] = s[0];
            }
        } else {
            // x = hi + lo with hi = bf16(x) and lo = bf16(x - hi); the packing instruction pairs (x0, x2), (x1, x3) for free
            float sh2[2] = {0.f, 0.f}, sl2[2] = {0.f, 0.f};
            uint4 oh[4], ol[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {  // eight floats -> four hi words and four lo words
                const uint4 ta = masked(2 * i, present), tb = masked(2 * i + 1, present);
                const float v[8] = {__uint_as_float(ta.x), __uint_as_float(ta.y), __uint_as_float(ta.z), __uint_as_float(ta.w),
                                    __uint_as_float(tb.x), __uint_as_float(tb.y), __uint_as_float(tb.z), __uint_as_float(tb.w)};
                uint32_t hw[4], lw[4];
                float &sh = sh2[SUM16 ? i / 2 : 0], &sl = sl2[SUM16 ? i / 2 : 0];
#pragma unroll
                for (int q = 0; q < 2; ++q) {  // elements 4q .. 4q+3
                    const float* e = v + 4 * q;
                    const uint32_t ha = pack_bf16(e[0], e[2]), hb = pack_bf16(e[1], e[3]);
                    const float l0 = e[0] - __uint_as_float(ha << 16), l2 = e[2] - __uint_as_float(ha & 0xffff0000u);
                    const float l1 = e[1] - __uint_as_float(hb << 16), l3 = e[3] - __uint_as_float(hb & 0xffff0000u);
                    hw[2 * q] = ha, hw[2 * q + 1] = hb;
                    lw[2 * q] = pack_bf16(l0, l2), lw[2 * q + 1] = pack_bf16(l1, l3);
                    sh = dot2_bf16(ha, ONES, sh);
                    sh = dot2_bf16(hb, ONES, sh);
                    sl = dot2_bf16(lw[2 * q], ONES, sl);
                    sl = dot2_bf16(lw[2 * q + 1], ONES, sl);
                }
                oh[i] = make_uint4(hw[0], hw[1], hw[2], hw[3]);
                ol[i] = make_uint4(lw[0], lw[1], lw[2], lw[3]);
            }
            if (HALF && row >= 4u) return;  // (rows 4 .. 7 of the buffer hold the lo parts of rows 0 .. 3)
            uint4* dh = reinterpret_cast<uint4*>(buf + row * XROW + sb * 64u);
            uint4* dl = reinterpret_cast<uint4*>(buf + (row + LO) * XROW + sb * 64u);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                dh[i] = oh[i];
                dl[i] = ol[i];
            }
            if constexpr (SUM16) {
                sums[(2u * sb) * 16u + row] = sh2[0];
                sums[(2u * sb) * 16u + row + LO] = sl2[0];
                sums[(2u * sb + 1u) * 16u + row] = sh2[1];
                sums[(2u * sb + 1u) * 16u + row + LO] = sl2[1];
            } else {
                sums[sb * 16u + row] = sh2[0];
                sums[sb * 16u + row + LO] = sl2[0];
            }
        }
    }
};

// Epilogue of both kernels: the sum of the parts of the waves that share rows and of the hi and lo rows (f32
// activations), through LDS; lanes g < 2 of the first wave of a group store activation rows 4g..4g+3 of weight row
// row0 + j.
template <bool X_BF16, int NSB>
__device__ __forceinline__ void store_rows(const RowsArgs& a, uint8_t* smem, const f32x4_t& acc, uint32_t row0) {
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t j = lane & 15u, g = lane >> 4;
    float4* red = reinterpret_cast<float4*>(smem);
    red[wave * 64u + lane] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    __syncthreads();
    constexpr uint32_t SHARE = 4u / NSB;  // waves that hold parts of the same rows
    if (wave % SHARE == 0 && g < 2u && row0 + j < a.n) {
        float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (uint32_t w = wave; w < wave + SHARE; ++w) {
            const float4 t = red[w * 64u + lane];
            o[0] += t.x, o[1] += t.y, o[2] += t.z, o[3] += t.w;
            if constexpr (!X_BF16) {
                const float4 u = red[w * 64u + lane + 32u];  // the lo rows: activation rows 8 + 4g + v
                o[0] += u.x, o[1] += u.y, o[2] += u.z, o[3] += u.w;
            }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v)
            if (4u * g + v < a.m) a.y[(size_t)(4u * g + v) * a.n + row0 + j] = o[v];
    }
}

// NSB = super-blocks of a 1024-element chunk a wave works through.  1: the workgroup owns 16 weight rows and its
// waves a quarter of k each (many workgroups for small matrices).  4: it owns 64 rows, each wave 16 of them over
// all of k, so a staged chunk of activations and its barrier serve four times the weights.  2: 32 rows, two waves
// per 16 rows (half the registers of 4 for the fetches in flight).
//
// Q5 = true: Q5_K weights (176-byte super-blocks: the same header, 32 bytes of fifth bits, then the nibbles).  A
// lane also fetches the eight qh bytes that sit over its nibble bytes and ORs bit 2c (2c + 1) of each into the
// values of sub-block 2c (2c + 1): 128 + q with q < 32 is still exact in bf16.
template <bool X_BF16, int NSB, bool Q5 = false>
__global__ __launch_bounds__(256) void q4k_rows_kernel(RowsArgs a) {
    constexpr uint32_t BYTES = Q5 ? Q5K_BYTES : Q4K_BYTES, QS = Q5 ? 48u : 16u;  // super-block size, offset of the nibbles
    extern __shared__ uint4 smem4[];
    uint8_t* smem = reinterpret_cast<uint8_t*>(smem4);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t j = lane & 15u, g = lane >> 4;
    constexpr uint32_t SHARE = 4u / NSB;  // waves per 16 rows
    const uint32_t row0 = (blockIdx.x * (uint32_t)NSB + wave / SHARE) * 16u, sb0 = (wave % SHARE) * NSB;
    const uint32_t r = row0 + j < a.n ? row0 + j : a.n - 1u;  // rows past the end repeat the last one, not stored
    const uint32_t nsb = a.k / 256u, nch = a.k / KC;
    const uint8_t* wrow = a.w + (size_t)r * nsb * BYTES + QS + 8u * g;  // this lane's eight bytes of chunk 0
    const uint32_t arow = (X_BF16 ? (j & 7u) : j) * XROW + 16u * g;          // this lane's row and k-group in a staged buffer

    struct WBlock {
        uint4 hdr;
        uint2 q[4];
        uint2 qh;  // Q5_K only
    };
    struct WSet {
        WBlock b[NSB];
    };
    auto load_w = [&](uint32_t ch, WSet& set) {
#pragma unroll
        for (int s = 0; s < NSB; ++s) {
            const uint8_t* p = wrow + (size_t)(ch * 4u + sb0 + s) * BYTES;
            set.b[s].hdr = *reinterpret_cast<const uint4*>(p - QS - 8u * g);
            if constexpr (Q5) set.b[s].qh = *reinterpret_cast<const uint2*>(p - 32u);  // qh bytes 8g..8g+7
#pragma unroll
            for (int c = 0; c < 4; ++c) set.b[s].q[c] = *reinterpret_cast<const uint2*>(p + 32 * c);
        }
    };

    constexpr uint32_t XBUF = kXBuf<X_BF16>, STAGE = kStage<X_BF16>;
    // The next chunk's weights and activations are requested before the current chunk's arithmetic.  The two
    // weight buffers swap roles from chunk to chunk (the loop is unrolled by two): copying one into the other
    // would make the compiler wait for the newest loads at once.
    // the conversion masks sit in VGPRs so that (w & m4) | magic is one v_and_or_b32 (one scalar operand
    // at most per VALU op); the copy is opaque so that they stay there
    uint32_t m4, magic;
    asm volatile("v_mov_b32 %0, %2\n\tv_mov_b32 %1, %3" : "=v"(m4), "=v"(magic) : "s"(M4), "s"(MAGIC));
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    Staged<X_BF16, false> st;
    auto super_block = [&](const WBlock& wb, uint32_t sbi, const uint8_t* bufc) {
        const uint8_t* xb = bufc + arow + sbi * 512u;  // super-block sbi of the chunk: 256 activations
        // sums of its eight sub-blocks as the first operand of a 16x16x4 f32 MFMA: lane (j, g) holds
        // S[activation row j][sub-block 4t + g]
        const float* sums = reinterpret_cast<const float*>(bufc + XBUF) + sbi * 128u + 16u * g + j;
        const float d = f16_bits_to_f32(wb.hdr.x & 0xffffu), dmin = f16_bits_to_f32(wb.hdr.x >> 16);
        // -sum_b off_b * S_b, off_b = 128 d sc_b + dmin m_b, for all sixteen activation rows at once: the weights'
        // side of that small product is off of sub-block 4t + g of this lane's row.  It is picked while the scales
        // are unpacked, from plain values: a select between elements of a local array makes the compiler index
        // the array in scratch memory.
        float ds[8], mine0 = 0.f, mine1 = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t sc0, sc1, m0, m1;
            q4k_scales(wb.hdr.y, wb.hdr.z, wb.hdr.w, c, sc0, sc1, m0, m1);
            ds[2 * c] = d * (float)sc0, ds[2 * c + 1] = d * (float)sc1;
            const float oe = fmaf(128.f, ds[2 * c], dmin * (float)m0), oo = fmaf(128.f, ds[2 * c + 1], dmin * (float)m1);
            const float o = (g & 1u) ? oo : oe;  // sub-blocks 2c and 2c + 1 are g = 2 (c & 1) and 2 (c & 1) + 1 of t = c / 2
            float& mine = c < 2 ? mine0 : mine1;
            mine = (g >> 1) == (uint32_t)(c & 1) ? o : mine;
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[0], -mine0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[64], -mine1, acc, 0, 0, 0);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t w0 = wb.q[c].x, w1 = wb.q[c].y;
            uint4 blo = make_uint4(and_or(w0, m4, magic), and_or(w0 >> 8, m4, magic), and_or(w1, m4, magic),
                                   and_or(w1 >> 8, m4, magic));
            uint4 bhi = make_uint4(and_or(w0 >> 4, m4, magic), and_or(w0 >> 12, m4, magic), and_or(w1 >> 4, m4, magic),
                                   and_or(w1 >> 12, m4, magic));
            if constexpr (Q5) {
                // fifth bits of bytes (0, 2) / (1, 3) of a word, for sub-block 2c (low nibbles) and 2c + 1 (high)
                constexpr uint32_t M1 = 0x00010001u;
                const uint32_t h0 = wb.qh.x >> (2 * c), h1 = wb.qh.y >> (2 * c);
                blo.x |= (h0 & M1) << 4, blo.y |= ((h0 >> 8) & M1) << 4, blo.z |= (h1 & M1) << 4, blo.w |= ((h1 >> 8) & M1) << 4;
                bhi.x |= ((h0 >> 1) & M1) << 4, bhi.y |= ((h0 >> 9) & M1) << 4, bhi.z |= ((h1 >> 1) & M1) << 4,
                    bhi.w |= ((h1 >> 9) & M1) << 4;
            }
            const uint4 alo = *reinterpret_cast<const uint4*>(xb + 128 * c);       // sub-block 2c: 64 bytes per sub-block
            const uint4 ahi = *reinterpret_cast<const uint4*>(xb + 128 * c + 64);  // sub-block 2c + 1
            const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
            const f32x4_t clo = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, alo), __builtin_bit_cast(bf16x8_t, blo), z, 0, 0, 0);
            const f32x4_t chi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ahi), __builtin_bit_cast(bf16x8_t, bhi), z, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[v] = fmaf(ds[2 * c + 1], chi[v], fmaf(ds[2 * c], clo[v], acc[v]));
        }
    };
    auto chunk = [&](uint32_t ch, const WSet& wb, WSet& wnext, const uint8_t* bufc, uint8_t* bufn) {
        // the last chunk requests itself again rather than nothing: see Staged::fetch
        const bool more = ch + 1 < nch;
        const uint32_t ahead = more ? ch + 1 : ch;
        st.fetch(a, ahead, tid);
        load_w(ahead, wnext);
#pragma unroll
        for (int s = 0; s < NSB; ++s) super_block(wb.b[s], sb0 + s, bufc);
        st.store(bufn, tid, a.m);
        __syncthreads();  // the other buffer is complete; this one may be overwritten by the next pass
    };
    WSet wa, wb2;
    st.fetch(a, 0, tid);
    load_w(0, wa);
    st.store(smem, tid, a.m);
    __syncthreads();
    for (uint32_t ch = 0; ch < nch; ch += 2) {
        chunk(ch, wa, wb2, smem, smem + STAGE);
        if (ch + 1 < nch) chunk(ch + 1, wb2, wa, smem + STAGE, smem);
    }

    store_rows<X_BF16, NSB>(a, smem, acc, row0);
}

typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;

// A word at a 2-byte aligned address (Q6_K blocks are 210 bytes); one global_load_dword.
__device__ __forceinline__ uint32_t ld4_unaligned(const uint8_t* p) {
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}

// The same for Q6_K.  Its scales cover 16 weights, so the product runs on v_mfma_f32_16x16x16_bf16, one
// instruction per scale group: lane (j, g) supplies weights 4g..4g+3 of the group -- one word of low or high
// nibbles and the matching two-bit fields of one word of qh, merged into bf16 (128 + q, q < 64) by two
// v_and_or_b32 per pair -- and receives row j's sums with activation rows 4g..4g+3:
//   acc += d*sc * C - 160 * d*sc * S16,   S16 = sum of the group's activations (128 + the format's 32),
// the second term again through the f32 MFMA, four instructions per super-block.
template <bool X_BF16, int NSB>
__global__ __launch_bounds__(256) void q6k_rows_kernel(RowsArgs a) {
    extern __shared__ uint4 smem4[];
    uint8_t* smem = reinterpret_cast<uint8_t*>(smem4);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t j = lane & 15u, g = lane >> 4;
    constexpr uint32_t SHARE = 4u / NSB;
    const uint32_t row0 = (blockIdx.x * (uint32_t)NSB + wave / SHARE) * 16u, sb0 = (wave % SHARE) * NSB;
    const uint32_t r = row0 + j < a.n ? row0 + j : a.n - 1u;
    const uint32_t nsb = a.k / 256u, nch = a.k / KC;
    const uint8_t* wrow = a.w + (size_t)r * nsb * Q6K_BYTES;
    const uint32_t arow = (X_BF16 ? (j & 7u) : j) * XROW + 8u * g;  // four activations (8 bytes) per lane and group

    struct WBlock {
        uint32_t ql[8];  // [h][u][s]: bytes 64h + 32u + 16s + 4g .. +3 of ql
        uint32_t qh[4];  // [h][s]: bytes 32h + 16s + 4g .. +3 of qh
        uint4 sc;        // the sixteen int8 scales
        uint32_t d;
    };
    struct WSet {
        WBlock b[NSB];
    };
    auto load_w = [&](uint32_t ch, WSet& set) {
#pragma unroll
        for (int s = 0; s < NSB; ++s) {
            WBlock& b = set.b[s];
            const uint8_t* p = wrow + (size_t)(ch * 4u + sb0 + s) * Q6K_BYTES;
            // (values, not addresses of the struct's fields: taking those would put the block into scratch memory)
#pragma unroll
            for (int i = 0; i < 8; ++i) b.ql[i] = ld4_unaligned(p + 64 * (i >> 2) + 32 * ((i >> 1) & 1) + 16 * (i & 1) + 4u * g);
#pragma unroll
            for (int i = 0; i < 4; ++i) b.qh[i] = ld4_unaligned(p + 128 + 32 * (i >> 1) + 16 * (i & 1) + 4u * g);
            b.sc = ld16_unaligned(p + 192);
            b.d = ld2(p + 208);
        }
    };

    constexpr uint32_t XBUF = kXBuf<X_BF16>, STAGE = kStage<X_BF16>;
    uint32_t m4, m2, magic;
    asm volatile("v_mov_b32 %0, %3\n\tv_mov_b32 %1, %4\n\tv_mov_b32 %2, %5" : "=v"(m4), "=v"(m2), "=v"(magic) : "s"(M4), "s"(0x00300030u), "s"(MAGIC));
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    Staged<X_BF16, true> st;
    auto super_block = [&](const WBlock& wb, uint32_t sbi, const uint8_t* bufc) {
        const uint8_t* xb = bufc + arow + sbi * 512u;  // super-block sbi of the chunk: 256 activations
        // lane (j, g) of the f32 MFMA: S16[activation row j][group 4t + g] of the super-block's sixteen groups
        const float* sums = reinterpret_cast<const float*>(bufc + XBUF) + sbi * 256u + 16u * g + j;
        const float d = f16_bits_to_f32(wb.d);
        const uint32_t scw[4] = {wb.sc.x, wb.sc.y, wb.sc.z, wb.sc.w};
        float ds[16];
#pragma unroll
        for (int G = 0; G < 16; ++G) ds[G] = d * (float)(int)(int8_t)((scw[G >> 2] >> (8 * (G & 3))) & 0xffu);
#pragma unroll
        for (int t = 0; t < 4; ++t) {  // the -160 d sc S16 term: this lane's side is the scale of group 4t + g of its row
            const float mine = d * (float)(int)(int8_t)((scw[t] >> (8u * g)) & 0xffu);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[64 * t], -160.f * mine, acc, 0, 0, 0);
        }
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const uint32_t hq = wb.qh[2 * h + s];
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {  // run rr of half h: group G = 8h + 2rr + s
                    const uint32_t w = wb.ql[4 * h + 2 * (rr & 1) + s] >> (rr >= 2 ? 4 : 0);
                    const uint32_t hs = hq >> (2 * rr);
                    const uint32_t b0 = and_or(hs << 4, m2, and_or(w, m4, magic));        // weights 4g, 4g + 2
                    const uint32_t b1 = and_or(hs >> 4, m2, and_or(w >> 8, m4, magic));   // weights 4g + 1, 4g + 3
                    const int G = 8 * h + 2 * rr + s;
                    const uint2 av = *reinterpret_cast<const uint2*>(xb + 32 * G);  // 16 activations = 32 bytes per group
                    const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
                    const f32x4_t c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(bf16x4_t, av),
                                                                                __builtin_bit_cast(bf16x4_t, make_uint2(b0, b1)), z, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[v] = fmaf(ds[G], c[v], acc[v]);
                }
            }
    };
    auto chunk = [&](uint32_t ch, const WSet& wb, WSet& wnext, const uint8_t* bufc, uint8_t* bufn) {
        const bool more = ch + 1 < nch;
        const uint32_t ahead = more ? ch + 1 : ch;
        st.fetch(a, ahead, tid);
        load_w(ahead, wnext);
#pragma unroll
        for (int s = 0; s < NSB; ++s) super_block(wb.b[s], sb0 + s, bufc);
        st.store(bufn, tid, a.m);
        __syncthreads();
    };
    WSet wa, wb2;
    st.fetch(a, 0, tid);
    load_w(0, wa);
    st.store(smem, tid, a.m);
    __syncthreads();
    for (uint32_t ch = 0; ch < nch; ch += 2) {
        chunk(ch, wa, wb2, smem, smem + STAGE);
        if (ch + 1 < nch) chunk(ch + 1, wb2, wa, smem + STAGE, smem);
    }

    store_rows<X_BF16, NSB>(a, smem, acc, row0);
}

// ---- the same products with the activations staged once per CU ----
// The kernels above stage a 1024-element chunk of the activations per workgroup and pass, behind a barrier: a workgroup of
// 64 weight rows reads 16 KB of activations for every 36 KB of weights, and its waves meet at every chunk.  Where all of k
// fits the CU's LDS (k = 4096: 82 KB for bf16 rows, 148 KB for f32 rows as hi + lo) one workgroup per CU stages the
// activations once, and each of its waves then walks groups of 16 weight rows over all of k on its own -- no barrier, the
// next super-block's weights requested before the current one's arithmetic, the CUs moving through the matrix front to
// back together.  Same arithmetic per super-block as above (the same functions of the same operands), the same sums in a
// different order across k.
template <bool Q5>
struct Q4kRows {
    static constexpr uint32_t BYTES = Q5 ? Q5K_BYTES : Q4K_BYTES, QS = Q5 ? 48u : 16u;
    static constexpr bool SUM16 = false;
    struct WBlock {
        uint4 hdr;
        uint2 q[4];
        uint2 qh;
    };
    uint32_t m4, magic;
    __device__ __forceinline__ void init() {
        asm volatile("v_mov_b32 %0, %2\n\tv_mov_b32 %1, %3" : "=v"(m4), "=v"(magic) : "s"(M4), "s"(MAGIC));
    }
    // p: the super-block of this lane's row
    __device__ __forceinline__ void load(WBlock& b, const uint8_t* p, uint32_t g) const {
        b.hdr = *reinterpret_cast<const uint4*>(p);
        if constexpr (Q5) b.qh = *reinterpret_cast<const uint2*>(p + 16u + 8u * g);
#pragma unroll
        for (int c = 0; c < 4; ++c) b.q[c] = *reinterpret_cast<const uint2*>(p + QS + 8u * g + 32 * c);
    }
    // xb: this lane's row and k-group of the super-block's staged activations; sums: its entry of the sub-block sums
    __device__ __forceinline__ void super_block(const WBlock& wb, const uint8_t* xb, const float* sums, uint32_t g, f32x4_t& acc) const {
        const float d = f16_bits_to_f32(wb.hdr.x & 0xffffu), dmin = f16_bits_to_f32(wb.hdr.x >> 16);
        float ds[8], mine0 = 0.f, mine1 = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t sc0, sc1, m0, m1;
            q4k_scales(wb.hdr.y, wb.hdr.z, wb.hdr.w, c, sc0, sc1, m0, m1);
            ds[2 * c] = d * (float)sc0, ds[2 * c + 1] = d * (float)sc1;
            const float oe = fmaf(128.f, ds[2 * c], dmin * (float)m0), oo = fmaf(128.f, ds[2 * c + 1], dmin * (float)m1);
            const float o = (g & 1u) ? oo : oe;
            float& mine = c < 2 ? mine0 : mine1;
            mine = (g >> 1) == (uint32_t)(c & 1) ? o : mine;
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[0], -mine0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[64], -mine1, acc, 0, 0, 0);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t w0 = wb.q[c].x, w1 = wb.q[c].y;
            uint4 blo = make_uint4(and_or(w0, m4, magic), and_or(w0 >> 8, m4, magic), and_or(w1, m4, magic), and_or(w1 >> 8, m4, magic));
            uint4 bhi = make_uint4(and_or(w0 >> 4, m4, magic), and_or(w0 >> 12, m4, magic), and_or(w1 >> 4, m4, magic),
                                   and_or(w1 >> 12, m4, magic));
            if constexpr (Q5) {
                constexpr uint32_t M1 = 0x00010001u;
                const uint32_t h0 = wb.qh.x >> (2 * c), h1 = wb.qh.y >> (2 * c);
                blo.x |= (h0 & M1) << 4, blo.y |= ((h0 >> 8) & M1) << 4, blo.z |= (h1 & M1) << 4, blo.w |= ((h1 >> 8) & M1) << 4;
                bhi.x |= ((h0 >> 1) & M1) << 4, bhi.y |= ((h0 >> 9) & M1) << 4, bhi.z |= ((h1 >> 1) & M1) << 4,
                    bhi.w |= ((h1 >> 9) & M1) << 4;
            }
            const uint4 alo = *reinterpret_cast<const uint4*>(xb + 128 * c);
            const uint4 ahi = *reinterpret_cast<const uint4*>(xb + 128 * c + 64);
            const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
            const f32x4_t clo = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, alo), __builtin_bit_cast(bf16x8_t, blo), z, 0, 0, 0);
            const f32x4_t chi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ahi), __builtin_bit_cast(bf16x8_t, bhi), z, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[v] = fmaf(ds[2 * c + 1], chi[v], fmaf(ds[2 * c], clo[v], acc[v]));
        }
    }
    static constexpr uint32_t kXLane = 16u;   // bytes of a staged row per lane group: eight activations
    static constexpr uint32_t kSumsPerSb = 128u;
    // the super-block as 16-byte pieces (see rows_stream_kernel, XPOSE): whole pieces, rows back to back in LDS
    static constexpr uint32_t PB = BYTES / 16u, PITCH = BYTES;
    static constexpr bool kTailD = false;
    __device__ __forceinline__ void read_lds(WBlock& b, const uint8_t* p, uint32_t g) const {
        b.hdr = *reinterpret_cast<const uint4*>(p);
        if constexpr (Q5) b.qh = *reinterpret_cast<const uint2*>(p + 16u + 8u * g);
#pragma unroll
        for (int c = 0; c < 4; ++c) b.q[c] = *reinterpret_cast<const uint2*>(p + QS + 8u * g + 32 * c);
    }
};

struct Q6kRows {
    static constexpr uint32_t BYTES = Q6K_BYTES;
    static constexpr bool SUM16 = true;
    struct WBlock {
        uint32_t ql[8];
        uint32_t qh[4];
        uint4 sc;
        uint32_t d;
    };
    uint32_t m4, m2, magic;
    __device__ __forceinline__ void init() {
        asm volatile("v_mov_b32 %0, %3\n\tv_mov_b32 %1, %4\n\tv_mov_b32 %2, %5" : "=v"(m4), "=v"(m2), "=v"(magic) : "s"(M4), "s"(0x00300030u), "s"(MAGIC));
    }
    __device__ __forceinline__ void load(WBlock& b, const uint8_t* p, uint32_t g) const {
#pragma unroll
        for (int i = 0; i < 8; ++i) b.ql[i] = ld4_unaligned(p + 64 * (i >> 2) + 32 * ((i >> 1) & 1) + 16 * (i & 1) + 4u * g);
#pragma unroll
        for (int i = 0; i < 4; ++i) b.qh[i] = ld4_unaligned(p + 128 + 32 * (i >> 1) + 16 * (i & 1) + 4u * g);
        b.sc = ld16_unaligned(p + 192);
        b.d = ld2(p + 208);
    }
    __device__ __forceinline__ void super_block(const WBlock& wb, const uint8_t* xb, const float* sums, uint32_t g, f32x4_t& acc) const {
        const float d = f16_bits_to_f32(wb.d);
        const uint32_t scw[4] = {wb.sc.x, wb.sc.y, wb.sc.z, wb.sc.w};
        float ds[16];
#pragma unroll
        for (int G = 0; G < 16; ++G) ds[G] = d * (float)(int)(int8_t)((scw[G >> 2] >> (8 * (G & 3))) & 0xffu);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float mine = d * (float)(int)(int8_t)((scw[t] >> (8u * g)) & 0xffu);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[64 * t], -160.f * mine, acc, 0, 0, 0);
        }
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const uint32_t hq = wb.qh[2 * h + s];
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const uint32_t w = wb.ql[4 * h + 2 * (rr & 1) + s] >> (rr >= 2 ? 4 : 0);
                    const uint32_t hs = hq >> (2 * rr);
                    const uint32_t b0 = and_or(hs << 4, m2, and_or(w, m4, magic));
                    const uint32_t b1 = and_or(hs >> 4, m2, and_or(w >> 8, m4, magic));
                    const int G = 8 * h + 2 * rr + s;
                    const uint2 av = *reinterpret_cast<const uint2*>(xb + 32 * G);
                    const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
                    const f32x4_t c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(bf16x4_t, av),
                                                                                __builtin_bit_cast(bf16x4_t, make_uint2(b0, b1)), z, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[v] = fmaf(ds[G], c[v], acc[v]);
                }
            }
    }
    static constexpr uint32_t kXLane = 8u;    // four activations per lane group
    static constexpr uint32_t kSumsPerSb = 256u;
    // thirteen pieces cover ql, qh and the scales (208 bytes); d, the last two bytes, comes by a load of its own (a
    // fourteenth piece would read past the end of the matrix's last block).  Rows 240 bytes apart in LDS: a multiple of 16
    // for the piece stores, and the sixteen rows' words fall into sixteen different groups of four banks.
    static constexpr uint32_t PB = 13u, PITCH = 240u;
    static constexpr bool kTailD = true;
    __device__ __forceinline__ void read_lds(WBlock& b, const uint8_t* p, uint32_t g) const {
#pragma unroll
        for (int i = 0; i < 8; ++i) b.ql[i] = *reinterpret_cast<const uint32_t*>(p + 64 * (i >> 2) + 32 * ((i >> 1) & 1) + 16 * (i & 1) + 4u * g);
#pragma unroll
        for (int i = 0; i < 4; ++i) b.qh[i] = *reinterpret_cast<const uint32_t*>(p + 128 + 32 * (i >> 1) + 16 * (i & 1) + 4u * g);
        b.sc = *reinterpret_cast<const uint4*>(p + 192);
    }
};

// Q8_0 through the same walk: eight 34-byte blocks = 272 bytes = seventeen pieces stand for a super-block.  An int8 weight is
// exact in bf16, so a block is one MFMA over the converted bytes and one scaling of its four results by d; no offsets, no
// activation sums.  A block starts at an even address: in LDS (super-blocks at multiples of 16) the eight weights of lane
// group g lie at byte 34 c + 2 + 8 g, a multiple of four for odd c and two past one for even c, where three aligned words
// are shifted into place.
struct Q80Rows {
    static constexpr uint32_t BYTES = 8u * Q8_0_BYTES;
    static constexpr bool SUM16 = false;
    struct WBlock {
        uint2 q[8];
        uint32_t d[8];
    };
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ void load(WBlock& b, const uint8_t* p, uint32_t g) const {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            b.q[c] = ld8_unaligned(p + 34 * c + 2 + 8u * g);
            b.d[c] = ld2(p + 34 * c);
        }
    }
    // (x0, x2), (x1, x3), (x4, x6), (x5, x7): the order of the staged activations
    static __device__ __forceinline__ uint32_t pair(uint32_t w, int lo, int hi) {
        const float a = (float)(int)(int8_t)(w >> (8 * lo)), b = (float)(int)(int8_t)(w >> (8 * hi));
        return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);  // the upper halves: small integers are exact
    }
    __device__ __forceinline__ void super_block(const WBlock& wb, const uint8_t* xb, const float*, uint32_t, f32x4_t& acc) const {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float d = f16_bits_to_f32(wb.d[c] & 0xffffu);
            const uint32_t w0 = wb.q[c].x, w1 = wb.q[c].y;
            const uint4 b = make_uint4(pair(w0, 0, 2), pair(w0, 1, 3), pair(w1, 0, 2), pair(w1, 1, 3));
            const uint4 av = *reinterpret_cast<const uint4*>(xb + 64 * c);
            const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
            const f32x4_t r = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av), __builtin_bit_cast(bf16x8_t, b), z, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[v] = fmaf(d, r[v], acc[v]);
        }
    }
    static constexpr uint32_t kXLane = 16u;  // eight activations per lane group
    static constexpr uint32_t kSumsPerSb = 128u;
    // rows 272 bytes = 68 words apart in LDS: the sixteen rows' words fall into sixteen different groups of four banks
    static constexpr uint32_t PB = 17u, PITCH = 272u;
    static constexpr bool kTailD = false;
    __device__ __forceinline__ void read_lds(WBlock& b, const uint8_t* p, uint32_t g) const {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if (c & 1) {
                const uint32_t* q = reinterpret_cast<const uint32_t*>(p + 34 * c + 2 + 8u * g);
                b.q[c] = make_uint2(q[0], q[1]);
                b.d[c] = *reinterpret_cast<const uint32_t*>(p + 34 * c - 2) >> 16;
            } else {
                const uint32_t* q = reinterpret_cast<const uint32_t*>(p + 34 * c + 8u * g);
                const uint32_t a0 = q[0], a1 = q[1], a2 = q[2];
                b.q[c] = make_uint2(__builtin_amdgcn_alignbyte(a1, a0, 2), __builtin_amdgcn_alignbyte(a2, a1, 2));
                b.d[c] = *reinterpret_cast<const uint32_t*>(p + 34 * c);
            }
        }
    }
};

// Q4_0 likewise: eight 18-byte blocks = 144 bytes = nine pieces.  Lane group g takes weights 8 g .. 8 g + 7 of a block: the
// low (g < 2) or high nibbles of bytes 8 (g & 1) .. + 7, as bf16 128 + q like the Q4_K nibbles; the 128 and the format's
// own offset of 8 leave through the activation sums, (128 + 8) d per block, in the small f32 MFMA.
struct Q40Rows {
    static constexpr uint32_t BYTES = 8u * Q4_0_BYTES;
    static constexpr bool SUM16 = false;
    struct WBlock {
        uint2 q[8];
        uint32_t d[8];
    };
    uint32_t m4, magic;
    __device__ __forceinline__ void init() {
        asm volatile("v_mov_b32 %0, %2\n\tv_mov_b32 %1, %3" : "=v"(m4), "=v"(magic) : "s"(M4), "s"(MAGIC));
    }
    __device__ __forceinline__ void load(WBlock& b, const uint8_t* p, uint32_t g) const {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            b.q[c] = ld8_unaligned(p + 18 * c + 2 + 8u * (g & 1u));
            b.d[c] = ld2(p + 18 * c);
        }
    }
    __device__ __forceinline__ void super_block(const WBlock& wb, const uint8_t* xb, const float* sums, uint32_t g, f32x4_t& acc) const {
        float d[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) d[c] = f16_bits_to_f32(wb.d[c] & 0xffffu);
        const float mine0 = g == 0u ? d[0] : g == 1u ? d[1] : g == 2u ? d[2] : d[3];
        const float mine1 = g == 0u ? d[4] : g == 1u ? d[5] : g == 2u ? d[6] : d[7];
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[0], -136.f * mine0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sums[64], -136.f * mine1, acc, 0, 0, 0);
        const uint32_t sh = 4u * (g >> 1);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint32_t w0 = wb.q[c].x >> sh, w1 = wb.q[c].y >> sh;
            const uint4 b = make_uint4(and_or(w0, m4, magic), and_or(w0 >> 8, m4, magic), and_or(w1, m4, magic), and_or(w1 >> 8, m4, magic));
            const uint4 av = *reinterpret_cast<const uint4*>(xb + 64 * c);
            const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
            const f32x4_t r = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av), __builtin_bit_cast(bf16x8_t, b), z, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[v] = fmaf(d[c], r[v], acc[v]);
        }
    }
    static constexpr uint32_t kXLane = 16u;
    static constexpr uint32_t kSumsPerSb = 128u;
    // rows 144 bytes = 36 words apart in LDS: sixteen different groups of four banks
    static constexpr uint32_t PB = 9u, PITCH = 144u;
    static constexpr bool kTailD = false;
    __device__ __forceinline__ void read_lds(WBlock& b, const uint8_t* p, uint32_t g) const {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if (c & 1) {  // 18 c + 2 is a multiple of four
                const uint32_t* q = reinterpret_cast<const uint32_t*>(p + 18 * c + 2 + 8u * (g & 1u));
                b.q[c] = make_uint2(q[0], q[1]);
                b.d[c] = *reinterpret_cast<const uint32_t*>(p + 18 * c - 2) >> 16;
            } else {
                const uint32_t* q = reinterpret_cast<const uint32_t*>(p + 18 * c + 8u * (g & 1u));
                const uint32_t a0 = q[0], a1 = q[1], a2 = q[2];
                b.q[c] = make_uint2(__builtin_amdgcn_alignbyte(a1, a0, 2), __builtin_amdgcn_alignbyte(a2, a1, 2));
                b.d[c] = *reinterpret_cast<const uint32_t*>(p + 18 * c);
            }
        }
    }
};

// XPOSE: the weights of a task (one super-block of each of the group's 16 rows) are fetched as 16-byte pieces, consecutive
// lanes consecutive pieces of a row's block (three to five load instructions per lane where every lane fetching its own
// operands takes five for Q4_K and fourteen for Q6_K, most of them four bytes wide), written to a region of LDS the wave
// owns and read back from there as the operands each lane needs.  The pieces of the next task are in flight, in registers,
// while the current one is worked on.
// HALF: up to four f32 rows staged in the space of eight bf16 rows (hi parts in rows 0 .. 3, lo parts in rows 4 .. 7), so that
// the piece buffers of the transposed fetch fit beside them where sixteen rows would not leave the room.
template <typename T, bool X_BF16, int W, bool XPOSE, bool HALF = false>
__global__ __launch_bounds__(64 * W) void rows_stream_kernel(RowsArgs a) {
    static_assert(W % 4 == 0, "the staging works in groups of 256 threads");
    extern __shared__ uint4 smem4[];
    uint8_t* smem = reinterpret_cast<uint8_t*>(smem4);
    constexpr bool ROWS8 = X_BF16 || HALF;  // eight staged rows
    constexpr uint32_t XBUF = kXBuf<ROWS8>, STAGE = kStage<ROWS8>;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t j = lane & 15u, g = lane >> 4;
    const uint32_t nsb = a.k / 256u, nch = (a.k + KC - 1u) / KC;  // (the last chunk may hold one to three super-blocks)

    // all of k, a 1024-element chunk per 256 threads and turn, each chunk a staging buffer of its own
    {
        Staged<X_BF16, T::SUM16, HALF> st;
        for (uint32_t ch = tid >> 8; ch < nch; ch += W / 4) {
            st.fetch(a, ch, tid & 255u);
            st.store(smem + (size_t)ch * STAGE, tid & 255u, a.m);
        }
    }
    T t;
    t.init();
    const uint32_t groups = (a.n + 15u) / 16u, stride = W * gridDim.x;
    const uint32_t first = wave * gridDim.x + blockIdx.x;
    const uint32_t mine = first < groups ? (groups - first + stride - 1u) / stride : 0u;
    const uint32_t ntask = mine * nsb;
    const size_t rowb = (size_t)nsb * T::BYTES;
    // the next task to fetch: group f_grp, super-block f_sb (past the last task: the last one again, not used)
    uint32_t f_grp = first, f_sb = 0, f_left = ntask;
    auto fetch_next = [&](typename T::WBlock& wb) {
        const uint32_t r = f_grp * 16u + j < a.n ? f_grp * 16u + j : a.n - 1u;  // rows past the end repeat the last one, not stored
        t.load(wb, a.w + (size_t)r * rowb + (size_t)f_sb * T::BYTES, g);
        if (f_left > 1u) {
            --f_left;
            if (++f_sb == nsb) {
                f_sb = 0;
                f_grp += stride;
            }
        }
    };
    // XPOSE: this lane's pieces l, l + 64, ... of a task's 16 * PB: row of the group, byte offset in the block, place in LDS
    constexpr uint32_t NP = 16u * T::PB, NI = (NP + 63u) / 64u;
    uint32_t p_row[NI], p_off[NI];
    uint4 pieces[NI];
    uint32_t tail_d = 0;
    size_t rbase[NI], rbase_d = 0;  // byte offset of the piece in the matrix for the group being fetched
    uint8_t* wl = smem + (size_t)nch * STAGE + (size_t)wave * (16u * T::PITCH);
    auto set_group = [&](uint32_t grp_) {
#pragma unroll
        for (uint32_t i = 0; i < NI; ++i) {
            const uint32_t r = grp_ * 16u + p_row[i] < a.n ? grp_ * 16u + p_row[i] : a.n - 1u;
            rbase[i] = (size_t)r * rowb + p_off[i];
        }
        const uint32_t rj = grp_ * 16u + j < a.n ? grp_ * 16u + j : a.n - 1u;
        rbase_d = (size_t)rj * rowb + 208u;
    };
    auto fetch_pieces = [&]() {
#pragma unroll
        for (uint32_t i = 0; i < NI; ++i) pieces[i] = ld16_unaligned(a.w + rbase[i] + (size_t)f_sb * T::BYTES);
        if constexpr (T::kTailD) tail_d = ld2(a.w + rbase_d + (size_t)f_sb * T::BYTES);
        if (f_left > 1u) {
            --f_left;
            if (++f_sb == nsb) {
                f_sb = 0;
                f_grp += stride;
                set_group(f_grp);
            }
        }
    };
    typename T::WBlock wa, wb;
    if constexpr (XPOSE) {
#pragma unroll
        for (uint32_t i = 0; i < NI; ++i) {
            const uint32_t q = lane + 64u * i < NP ? lane + 64u * i : NP - 1u;  // (past the end: the last piece again, stored to the same place)
            p_row[i] = q / T::PB;
            p_off[i] = 16u * (q % T::PB);
        }
        set_group(f_grp < groups ? f_grp : 0u);
        if (ntask) fetch_pieces();
    } else {
        if (ntask) fetch_next(wa);
    }
    __syncthreads();

    const uint32_t arow = (ROWS8 ? (j & 7u) : j) * XROW + T::kXLane * g;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    uint32_t sb = 0, grp = first;
    auto task = [&](typename T::WBlock& cur, typename T::WBlock& nxt) {
        if constexpr (XPOSE) {
#pragma unroll
            for (uint32_t i = 0; i < NI; ++i) *reinterpret_cast<uint4*>(wl + p_row[i] * T::PITCH + p_off[i]) = pieces[i];
            if constexpr (T::kTailD) cur.d = tail_d;
            fetch_pieces();
            t.read_lds(cur, wl + j * T::PITCH, g);
        } else {
            fetch_next(nxt);
        }
        const uint8_t* bufc = smem + (size_t)(sb >> 2) * STAGE;
        t.super_block(cur, bufc + arow + (sb & 3u) * 512u, reinterpret_cast<const float*>(bufc + XBUF) + (sb & 3u) * T::kSumsPerSb + 16u * g + j,
                      g, acc);
        if (++sb == nsb) {
            // lane (j, g): activation rows 4g .. 4g + 3 of weight row 16 grp + j; f32 activations: rows 8 .. 15 (HALF: 4 .. 7) are
            // the lo parts
            float o[4] = {acc[0], acc[1], acc[2], acc[3]};
            if constexpr (!X_BF16) {
#pragma unroll
                for (int v = 0; v < 4; ++v) o[v] = HALF ? xor16_add(o[v]) : xor32_add(o[v]);
            }
            const uint32_t row = grp * 16u + j;
            if (g < (HALF ? 1u : 2u) && row < a.n) {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (4u * g + v < a.m) a.y[(size_t)(4u * g + v) * a.n + row] = o[v];
            }
            acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
            sb = 0;
            grp += stride;
        }
    };
    for (uint32_t i = 0; i < ntask; i += 2) {
        task(wa, wb);
        if (i + 1 < ntask) task(wb, wa);
    }
}

}  // namespace

// Q4_K and Q5_K from three rows on, Q6_K from four: below that, one GEMV per row is as fast.  Measured, bf16 activations:
// Q4_K 12288 x 4096: 10 / 15 / 19 / 24 us for 1..4 GEMVs against 15..16 us here whatever the row count; Q6_K
// 151936 x 4096: 96 us per GEMV row against 310 us here.
bool gemv_rows_supported(hq_ggml_type t, uint32_t m, uint32_t k) {
    const uint32_t from = t == HQ_Q6_K ? 4u : 3u;
    return (t == HQ_Q4_K || t == HQ_Q5_K || t == HQ_Q6_K) && m >= from && m <= 8 && k % KC == 0;
}

namespace {
constexpr int kStreamWaves = 16;
constexpr size_t kLdsPerCu = 160 * 1024 - 512;
// Whether the stage-once form takes the product (all of k in LDS, two groups of 16 rows or more per CU), its LDS bytes,
// and whether the wave-owned piece buffers of the transposed fetch fit beside the activations.
// (bf: eight staged rows -- bf16 rows, or up to four f32 rows as hi and lo parts)
// min_groups8: groups of 16 rows per CU the matrix must have, in eighths (16 = two groups)
// waves12: sixteen staged rows (f32 activations) whose piece buffers fit for twelve waves only (k <= 3072 as f32)
bool rows_stream_plan(hq_ggml_type t, bool bf, uint32_t n, uint32_t k, uint32_t cus, size_t* lds, bool* xpose, uint32_t min_groups8 = 16u,
                      bool* waves12 = nullptr) {
    const size_t lds_all = (size_t)((k + KC - 1u) / KC) * (bf ? kStage<true> : kStage<false>);
    if (k % 256u || lds_all > kLdsPerCu || (uint64_t)((n + 15u) / 16u) * 8u < (uint64_t)min_groups8 * cus) return false;
    const size_t pitch16 = 16u * (t == HQ_Q4_K ? Q4kRows<false>::PITCH : t == HQ_Q5_K ? Q4kRows<true>::PITCH : t == HQ_Q6_K ? Q6kRows::PITCH : t == HQ_Q8_0 ? Q80Rows::PITCH : Q40Rows::PITCH);
    *xpose = lds_all + kStreamWaves * pitch16 <= kLdsPerCu;
    *lds = lds_all + (*xpose ? kStreamWaves * pitch16 : 0);
    if (waves12) {
        *waves12 = !bf && !*xpose && lds_all + 12u * pitch16 <= kLdsPerCu;
        if (*waves12) {
            *xpose = true;
            *lds = lds_all + 12u * pitch16;
        }
    }
    return true;
}
}  // namespace

// bf16 rows over a matrix the stage-once form takes with its transposed fetch: one pass for any 3 .. 8 rows at about the
// cost of one and a half one-row products (Q6_K 151936 x 4096: 134 us; Q4_K 65536 x 4096: 41 us).
bool gemv_rows_stream_fast(hq_ggml_type t, hq_act_dtype xdt, uint32_t m, uint32_t n, uint32_t k) {
    if (xdt != HQ_BF16 || m < 3 || m > 8 || (t != HQ_Q4_K && t != HQ_Q5_K && t != HQ_Q6_K)) return false;
    uint32_t cus = 0;
    if (cu_count(&cus)) return false;
    size_t lds = 0;
    bool xpose = false;
    return rows_stream_plan(t, true, n, k, cus, &lds, &xpose) && xpose;
}

// k that is whole super-blocks but not whole 1024-element chunks (2816, 3584, 5120 ...): only the stage-once form walks it,
// with either activation type.  Such k has no multi-row streaming passes either, so the form starts at three rows for
// every type (Q6_K 262144 x 2816 f32: 228 against 318 us), and at two where the weights go through the transposed fetch
// (bf16 rows: Q6_K 262144 x 2816 146 against 191 us for two passes, Q4_K 90 against 153, Q5_K 152064 x 3584 86 against 130).
// Small K-quant matrices whose k is not whole chunks have no other kernel that reads the weights once for all rows: from four
// rows on the stage-once form takes them down to an eighth of a group per CU (Q5_K 4096 x 2816: 11.5 us for 4 .. 8 rows against
// 17 / 33 us as a pass per row; 1024 x 2816: 11.4 against 12.2 / 24).
inline uint32_t rows_stream_min_groups8(hq_ggml_type t, uint32_t m, uint32_t k) {
    return (t == HQ_Q4_K || t == HQ_Q5_K || t == HQ_Q6_K) && k % KC != 0 && k > KC && m >= 4 ? 1u : 16u;  // (k < 1024: a pass per row is quick)
}

bool gemv_rows_stream_takes(hq_ggml_type t, hq_act_dtype xdt, uint32_t m, uint32_t n, uint32_t k) {
    if (m < 2 || m > 8 || (t != HQ_Q4_K && t != HQ_Q5_K && t != HQ_Q6_K && t != HQ_Q8_0 && t != HQ_Q4_0)) return false;
    uint32_t cus = 0;
    if (cu_count(&cus)) return false;
    size_t lds = 0;
    bool xpose = false, xpose_h = false;
    // up to four f32 rows as hi and lo parts in the space of eight bf16 rows, with the transposed fetch
    const uint32_t mg8 = rows_stream_min_groups8(t, m, k);
    const bool half = xdt != HQ_BF16 && m <= 4 && rows_stream_plan(t, true, n, k, cus, &lds, &xpose_h, mg8) && xpose_h;
    bool w12 = false;
    if (!rows_stream_plan(t, xdt == HQ_BF16, n, k, cus, &lds, &xpose, mg8, &w12) && !half) return false;
    // (five to eight f32 rows: the transposed fetch with twelve waves where sixteen staged rows leave room for that many piece
    // buffers -- k <= 3072: Q6_K 262144 x 2816 228 us without it, Q8_0 two passes of four rows 280)
    const bool fast = (xdt == HQ_BF16 && xpose) || half || w12;
    // Q8_0: where the transposed fetch fits, from two rows on (bf16, 262144 x 2816: 140 .. 150 us for 2 .. 8 rows where the
    // kernel of exact f32 products takes 237 .. 426 and one row 126; 12288 x 4096: 15.4 against 17.5 .. 30.0); without the
    // transposed fetch, and with five f32 rows or more (hi + lo parts: twice the LDS), that kernel stays ahead
    if (t == HQ_Q8_0) return fast && (xdt == HQ_BF16 || m >= 3 || n >= 32768);  // (two f32 rows, 12288 x 4096: 18.6 against 17.5 us)
    // Q4_0 likewise (262144 x 2816: 93 .. 96 us for 2 .. 8 rows, one row 91; 151936 x 4096: 78 .. 81, one row 58; that kernel: 112 ..
    // 259); two rows of a small matrix stay with it (12288 x 4096: 13.2 against 14.9 us; from three rows 16.6 .. 25.7 against 14.9)
    if (t == HQ_Q4_0) return fast && (m >= 3 || n >= 32768);
    // K-quants.  Whole chunks: from three rows (Q6_K with bf16 rows: four; below, one-row or multi-row streaming passes are as
    // fast), and from two f32 rows on large matrices (head 151936 x 4096: 128 us for 2 .. 4 rows against 158 for two passes, 240
    // for the sixteen-row staging; Q4_K 65536 x 4096: 35 against 57).  Other k: no streaming passes, from two rows on with the
    // transposed fetch, else three.
    const uint32_t from = k % KC == 0 ? (half ? (n >= 32768 ? 2u : 3u) : t == HQ_Q6_K ? 4u : 3u) : fast ? 2u : 3u;
    return m >= from;
}

int launch_gemv_rows(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m, uint32_t n,
                     uint32_t k, hq_ggml_type t) {
    RowsArgs a{x, static_cast<const uint8_t*>(w), y, m, n, k};
    const bool bf = xdt == HQ_BF16;
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    size_t lds_k = 0;
    bool xpose = false;
    const uint32_t mg8 = rows_stream_min_groups8(t, m, k);
    if (!bf && m <= 4 && rows_stream_plan(t, true, n, k, cus, &lds_k, &xpose, mg8) && xpose) {
        constexpr int W = kStreamWaves;
        void (*sk)(RowsArgs) = t == HQ_Q4_K   ? rows_stream_kernel<Q4kRows<false>, false, W, true, true>
                               : t == HQ_Q5_K ? rows_stream_kernel<Q4kRows<true>, false, W, true, true>
                               : t == HQ_Q6_K ? rows_stream_kernel<Q6kRows, false, W, true, true>
                               : t == HQ_Q8_0 ? rows_stream_kernel<Q80Rows, false, W, true, true>
                                              : rows_stream_kernel<Q40Rows, false, W, true, true>;
        if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(sk), lds_k, "hipFuncSetAttribute(rows stream kernel LDS)")) return rc;
        hipLaunchKernelGGL(sk, dim3(cus), dim3(64 * W), lds_k, s, a);
        return check_launch("rows stream kernel launch");
    }
    bool w12 = false;
    if (rows_stream_plan(t, bf, n, k, cus, &lds_k, &xpose, mg8, &w12) && w12) {
        void (*sk)(RowsArgs) = t == HQ_Q4_K   ? rows_stream_kernel<Q4kRows<false>, false, 12, true>
                               : t == HQ_Q5_K ? rows_stream_kernel<Q4kRows<true>, false, 12, true>
                               : t == HQ_Q6_K ? rows_stream_kernel<Q6kRows, false, 12, true>
                               : t == HQ_Q8_0 ? rows_stream_kernel<Q80Rows, false, 12, true>
                                              : rows_stream_kernel<Q40Rows, false, 12, true>;
        if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(sk), lds_k, "hipFuncSetAttribute(rows stream kernel LDS)")) return rc;
        hipLaunchKernelGGL(sk, dim3(cus), dim3(64 * 12), lds_k, s, a);
        return check_launch("rows stream kernel launch");
    }
    if (rows_stream_plan(t, bf, n, k, cus, &lds_k, &xpose, mg8)) {
        constexpr int W = kStreamWaves;
        void (*sk)(RowsArgs);
        if (xpose)
            sk = t == HQ_Q4_K   ? (bf ? rows_stream_kernel<Q4kRows<false>, true, W, true> : rows_stream_kernel<Q4kRows<false>, false, W, true>)
                 : t == HQ_Q5_K ? (bf ? rows_stream_kernel<Q4kRows<true>, true, W, true> : rows_stream_kernel<Q4kRows<true>, false, W, true>)
                 : t == HQ_Q6_K ? (bf ? rows_stream_kernel<Q6kRows, true, W, true> : rows_stream_kernel<Q6kRows, false, W, true>)
                 : t == HQ_Q8_0 ? (bf ? rows_stream_kernel<Q80Rows, true, W, true> : rows_stream_kernel<Q80Rows, false, W, true>)
                                : (bf ? rows_stream_kernel<Q40Rows, true, W, true> : rows_stream_kernel<Q40Rows, false, W, true>);
        else
            sk = t == HQ_Q4_K   ? (bf ? rows_stream_kernel<Q4kRows<false>, true, W, false> : rows_stream_kernel<Q4kRows<false>, false, W, false>)
                 : t == HQ_Q5_K ? (bf ? rows_stream_kernel<Q4kRows<true>, true, W, false> : rows_stream_kernel<Q4kRows<true>, false, W, false>)
                 : t == HQ_Q6_K ? (bf ? rows_stream_kernel<Q6kRows, true, W, false> : rows_stream_kernel<Q6kRows, false, W, false>)
                 : t == HQ_Q8_0 ? (bf ? rows_stream_kernel<Q80Rows, true, W, false> : rows_stream_kernel<Q80Rows, false, W, false>)
                                : (bf ? rows_stream_kernel<Q40Rows, true, W, false> : rows_stream_kernel<Q40Rows, false, W, false>);
        if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(sk), lds_k, "hipFuncSetAttribute(rows stream kernel LDS)")) return rc;
        hipLaunchKernelGGL(sk, dim3(cus), dim3(64 * W), lds_k, s, a);
        return check_launch("rows stream kernel launch");
    }
    if (k % KC || t == HQ_Q8_0 || t == HQ_Q4_0) return fail(HQ_ERR_INVALID_ARGUMENT, "small-batch kernel: k must be a multiple of 1024 for this matrix");
    const int lds = 2 * (bf ? kStage<true> : kStage<false>);
    // more rows per workgroup once that still gives every CU three workgroups of the first round; Q6_K stops at
    // two super-blocks per wave (at four, the fetches in flight leave one wave per SIMD) except with f32
    // activations, whose LDS footprint limits the CU to two workgroups anyway
    const uint32_t nsb = n < WIDE_MIN_ROWS ? 1u : t != HQ_Q6_K || !bf ? 4u : 2u;
    void (*kern)(RowsArgs);
    if (t == HQ_Q4_K)
        kern = nsb == 4 ? (bf ? q4k_rows_kernel<true, 4> : q4k_rows_kernel<false, 4>)
                        : (bf ? q4k_rows_kernel<true, 1> : q4k_rows_kernel<false, 1>);
    else if (t == HQ_Q5_K)
        kern = nsb == 4 ? (bf ? q4k_rows_kernel<true, 4, true> : q4k_rows_kernel<false, 4, true>)
                        : (bf ? q4k_rows_kernel<true, 1, true> : q4k_rows_kernel<false, 1, true>);
    else
        kern = nsb == 4 ? q6k_rows_kernel<false, 4>
               : nsb == 2 ? q6k_rows_kernel<true, 2>
                          : (bf ? q6k_rows_kernel<true, 1> : q6k_rows_kernel<false, 1>);
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), (size_t)lds, "hipFuncSetAttribute(rows kernel LDS)"))
        return rc;
    const uint32_t rows_per_wg = 16u * nsb;
    hipLaunchKernelGGL(kern, dim3((n + rows_per_wg - 1u) / rows_per_wg), dim3(256), lds, s, a);
    return check_launch("rows kernel launch");
}

}  // namespace hq

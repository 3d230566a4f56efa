// Batched-prefill quantized GEMM (m > 8): y[m,n] = x[m,k] . W[n,k]^T with W in
// GGML Q4_K / Q8_0 blocks, on the bf16 matrix cores with fp32 accumulation.
//
// Rounding a dequantised weight to bf16 would cost ~1e-3 relative error per
// product, so the tiles that feed the MFMA hold only values bf16 represents
// EXACTLY, and the block scales are applied in fp32:
//   Q4_K  w = d*sc*q - dmin*mn, sc / mn the 6-bit codes of a 32-element sub-block.
//         The LDS weight tile holds (128+q) (one and/or against the bf16 magic
//         0x4300), the activation tile holds x (bf16, or an exact hi+lo split of
//         f32).  Per sub-block P = sum_k x*(128+q) comes from two
//         v_mfma_f32_32x32x16_bf16 into a scratch accumulator and
//         acc += (d*sc)[n]*P on the VALU (one FMA per output per 32 k).  What is
//         left,  -sum_sb (128*d*sc + dmin*mn)[n,sb] * S[m,sb]  with S the
//         sub-block sums of x, is two more contractions over the 8 sub-blocks of
//         a super-block, T = sum_sb sc*S and U = sum_sb mn*S, that run on the
//         MFMA as well: sc and mn are small integers (exact in bf16) and S is
//         split three ways (hi+mid+lo, exact to 2^-25; the 128 would amplify a
//         coarser split).  Then acc -= 128*d[n]*T + dmin[n]*U, once per super-block.
//   Q8_0  w = d*q, q int8 (exact in bf16): P per 32-element block, acc += d[n]*P.
// So every product inside the MFMA is exact and all rounding happens in fp32
// accumulation, like the GEMV path.
//
// Tiling: workgroup = 256 threads = 2x2 waves; tile 256 (tokens) x 128 (weight
// rows) x 64 (k); a wave owns 128x64 = 4x2 MFMA tiles (128 accumulator
// registers).  Weights are unpacked once per workgroup into LDS and re-used by
// the 256 token rows; LDS rows are padded to 144 bytes so the 16-byte fragment
// reads are bank-conflict free.  Activations go to LDS as they are; the
// unpacked nibble pairs come out of the masked shifts as (e0,e2),(e1,e3) and
// one v_perm per word restores k order.
#include "hq_internal.h"

namespace hq {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int BN = 128, BK = 64;  // BM (token rows per workgroup) is a template parameter: 256 or 128
constexpr int LDS_ROW = BK + 8;  // bf16 elements per padded tile row (144 bytes)

struct GemmArgs {
    const void* x;
    const uint8_t* w;
    float* y;
    uint32_t m, n, k;
};

__device__ __forceinline__ bf16x8_t as_frag(uint4 v) { return __builtin_bit_cast(bf16x8_t, v); }

// hi = bf16(x) (round to nearest even), lo = bf16(x - hi): hi + lo reproduces x to 2^-17.
__device__ __forceinline__ void split_bf16(float x, uint32_t& hi, uint32_t& lo) {
    hi = f32_to_bf16_bits(x);
    lo = f32_to_bf16_bits(x - bf16_bits_to_f32(hi));
}

// Round-to-nearest-even bf16 bits of a finite value (no NaN special case).
__device__ __forceinline__ uint32_t bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
    return v + __int_as_float(t);
}

// LDS carve-up (bytes).  A_lo only exists for f32 activations.
template <bool X_BF16, int BM>
struct Lds {
    static constexpr int kA = 0;
    static constexpr int kAlo = kA + BM * LDS_ROW * 2;
    static constexpr int kB = X_BF16 ? kAlo : kAlo + BM * LDS_ROW * 2;
    static constexpr int kDsc = kB + BN * LDS_ROW * 2;   // [BN][2] f32: scales of this stage's two groups
    static constexpr int kS = kDsc + BN * 2 * 4;         // [BM][8] f32: sub-block sums of x over the super-block
    static constexpr int kSC = kS + BM * 8 * 4;          // [BN][16] bf16: (sc[8], sc[8])
    static constexpr int kMN = kSC + BN * 16 * 2;        // [BN][16] bf16: (mn[8], mn[8])
    static constexpr int kDD = kMN + BN * 16 * 2;        // [BN][2]  f32: (-128*d, -dmin)
    static constexpr int kTotal = kDD + BN * 2 * 4;
};

// Global-memory operands of one stage, fetched one stage ahead of their use so that the
// loads are in flight while the previous stage's tiles are being multiplied.
template <int TYPE, bool X_BF16, int BM>
struct StageRegs {
    uint4 a[(X_BF16 ? 1 : 2) * (BM / 32)];  // 8 chunks of 8 activations (bf16: 16 bytes, f32: 32 bytes each)
    uint4 b0, b1;              // Q4_K: 16 nibble bytes (b0) + block header (b1); Q8_0: the 32 int8
    uint32_t d;                // Q8_0: f16 scale bits
};

template <int TYPE, bool X_BF16, int BM>
__device__ __forceinline__ void load_stage(const GemmArgs& a, uint32_t st, uint32_t m0, uint32_t n0,
                                           uint32_t row_bytes, StageRegs<TYPE, X_BF16, BM>& r) {
    const uint32_t tid = threadIdx.x, k0 = st * BK;
#pragma unroll
    for (int i = 0; i < BM / 32; ++i) {
        const uint32_t row = (tid >> 3) + 32u * i, c8 = tid & 7u;
        uint32_t gm = m0 + row;
        gm = gm < a.m ? gm : a.m - 1u;  // rows past the end are zeroed when they are written to LDS
        if constexpr (X_BF16) {
            r.a[i] = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(a.x) + (size_t)gm * a.k + k0 + 8 * c8);
        } else {
            const uint4* p = reinterpret_cast<const uint4*>(static_cast<const float*>(a.x) + (size_t)gm * a.k + k0 + 8 * c8);
            r.a[2 * i] = p[0];
            r.a[2 * i + 1] = p[1];
        }
    }
    const uint32_t row = tid >> 1, h = tid & 1u;
    uint32_t gn = n0 + row;
    gn = gn < a.n ? gn : a.n - 1u;
    const uint8_t* rp = a.w + (size_t)gn * row_bytes;
    if constexpr (TYPE == HQ_Q4_K) {
        const uint8_t* blk = rp + (size_t)(k0 >> 8) * Q4K_BYTES;
        r.b0 = *reinterpret_cast<const uint4*>(blk + 16 + 32 * (st & 3u) + 16 * h);
        r.b1 = *reinterpret_cast<const uint4*>(blk);
    } else {
        const uint8_t* blk = rp + (size_t)((k0 >> 5) + h) * Q8_0_BYTES;
        r.b0 = ld16_unaligned(blk + 2);
        r.b1 = ld16_unaligned(blk + 18);
        r.d = ld2(blk);
    }
}

template <int TYPE, bool X_BF16, int BM>
__global__ __launch_bounds__(256, 2) void gemm_kernel(GemmArgs a) {
    extern __shared__ uint4 smem4[];
    uint8_t* smem = reinterpret_cast<uint8_t*>(smem4);
    using L = Lds<X_BF16, BM>;
    constexpr int MT = BM / 64;   // 32-row MFMA tiles per wave (a wave owns BM/2 x 64)
    constexpr int NCH = BM / 32;  // 8-activation chunks staged per thread
    constexpr bool Q4 = TYPE == HQ_Q4_K;
    constexpr int NA = X_BF16 ? 1 : 2;  // activation tiles (hi, lo)

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    // Tile order.  Workgroups are handed to the 8 XCDs round-robin and every XCD has its own L2, so
    // workgroup L runs on XCD L % 8.  Give each XCD whole rows of tiles (same activation tile, the
    // 2 MB of which then stay in that XCD's 4 MB L2) and let it sweep the weight tiles.
    const uint32_t tiles_n = (a.n + BN - 1) / BN, tiles_m = (a.m + BM - 1) / BM;
    uint32_t tm, tn;
    {
        const uint32_t Lw = blockIdx.x, xcd = Lw & 7u, idx = Lw >> 3;
        const uint32_t rows_here = (tiles_m + 7u - xcd) / 8u;  // tile rows r with r % 8 == xcd
        if (idx >= rows_here * tiles_n) return;                // the grid is padded to 8 * ceil(tiles_m/8) * tiles_n
        tm = xcd + 8u * (idx / tiles_n);
        tn = idx % tiles_n;
    }
    const uint32_t m0 = tm * BM, n0 = tn * BN;
    const uint32_t l32 = lane & 31u, lg = lane >> 5;

    f32x16_t acc[MT][2];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const uint32_t nstages = a.k / BK;
    const uint32_t row_bytes = Q4 ? (a.k / 256) * Q4K_BYTES : (a.k / 32) * Q8_0_BYTES;

    StageRegs<TYPE, X_BF16, BM> regs;
    load_stage<TYPE, X_BF16, BM>(a, 0, m0, n0, row_bytes, regs);

    // Q4_K: an outer iteration is one super-block (4 stages of 64 k) followed by its offset / min
    // contraction; Q8_0: one stage per outer iteration.
    constexpr uint32_t SPO = Q4 ? 4 : 1;
    for (uint32_t so = 0; so < nstages; so += SPO) {
#pragma unroll 1
        for (uint32_t st = so; st < so + SPO; ++st) {
            // ---------------- registers -> LDS: activations, BM rows x 64 k in chunks of 8 ----------------
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const uint32_t row = (tid >> 3) + 32u * i, c8 = tid & 7u;
                uint4 hi, lo = make_uint4(0, 0, 0, 0);
                if constexpr (X_BF16) {
                    hi = regs.a[i];
                } else {
                    const uint4 u0 = regs.a[2 * i], u1 = regs.a[2 * i + 1];
                    const uint32_t e[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
                    uint32_t h[8], l[8];
#pragma unroll
                    for (int q = 0; q < 8; ++q) split_bf16(__uint_as_float(e[q]), h[q], l[q]);
                    hi = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
                    lo = make_uint4(l[0] | (l[1] << 16), l[2] | (l[3] << 16), l[4] | (l[5] << 16), l[6] | (l[7] << 16));
                }
                if (m0 + row >= a.m) hi = lo = make_uint4(0, 0, 0, 0);
                *reinterpret_cast<uint4*>(smem + L::kA + (row * LDS_ROW + 8 * c8) * 2) = hi;
                if constexpr (!X_BF16) *reinterpret_cast<uint4*>(smem + L::kAlo + (row * LDS_ROW + 8 * c8) * 2) = lo;
                if constexpr (Q4) {
                    // Sum of the 8 activations exactly as the MFMA sees them (dot with ones), then over
                    // the sub-block: chunks 0..3 and 4..7 of a row sit in one quad each.
                    constexpr uint32_t ONES = 0x3f803f80u;
                    float s = dot2_bf16(hi.x, ONES, dot2_bf16(hi.y, ONES, dot2_bf16(hi.z, ONES, dot2_bf16(hi.w, ONES, 0.f))));
                    if constexpr (!X_BF16)
                        s = dot2_bf16(lo.x, ONES, dot2_bf16(lo.y, ONES, dot2_bf16(lo.z, ONES, dot2_bf16(lo.w, ONES, s))));
                    s = dpp_add<0xB1>(s);
                    s = dpp_add<0x4E>(s);
                    if ((c8 & 3u) == 0) reinterpret_cast<float*>(smem + L::kS)[row * 8 + 2 * (st & 3u) + (c8 >> 2)] = s;
                }
            }
            // ---------------- registers -> LDS: weights, 128 rows x 64 k ----------------
            {
                const uint32_t row = tid >> 1, h = tid & 1u;
                uint8_t* brow = smem + L::kB + row * LDS_ROW * 2;
                if constexpr (Q4) {
                    const uint32_t c = st & 3u;  // 64-element chunk of the super-block
                    const uint32_t w[4] = {regs.b0.x, regs.b0.y, regs.b0.z, regs.b0.w};
                    uint32_t lo[8], hi[8];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        // a masked shift yields the pairs (e0,e2) and (e1,e3); v_perm puts them back in k order
                        const uint32_t a02 = (w[j] & 0x000f000fu) | 0x43004300u;
                        const uint32_t a13 = ((w[j] >> 8) & 0x000f000fu) | 0x43004300u;
                        const uint32_t b02 = ((w[j] >> 4) & 0x000f000fu) | 0x43004300u;
                        const uint32_t b13 = ((w[j] >> 12) & 0x000f000fu) | 0x43004300u;
                        lo[2 * j] = __builtin_amdgcn_perm(a13, a02, 0x05040100u);      // (e0, e1)
                        lo[2 * j + 1] = __builtin_amdgcn_perm(a13, a02, 0x07060302u);  // (e2, e3)
                        hi[2 * j] = __builtin_amdgcn_perm(b13, b02, 0x05040100u);
                        hi[2 * j + 1] = __builtin_amdgcn_perm(b13, b02, 0x07060302u);
                    }
                    uint4* d0 = reinterpret_cast<uint4*>(brow + (16 * h) * 2);
                    d0[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                    d0[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
                    uint4* d1 = reinterpret_cast<uint4*>(brow + (32 + 16 * h) * 2);
                    d1[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
                    d1[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
                    if (h == 0) {
                        const uint4 hdr = regs.b1;
                        uint32_t sc0, sc1, mn0, mn1;
                        q4k_scales(hdr.y, hdr.z, hdr.w, (int)c, sc0, sc1, mn0, mn1);
                        const float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
                        float* dsc = reinterpret_cast<float*>(smem + L::kDsc) + row * 2;
                        dsc[0] = d * (float)sc0;
                        dsc[1] = d * (float)sc1;
                        // integer codes as bf16 (exact) for the T / U contractions
                        const uint32_t b0 = __float_as_uint((float)sc0) >> 16, b1 = __float_as_uint((float)sc1) >> 16;
                        const uint32_t c0 = __float_as_uint((float)mn0) >> 16, c1 = __float_as_uint((float)mn1) >> 16;
                        uint32_t* SC = reinterpret_cast<uint32_t*>(smem + L::kSC + row * 32);
                        uint32_t* MN = reinterpret_cast<uint32_t*>(smem + L::kMN + row * 32);
                        SC[c] = SC[4 + c] = b0 | (b1 << 16);  // slots 2c, 2c+1 and 8+2c, 8+2c+1
                        MN[c] = MN[4 + c] = c0 | (c1 << 16);
                        if (c == 0) {
                            float* dd = reinterpret_cast<float*>(smem + L::kDD) + row * 2;
                            dd[0] = -128.f * d;  // the weight tile holds 128+q
                            dd[1] = -dmin;
                        }
                    }
                } else {
                    // Q8_0: this thread converts block h (32 int8) of the row's two blocks in the stage
                    const uint32_t w[8] = {regs.b0.x, regs.b0.y, regs.b0.z, regs.b0.w,
                                           regs.b1.x, regs.b1.y, regs.b1.z, regs.b1.w};
                    uint32_t o[16];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        // an int8 is exact in bf16: take the top half of its f32 image
                        const uint32_t e0 = __float_as_uint(sbyte(w[j], 0)), e1 = __float_as_uint(sbyte(w[j], 1));
                        const uint32_t e2 = __float_as_uint(sbyte(w[j], 2)), e3 = __float_as_uint(sbyte(w[j], 3));
                        o[2 * j] = (e0 >> 16) | (e1 & 0xffff0000u);
                        o[2 * j + 1] = (e2 >> 16) | (e3 & 0xffff0000u);
                    }
                    uint4* dq = reinterpret_cast<uint4*>(brow + (32 * h) * 2);
#pragma unroll
                    for (int j = 0; j < 4; ++j) dq[j] = make_uint4(o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]);
                    reinterpret_cast<float*>(smem + L::kDsc)[row * 2 + h] = f16_bits_to_f32(regs.d);
                }
            }
            __syncthreads();

            // next stage's operands start their trip from L2 / HBM now
            if (st + 1 < nstages) load_stage<TYPE, X_BF16, BM>(a, st + 1, m0, n0, row_bytes, regs);

            // ---------------- MFMA over the stage's two scale groups ----------------
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                bf16x8_t bf[2][2];
                float dsc[2];
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    const uint32_t brow = wn * 64 + nt * 32 + l32;
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
                        bf[nt][ks] = as_frag(*reinterpret_cast<const uint4*>(
                            smem + L::kB + (brow * LDS_ROW + 32 * g + 16 * ks + 8 * lg) * 2));
                    dsc[nt] = reinterpret_cast<const float*>(smem + L::kDsc)[brow * 2 + g];
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const uint32_t arow = wm * (BM / 2) + mt * 32 + l32;
                    bf16x8_t af[NA][2];
#pragma unroll
                    for (int t = 0; t < NA; ++t)
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks)
                            af[t][ks] = as_frag(*reinterpret_cast<const uint4*>(
                                smem + (t == 0 ? L::kA : L::kAlo) + (arow * LDS_ROW + 32 * g + 16 * ks + 8 * lg) * 2));
#pragma unroll
                    for (int nt = 0; nt < 2; ++nt) {
                        f32x16_t p;
#pragma unroll
                        for (int v = 0; v < 16; ++v) p[v] = 0.f;
#pragma unroll
                        for (int t = 0; t < NA; ++t)
#pragma unroll
                            for (int ks = 0; ks < 2; ++ks)
                                p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[t][ks], bf[nt][ks], p, 0, 0, 0);
#pragma unroll
                        for (int v = 0; v < 16; ++v) acc[mt][nt][v] = fmaf(p[v], dsc[nt], acc[mt][nt][v]);
                    }
                }
            }
            __syncthreads();  // every wave is done with the tiles before the next stage overwrites them
        }

        // ---------------- Q4_K: offset and min terms once per super-block ----------------
        if constexpr (Q4) {
            const uint4 zero4 = make_uint4(0, 0, 0, 0);
            bf16x8_t scf[2], sc0f[2], mnf[2];
            float d128[2], dmn[2];
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                const uint32_t brow = wn * 64 + nt * 32 + l32;
                scf[nt] = as_frag(*reinterpret_cast<const uint4*>(smem + L::kSC + brow * 32 + 16 * lg));
                // (sc[8], 0[8]): the upper lane group contributes nothing
                sc0f[nt] = as_frag(lg ? zero4 : *reinterpret_cast<const uint4*>(smem + L::kSC + brow * 32));
                mnf[nt] = as_frag(*reinterpret_cast<const uint4*>(smem + L::kMN + brow * 32 + 16 * lg));
                d128[nt] = reinterpret_cast<const float*>(smem + L::kDD)[brow * 2];
                dmn[nt] = reinterpret_cast<const float*>(smem + L::kDD)[brow * 2 + 1];
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint32_t arow = wm * (BM / 2) + mt * 32 + l32;
                // S = hi + mid + lo exactly (3 x 8 significant bits).  Lane group 0 feeds k slots 0..7
                // = S_hi (first operand) / S_lo (second), lane group 1 feeds slots 8..15 = S_mid / 0.
                const float4* Sp = reinterpret_cast<const float4*>(smem + L::kS + arow * 32);
                const float4 s0 = Sp[0], s1 = Sp[1];
                const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
                uint32_t fa[8], fb[8];
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const uint32_t sh = bf16_rne(sv[q]);
                    const float r1 = sv[q] - bf16_bits_to_f32(sh);
                    const uint32_t sm = bf16_rne(r1);
                    const uint32_t sl = bf16_rne(r1 - bf16_bits_to_f32(sm));
                    fa[q] = lg ? sm : sh;
                    fb[q] = lg ? 0u : sl;
                }
                const bf16x8_t sa = as_frag(make_uint4(fa[0] | (fa[1] << 16), fa[2] | (fa[3] << 16),
                                                       fa[4] | (fa[5] << 16), fa[6] | (fa[7] << 16)));
                const bf16x8_t sb = as_frag(make_uint4(fb[0] | (fb[1] << 16), fb[2] | (fb[3] << 16),
                                                       fb[4] | (fb[5] << 16), fb[6] | (fb[7] << 16)));
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    f32x16_t t;
#pragma unroll
                    for (int v = 0; v < 16; ++v) t[v] = 0.f;
                    t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(sa, scf[nt], t, 0, 0, 0);   // sc*(S_hi+S_mid)
                    t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(sb, sc0f[nt], t, 0, 0, 0);  // sc*S_lo
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[mt][nt][v] = fmaf(t[v], d128[nt], acc[mt][nt][v]);
#pragma unroll
                    for (int v = 0; v < 16; ++v) t[v] = 0.f;
                    t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(sa, mnf[nt], t, 0, 0, 0);   // mn*(S_hi+S_mid)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[mt][nt][v] = fmaf(t[v], dmn[nt], acc[mt][nt][v]);
                }
            }
            __syncthreads();  // the next super-block's staging rewrites the S / code arrays
        }
    }

    // ---------------- store: value v of a lane is row 8*(v/4) + 4*(lane/32) + v%4, column lane%32 ----------------
    const uint32_t N = a.n;
    const bool full = m0 + BM <= a.m && n0 + BN <= a.n;  // uniform: the whole tile is inside y
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
            const uint32_t gn = n0 + wn * 64 + nt * 32 + l32;
            const uint32_t gmb = m0 + wm * (BM / 2) + mt * 32 + 4 * lg;
            float* yp = a.y + (size_t)gmb * N + gn;
            if (full) {
#pragma unroll
                for (int v = 0; v < 16; ++v) yp[(size_t)((8 * (v >> 2) + (v & 3)) * N)] = acc[mt][nt][v];
            } else if (gn < a.n) {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (gmb + 8 * (v >> 2) + (v & 3) < a.m) yp[(size_t)((8 * (v >> 2) + (v & 3)) * N)] = acc[mt][nt][v];
            }
        }
}

template <int TYPE, bool X_BF16, int BM>
int launch_t(hipStream_t s, const GemmArgs& a) {
    auto kern = gemm_kernel<TYPE, X_BF16, BM>;
    constexpr int lds = Lds<X_BF16, BM>::kTotal;
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), (size_t)lds, "hipFuncSetAttribute(gemm LDS)"))
        return rc;
    const uint32_t tiles_n = (a.n + BN - 1) / BN, tiles_m = (a.m + BM - 1) / BM;
    const dim3 grid(8u * ((tiles_m + 7u) / 8u) * tiles_n);  // see the tile order in the kernel
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, a);
    return check_launch("gemm kernel launch");
}

}  // namespace

bool gemm_supported(hq_ggml_type t, uint32_t k) {
    return (t == HQ_Q4_K && k % 256 == 0) || (t == HQ_Q8_0 && k % BK == 0);
}

int launch_gemm(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m, uint32_t n,
                uint32_t k, hq_ggml_type t) {
    GemmArgs a{x, static_cast<const uint8_t*>(w), y, m, n, k};
    const bool bf = xdt == HQ_BF16;
    // Q4_K carries the extra sub-block-sum state, so it runs 128-row tiles (64 accumulator registers
    // per lane); Q8_0 has the registers for 256-row tiles.
    if (t == HQ_Q4_K) return bf ? launch_t<HQ_Q4_K, true, 128>(s, a) : launch_t<HQ_Q4_K, false, 128>(s, a);
    if (t == HQ_Q8_0) return bf ? launch_t<HQ_Q8_0, true, 256>(s, a) : launch_t<HQ_Q8_0, false, 128>(s, a);
    return fail(HQ_ERR_UNSUPPORTED, "gemm: ggml type %d", (int)t);
}

}  // namespace hq

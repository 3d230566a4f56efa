// Batched-prefill GEMM for Q4_K, Q6_K and Q8_0 weights (m > 8): y[m,n] = x[m,k] . W[n,k]^T on the
// f16 matrix cores (v_mfma_f32_32x32x16_f16) with fp32 accumulation.
//
// Numerics.  The weight tile holds the dequantised weights rounded to f16, which
// is what the reference's mul_mm kernels multiply as well (their weight tile is
// simdgroup_half8x8): w = d*sc*q - dmin*mn is formed in fp32 (exact up to one
// rounding) and rounded once to f16, a relative error of at most 2^-12 per
// weight.  The activations are f16 too.  f16 has a narrow exponent range, so a
// pre-pass rescales every activation row by a power of two that brings its
// largest magnitude into [512, 1024) and the epilogue scales back: bf16
// activations are represented exactly (8-bit significands; values more than
// 2^-34 below the row maximum lose bits, far under fp32 resolution of the
// result), f32 activations are rounded to 11 bits.  Products are exact in the
// MFMA and accumulate in fp32.  Weight rows get a power-of-two scale of their own
// (from the row's largest super-block scale) for the same reason.  The result
// agrees with an f64 product over the
// exact weights to about 1.5e-4 of the output's scale (rms), where the kernels
// that keep every product exact reach 1e-6.
//
// Structure.  Workgroup = 256 threads = 4 waves side by side along the weight
// rows, tile 256 (tokens) x 128 (weight rows) x 64 (k) per stage; a wave owns
// all 256 tokens x 32 weight rows = 8x1 MFMA tiles (128 accumulator
// registers).  Two workgroups fit a CU.  The SIMD issues MFMA and VALU
// instructions through one port and an MFMA hides only about four VALU
// instructions behind it, so the kernel is bound by instructions per MFMA, not
// by latency: with tall wave tiles every weight is dequantised by exactly one
// wave of the workgroup (a 2x2 wave grid does it twice, 7.4 instead of 3.7
// VALU instructions per MFMA) at the price of twice the LDS reads, which the
// LDS (64 banks, 256 bytes per clock) has room for.  Problems of less than half
// a round of workgroups use tiles of 64 weight rows (2x2 waves of 128x32) to
// spread over more CUs.
//   * Activations: the pre-pass output goes global -> LDS directly
//     (global_load_lds_dwordx4, no registers, no VALU), double buffered, one
//     barrier per stage.  A wave instruction fills 1 KB of LDS with lane i at
//     byte 16*i, so tile rows are 128 bytes without padding and the 16-byte
//     chunks of a row are XOR-swizzled with the row number.  LDS has 64 banks
//     and serves a 16-byte read of 16 lanes per cycle, so the 16 rows that 16
//     consecutive lanes read must land in 16 different 16-byte slots of 256
//     bytes: the key is (row / 2) % 8 (rows of equal parity share a half).
//   * Weights never touch LDS: a lane fetches the 16 nibble bytes it needs for
//     its own fragments (row lane%32, bytes 16*(lane/32).. of the 64-element
//     chunk) straight from global memory, a stage ahead, and dequantises them
//     in registers: no LDS traffic, no extra barrier, and each wave produces
//     exactly the fragments it consumes.
//   * k order.  Inside a stage the MFMA contraction index is a permutation of k
//     chosen so that a lane's fragments come from its own 16 nibble bytes: lane
//     group g of k-step s covers k = 16g + 8s + j (s < 2, low nibbles) or
//     32 + 16g + 8(s-2) + j (high nibbles); for the activations that is only
//     the address of the fragment.
#include <type_traits>

#include "hq_internal.h"

namespace hq {
namespace {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int BK = 64;
constexpr int ROW = BK;  // f16 elements per LDS tile row (128 bytes, chunks XOR-swizzled)

// workspace: [xh m*k f16][rs m f32][wdown n f32]
struct Workspace {
    size_t xh, rs, wdown, total;
};
__host__ __device__ inline Workspace workspace_layout(uint32_t m, uint32_t n, uint32_t k) {
    Workspace w;
    w.xh = 0;
    w.rs = ((size_t)m * k * 2 + 255) & ~(size_t)255;
    w.wdown = w.rs + (((size_t)m * 4 + 255) & ~(size_t)255);
    w.total = w.wdown + (((size_t)n * 4 + 255) & ~(size_t)255);
    return w;
}

template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
    return fmaxf(v, __int_as_float(t));
}

__device__ __forceinline__ uint32_t f16_bits(float v) {
    return (uint32_t)__builtin_bit_cast(unsigned short, (_Float16)v);
}

// Largest possible |w| of the blocks first, first + step, ... (< count) of a weight row, from their scales alone
// (Q4_K: |d|*63*15 + |dmin|*63, Q5_K: |d|*63*31 + |dmin|*63, Q6_K: |d|*128*32, Q8_0: |d|*128, Q4_0: |d|*8); blocks are
// the type's own (super-blocks of 256 for the K-quants, blocks of 32 otherwise).  inf / nan scales do not count.
template <int TYPE>
__device__ __forceinline__ float weight_row_bound(const uint8_t* wrow, uint32_t k, uint32_t first, uint32_t step) {
    float bound = 0.f;
    if constexpr (TYPE == HQ_Q4_K || TYPE == HQ_Q5_K) {
        constexpr uint32_t BYTES = TYPE == HQ_Q5_K ? Q5K_BYTES : Q4K_BYTES;
        constexpr float DQ = TYPE == HQ_Q5_K ? 1953.f : 945.f;
        for (uint32_t sb = first; sb < k / 256; sb += step) {
            const uint32_t dd = *reinterpret_cast<const uint32_t*>(wrow + (size_t)sb * BYTES);
            const float b = fabsf(f16_bits_to_f32(dd & 0xffffu)) * DQ + fabsf(f16_bits_to_f32(dd >> 16)) * 63.f;
            bound = b <= 3.0e38f ? fmaxf(bound, b) : bound;
        }
    } else if constexpr (TYPE == HQ_Q6_K) {
        for (uint32_t sb = first; sb < k / 256; sb += step) {
            const float v = fabsf(f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(wrow + (size_t)sb * Q6K_BYTES + 208))) * 4096.f;
            bound = v <= 3.0e38f ? fmaxf(bound, v) : bound;
        }
    } else {
        constexpr uint32_t BYTES = TYPE == HQ_Q4_0 ? Q4_0_BYTES : Q8_0_BYTES;
        constexpr float QMAX = TYPE == HQ_Q4_0 ? 8.f : 128.f;
        for (uint32_t b = first; b < k / 32; b += step) {
            const float v = fabsf(f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(wrow + (size_t)b * BYTES))) * QMAX;
            bound = v <= 3.0e38f ? fmaxf(bound, v) : bound;
        }
    }
    return bound;
}
// The power of two 2^-e that brings a row whose largest possible |w| is `bound` to about 2^14.
__device__ __forceinline__ float weight_row_scale(float bound) {
    int ex = 0;
    if (bound > 0.f) (void)frexpf(bound, &ex);  // bound = f * 2^ex, f in [0.5, 1)
    return ldexpf(1.f, -(bound > 0.f ? ex - 14 : 0));  // |e| <= 40: normal
}

// Lanes that share one weight row in the scan of the block headers: a power of two, at most 16 and no more than the
// row has blocks (a row of two super-blocks under 16 lanes would leave 14 of them idle).
template <int TYPE>
__host__ __device__ __forceinline__ uint32_t weight_scan_lanes(uint32_t k) {
    const uint32_t blocks = k / ((TYPE == HQ_Q8_0 || TYPE == HQ_Q4_0) ? 32u : 256u);
    uint32_t lanes = 16u;
    while (lanes > 1u && lanes / 2u >= blocks) lanes /= 2u;
    return lanes;
}

// One group of 256 threads (t = thread within the group): the scales of 256 / lanes weight rows from first_row on,
// `lanes` = weight_scan_lanes(k) lanes per row over the row's block headers.
template <int TYPE>
__device__ __forceinline__ void prep_weight_rows(const uint8_t* __restrict__ w, float* __restrict__ scales, uint32_t n,
                                                 uint32_t k, uint32_t first_row, uint32_t t, uint32_t lanes) {
    const uint32_t wr = first_row + t / lanes, sub = t & (lanes - 1u);
    constexpr uint32_t BLOCK = TYPE == HQ_Q4_K ? Q4K_BYTES : TYPE == HQ_Q5_K ? Q5K_BYTES : TYPE == HQ_Q6_K ? Q6K_BYTES
                               : TYPE == HQ_Q4_0 ? Q4_0_BYTES : Q8_0_BYTES;
    constexpr uint32_t PER = (TYPE == HQ_Q8_0 || TYPE == HQ_Q4_0) ? 32u : 256u;
    float bound = weight_row_bound<TYPE>(w + (size_t)(wr < n ? wr : n - 1u) * (k / PER) * BLOCK, k, sub, lanes);
    if (lanes > 1u) bound = dpp_max<0xB1>(bound);  // as many of the four steps as cover the row's lanes
    if (lanes > 2u) bound = dpp_max<0x4E>(bound);
    if (lanes > 4u) bound = dpp_max<0x141>(bound);
    if (lanes > 8u) bound = dpp_max<0x140>(bound);
    if (sub == 0 && wr < n) scales[wr] = weight_row_scale(bound);
}

// One group of GROUP threads (256, or 64 = one wave for short rows): row scale and f16 conversion of activation row
// `row` (rows >= m: the last row is read and nothing is stored).  GROUP 256: every thread of the workgroup calls it (one
// barrier inside); red: four floats of the group.  GROUP 64: no barrier, red unused.
template <bool X_BF16, uint32_t GROUP = 256>
__device__ __forceinline__ void prep_activation_row(const void* __restrict__ x, uint8_t* __restrict__ ws, const Workspace& L,
                                                    uint32_t m, uint32_t k, uint32_t perm_hd, uint32_t row_in, uint32_t t,
                                                    float* red) {
    const bool valid = row_in < m;
    const uint32_t out_row = valid ? row_in : m - 1u, row = out_row;
    const uint32_t chunks = k / 8;

    // perm_hd != 0: x is stored [k / perm_hd][m][perm_hd] (heads outermost), element (row, kk) at
    // ((kk / perm_hd) * m + row) * perm_hd + kk % perm_hd; perm_hd is a multiple of 8, so a chunk stays inside a head
    auto elem0 = [&](uint32_t i) -> size_t {
        const uint32_t kk = 8u * i;
        return perm_hd ? ((size_t)(kk / perm_hd) * m + row) * perm_hd + kk % perm_hd : (size_t)row * k + kk;
    };
    struct Raw {
        uint4 a, b;  // bf16: a holds the eight values; f32: a and b four each
    };
    auto load_raw = [&](uint32_t i) -> Raw {
        Raw r{};
        if constexpr (X_BF16) {
            r.a = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(x) + elem0(i));
        } else {
            const uint4* p = reinterpret_cast<const uint4*>(static_cast<const float*>(x) + elem0(i));
            r.a = p[0], r.b = p[1];
        }
        return r;
    };
    auto decode = [&](const Raw& r, float* v) {
        if constexpr (X_BF16) {
            const uint32_t w[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[2 * j] = bf16_bits_to_f32(w[j] & 0xffffu);
                v[2 * j + 1] = bf16_bits_to_f32(w[j] >> 16);
            }
        } else {
            const uint32_t w[8] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = __uint_as_float(w[j]);
        }
    };
    auto fold = [&](const Raw& r, float& amax) {
        float v[8];
        decode(r, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float a = fabsf(v[j]);
            amax = a <= 3.0e38f ? fmaxf(amax, a) : amax;  // inf / nan do not set the scale
        }
    };
    auto convert = [&](const Raw& r, uint32_t i, float scale) {
        float v[8];
        decode(r, v);
        uint32_t h[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) h[j] = f16_bits(v[j] * scale);
        *reinterpret_cast<uint4*>(ws + L.xh + ((size_t)out_row * k + 8 * i) * 2) =
            make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
    };

    // largest finite magnitude of the row; a row of up to 2 * GROUP chunks (k <= 4096 for a group of 256) stays in
    // registers for the conversion, longer ones are read a second time
    const bool kept = chunks <= 2u * GROUP;
    Raw held[2];
    float amax = 0.f;
    if (kept) {
#pragma unroll
        for (uint32_t j = 0; j < 2; ++j) {
            const uint32_t i = t + j * GROUP;
            held[j] = load_raw(i < chunks ? i : chunks - 1u);
        }
#pragma unroll
        for (uint32_t j = 0; j < 2; ++j)
            if (t + j * GROUP < chunks) fold(held[j], amax);
    } else {
        for (uint32_t i = t; i < chunks; i += GROUP) fold(load_raw(i), amax);
    }
    amax = dpp_max<0xB1>(amax);
    amax = dpp_max<0x4E>(amax);
    amax = dpp_max<0x141>(amax);
    amax = dpp_max<0x140>(amax);
    amax = xor32_max(xor16_max(amax));
    if constexpr (GROUP == 256) {
        if ((t & 63u) == 0) red[t >> 6] = amax;
        __syncthreads();
        amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    }

    int ex = 0;
    if (amax > 0.f) (void)frexpf(amax, &ex);  // amax = f * 2^ex, f in [0.5, 1)
    int sh = 10 - ex;                          // amax * 2^sh in [512, 1024)
    sh = sh < -100 ? -100 : sh > 100 ? 100 : sh;
    if (amax == 0.f) sh = 0;
    const float scale = ldexpf(1.f, sh);
    if (!valid) return;
    if (t == 0) reinterpret_cast<float*>(ws + L.rs)[out_row] = ldexpf(1.f, -sh);

    if (kept) {
#pragma unroll
        for (uint32_t j = 0; j < 2; ++j)
            if (t + j * GROUP < chunks) convert(held[j], t + j * GROUP, scale);
    } else {
        for (uint32_t i = t; i < chunks; i += GROUP) convert(load_raw(i), i, scale);
    }
}

// Pre-pass.  The first scan_wgs workgroups (none when the caller brings the scales): 256 / weight_scan_lanes(k) weight
// rows each, that many lanes per row over the row's block headers; they are one load per lane and go first so that
// they run beside the activation rows instead of behind them.  The next m workgroups: one per activation row, row
// scale and f16 conversion.  Per weight row, a
// power of two that brings the row's largest possible |w| (Q4_K: |d|*63*15 + |dmin|*63, Q6_K:
// |d|*128*32, Q8_0: |d|*128) to about 2^14, so that neither large super-block scales overflow f16 nor small ones fall into its
// subnormals; the main kernel multiplies the weights by it before they are rounded (exact) and its
// epilogue divides it out.
template <bool X_BF16, int TYPE>
__global__ __launch_bounds__(256) void tile_prep_kernel(const void* __restrict__ x, const uint8_t* __restrict__ w,
                                                        const uint8_t* __restrict__ w2, uint8_t* __restrict__ ws, uint32_t m,
                                                        uint32_t n, uint32_t k, uint32_t perm_hd, uint32_t scan_wgs) {
    __shared__ float red[4];
    // (w2: a second matrix of n rows -- the SwiGLU form -- scanned by the second half of the scan workgroups; its scales
    // follow the first matrix's)
    const Workspace L = workspace_layout(m, w2 ? 2u * n : n, k);
    if (blockIdx.x < scan_wgs) {
        const uint32_t lanes = weight_scan_lanes<TYPE>(k);
        const uint32_t per_matrix = w2 ? scan_wgs / 2u : scan_wgs, second = blockIdx.x >= per_matrix ? 1u : 0u;
        prep_weight_rows<TYPE>(second ? w2 : w, reinterpret_cast<float*>(ws + L.wdown) + second * n, n, k,
                               (blockIdx.x - second * per_matrix) * (256u / lanes), threadIdx.x, lanes);
    } else
        prep_activation_row<X_BF16>(x, ws, L, m, k, perm_hd, blockIdx.x - scan_wgs, threadIdx.x, red);
}

// The weight-row scales alone: what the pre-pass's weight workgroups compute, for a caller that keeps them.
template <int TYPE>
__global__ __launch_bounds__(256) void weight_scales_kernel(const uint8_t* __restrict__ w, float* __restrict__ scales,
                                                            uint32_t n, uint32_t k) {
    const uint32_t lanes = weight_scan_lanes<TYPE>(k);
    prep_weight_rows<TYPE>(w, scales, n, k, blockIdx.x * (256u / lanes), threadIdx.x, lanes);
}

struct GemmArgs {
    const uint8_t* ws;  // workspace filled by the pre-pass
    const uint8_t* w;
    float* y;
    uint32_t m, n, k;
    // The grouped (expert) form looks at a slice of a larger problem: the workspace is laid out for
    // lay_m activation rows and lay_n weight rows, the slice's weight rows start at wd_off in the
    // table of weight-row scales, activation row r of the workspace is output row row_map[r].  The
    // dense form has lay_m = m, lay_n = n, wd_off = 0, row_map = nullptr.
    uint32_t lay_m, lay_n, wd_off;
    const uint32_t* row_map;
    // The 256-element runs [sb0, sb1) of every row that the workgroup multiplies (K-quants: super-blocks; Q8_0 / Q4_0:
    // eight blocks, the last run may be half a one): all of them except in the split form of the small tiles, whose
    // workgroups each write the partial sums of a slice of k
    uint32_t sb0, sb1;
    // Grouped form: the workspace holds one converted row per TOKEN and tile row r reads token row_map[r] / gather_div
    // (the routed rows of a token share its activations: top_k of them at gate / up, one at down).
    uint32_t gather_div;
    // the weight rows' scales (lay_n floats): the pre-pass's in the workspace, or the caller's, computed once for weights
    // that do not change (hq_weight_row_scales_ggml)
    const float* wscale;
    // SwiGLU form of the grouped Q4_K / Q5_K tiles: a second stack (the up projection beside the gate projection in
    // `w`) and its rows' scales; the tile multiplies both and stores silu(gate) * up.  Null otherwise.
    const uint8_t* w2;
    const float* wscale2;
    // Dense form only, may be null: a [m][n] f32 matrix g; the epilogue stores silu(g) * (x . W^T) instead of the
    // product (the up projection of a SwiGLU layer finishing the gating of the gate projection computed before it).
    const float* gate_in;
};

__device__ __forceinline__ f16x8_t as_frag(uint4 v) { return __builtin_bit_cast(f16x8_t, v); }

typedef __attribute__((ext_vector_type(2))) float f32x2_t;

__device__ __forceinline__ uint4 ld16(const uint8_t* p) { return *reinterpret_cast<const uint4*>(p); }

// Two f16 weights from bytes 2*part and 2*part + 1 of u (each below 256): the bytes are placed under the f16 bit
// pattern of 1024 by one byte permute (0x6400 | b = 1024 + b, exact), then scale * (1024 + b) + c per value as a
// mixed-precision FMA (f16 operand, f32 scale and constant, f32 arithmetic, f16 result); c carries -1024 * scale and the
// format's own offset.  Three instructions for two weights where conversion, FMA and packing took five.
__device__ __forceinline__ uint32_t mix_pair(uint32_t u, int part, float scale, float c) {
    const uint32_t pq = __builtin_amdgcn_perm(0x64646464u, u, part ? 0x04030402u : 0x04010400u);
    uint32_t r;
    asm("v_fma_mixlo_f16 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(pq), "v"(scale), "v"(c));
    asm("v_fma_mixhi_f16 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(r) : "v"(pq), "v"(scale), "v"(c));
    return r;
}

constexpr int WAVES = 4;           // one per SIMD; two workgroups share a CU
constexpr int BM = 256;            // token rows per workgroup of the prefill-sized tiles
constexpr int BM_SMALL = 64;       // ... of the Q4_K / Q5_K tiles for a few token rows (up to 128)
constexpr int BM_MID = 128;        // ... of the tiles for sparsely filled experts
constexpr int BN_WIDE = 128, BN_NARROW = 64;    // weight rows per workgroup

// Activation side of a workgroup tile, the same for every weight type: the pre-pass output goes
// global -> LDS in 1 KB wave instructions; wave w, instruction i (< kDma) fills 8 LDS rows of
// the tile, (w * kDma + i) * 8 .. +8; lane L owns row L/8 of them and LDS chunk L%8, which
// holds global chunk (L%8) ^ ((row/2)%8), and (row/2)%8 = L/16 + 4*(i%2).  Rows past the end of x read
// the last row instead (their results are never stored).  BMT = token rows of the tile.
template <int BMT, bool GATHER = false>
struct ActTileT {
    static constexpr int kDma = (BMT / 8) / WAVES;  // BMT / 8 one-KB fetches fill the activation tile
    static constexpr int kTile = BMT * ROW * 2;     // bytes of one activation buffer; two of them in LDS
    uint8_t* smem;
    const uint8_t* xtile;
    uint32_t a_swz, a_row0, a_rows_left, a_last, row_pitch, wave_u, lds_base;
    uint32_t g_tok[GATHER ? kDma : 1];  // GATHER: the token row behind this lane's row of fetch i

    __device__ __forceinline__ void init(const GemmArgs& a, const Workspace& W, uint32_t m0, uint32_t lane, uint32_t wave) {
        extern __shared__ uint4 smem4[];
        smem = reinterpret_cast<uint8_t*>(smem4);
        row_pitch = a.k * 2u;
        a_swz = ((lane & 7u) ^ (lane >> 4)) << 4;
        a_row0 = wave * (8u * kDma) + (lane >> 3);
        a_rows_left = a.m - m0;  // >= 1
        a_last = (a_rows_left - 1u) * row_pitch + a_swz;
        xtile = a.ws + W.xh + (GATHER ? (size_t)0 : (size_t)m0 * row_pitch);
        if constexpr (GATHER) {
#pragma unroll
            for (int i = 0; i < kDma; ++i) {
                const uint32_t r = a_row0 + 8u * i;
                g_tok[i] = a.row_map[m0 + (r < a_rows_left ? r : a_rows_left - 1u)] / a.gather_div;
            }
        }
        wave_u = __builtin_amdgcn_readfirstlane(wave);  // the same value, known to be uniform
        // LDS byte address of the tile buffers (wave-uniform, goes to M0)
        lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem);
    }
    // Fetch i of stage st into buffer buf.  Issued as inline assembly: the compiler would otherwise
    // wait for every outstanding global_load_lds before any later LDS read (it cannot tell the two
    // buffers apart), which exposes the whole fetch latency in every stage.  The waits are placed by
    // hand by the callers.
    __device__ __forceinline__ void fetch(uint32_t st, uint32_t buf, int i) const {
        const uint32_t r = a_row0 + 8u * i;
        const uint8_t* src = xtile + (size_t)st * (BK * 2);
        if constexpr (GATHER)
            src += (size_t)g_tok[i] * row_pitch + (a_swz ^ ((i & 1u) << 6));
        else
            src += r < a_rows_left ? r * row_pitch + (a_swz ^ ((i & 1u) << 6)) : a_last ^ ((i & 1u) << 6);
        const uint32_t dst = lds_base + buf * kTile + (wave_u * kDma + i) * 1024u;
        asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(dst) : "memory", "m0");
        __builtin_amdgcn_sched_barrier(0);  // one address at a time: keeps eight 64-bit pointers out of the registers
    }
    __device__ __forceinline__ void fetch_all(uint32_t st, uint32_t buf) const {
#pragma unroll
        for (int i = 0; i < kDma; ++i) fetch(st, buf, i);
    }
    // The 8 activations of 16-byte chunk kchunk (of the row's 64 per stage) of tile row `row`.
    __device__ __forceinline__ uint4 frag(uint32_t buf, uint32_t row, uint32_t kchunk) const {
        return *reinterpret_cast<const uint4*>(smem + buf * kTile + row * (ROW * 2) + ((kchunk ^ ((row >> 1) & 7u)) << 4));
    }
};
using ActTile = ActTileT<BM>;


// Stores a wave's accumulators.  The weights are the MFMA's first operand, so an accumulator tile
// is indexed [weight row][token]: value v of a lane belongs to token lane%32 and weight row
// 8*(v/4) + 4*(lane/32) + v%4 of the tile, four consecutive outputs of one token per v/4, one
// 16-byte store.  Undoes the activation-row and weight-row scales.
template <int MT, int NT>
__device__ __forceinline__ void store_tile(const GemmArgs& a, const Workspace& W, const f32x16_t (&acc)[MT][NT],
                                           uint32_t mbase, uint32_t nbase, uint32_t l32, uint32_t lg) {
    const float* rs = reinterpret_cast<const float*>(a.ws + W.rs);
    const float* wd = a.wscale;
    const bool vec_ok = a.n % 4 == 0 && (reinterpret_cast<uintptr_t>(a.y) & 15u) == 0;  // uniform
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const uint32_t gnb = nbase + nt * 32 + 4 * lg;
        float wup[16];  // 2^e of the 16 weight rows, from their 2^-e
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            uint32_t gn = gnb + 8 * (v >> 2) + (v & 3);
            gn = gn < a.n ? gn : a.n - 1u;
            wup[v] = __uint_as_float(0x7f000000u - __float_as_uint(wd[a.wd_off + gn]));
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const uint32_t gm = mbase + mt * 32 + l32;
            if (gm >= a.m) continue;
            const uint32_t orow = a.row_map ? a.row_map[gm] : gm;
            const float rsv = rs[a.gather_div ? orow / a.gather_div : gm];
            float* yp = a.y + (size_t)orow * a.n + gnb;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float o0 = acc[mt][nt][4 * g] * (rsv * wup[4 * g]), o1 = acc[mt][nt][4 * g + 1] * (rsv * wup[4 * g + 1]);
                float o2 = acc[mt][nt][4 * g + 2] * (rsv * wup[4 * g + 2]), o3 = acc[mt][nt][4 * g + 3] * (rsv * wup[4 * g + 3]);
                const uint32_t gn = gnb + 8 * g;
                if (a.gate_in) {  // (uniform) silu(gate) * up, the stand-alone kernel's arithmetic
                    const float* gp = a.gate_in + (size_t)orow * a.n + gnb + 8 * g;
                    if (vec_ok && (reinterpret_cast<uintptr_t>(a.gate_in) & 15u) == 0) {
                        if (gn < a.n) {
                            const float4 gv = *reinterpret_cast<const float4*>(gp);
                            o0 = silu_mul_f32(gv.x, o0), o1 = silu_mul_f32(gv.y, o1), o2 = silu_mul_f32(gv.z, o2), o3 = silu_mul_f32(gv.w, o3);
                        }
                    } else {
                        if (gn < a.n) o0 = silu_mul_f32(gp[0], o0);
                        if (gn + 1 < a.n) o1 = silu_mul_f32(gp[1], o1);
                        if (gn + 2 < a.n) o2 = silu_mul_f32(gp[2], o2);
                        if (gn + 3 < a.n) o3 = silu_mul_f32(gp[3], o3);
                    }
                }
                if (vec_ok) {
                    if (gn < a.n) *reinterpret_cast<float4*>(yp + 8 * g) = make_float4(o0, o1, o2, o3);
                } else {
                    if (gn < a.n) yp[8 * g] = o0;
                    if (gn + 1 < a.n) yp[8 * g + 1] = o1;
                    if (gn + 2 < a.n) yp[8 * g + 2] = o2;
                    if (gn + 3 < a.n) yp[8 * g + 3] = o3;
                }
            }
        }
    }
}

// The epilogue of the SwiGLU form: acc[mt][0] holds the gate products and acc[mt][1] the up products of the same
// output elements; both are scaled as store_tile scales them and silu(gate) * up is stored (silu_mul_f32: the bits
// of the stand-alone kernel over the two separately stored products).
template <int MT>
__device__ __forceinline__ void store_tile_swiglu(const GemmArgs& a, const Workspace& W, const f32x16_t (&acc)[MT][2],
                                                  uint32_t mbase, uint32_t nbase, uint32_t l32, uint32_t lg) {
    const float* rs = reinterpret_cast<const float*>(a.ws + W.rs);
    const bool vec_ok = a.n % 4 == 0 && (reinterpret_cast<uintptr_t>(a.y) & 15u) == 0;  // uniform
    const uint32_t gnb = nbase + 4 * lg;
    float wup_g[16], wup_u[16];  // 2^e of the 16 weight rows of either stack, from their 2^-e
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        uint32_t gn = gnb + 8 * (v >> 2) + (v & 3);
        gn = gn < a.n ? gn : a.n - 1u;
        wup_g[v] = __uint_as_float(0x7f000000u - __float_as_uint(a.wscale[a.wd_off + gn]));
        wup_u[v] = __uint_as_float(0x7f000000u - __float_as_uint(a.wscale2[a.wd_off + gn]));
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const uint32_t gm = mbase + mt * 32 + l32;
        if (gm >= a.m) continue;
        const uint32_t orow = a.row_map ? a.row_map[gm] : gm;
        const float rsv = rs[a.gather_div ? orow / a.gather_div : gm];
        float* yp = a.y + (size_t)orow * a.n + gnb;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float gv = acc[mt][0][4 * g + i] * (rsv * wup_g[4 * g + i]), uv = acc[mt][1][4 * g + i] * (rsv * wup_u[4 * g + i]);
                o[i] = silu_mul_f32(gv, uv);
            }
            const uint32_t gn = gnb + 8 * g;
            if (vec_ok) {
                if (gn < a.n) *reinterpret_cast<float4*>(yp + 8 * g) = make_float4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (gn + i < a.n) yp[8 * g + i] = o[i];
            }
        }
    }
}

// One workgroup tile of Q4_K weights: rows m0.. of the activations, weight rows n0...  The four
// waves form a (4 / WN) x WN grid; a wave owns MT x NT MFMA tiles of 32 x 32.
// TYPE = HQ_Q5_K: the same tile over 176-byte super-blocks; a lane also keeps the sixteen qh bytes that go with
// its nibble bytes (they serve all four chunks of the super-block, bit 2c + hi for sub-block 2c + hi) and ORs the
// fifth bit into the masked nibbles, three more VALU instructions per four weights.
// SWIGLU (NT = 2): the wave's two weight tiles are the same 32 rows of two stacks (a.w: gate, a.w2: up) and the
// epilogue stores silu(gate) * up.
template <int MT, int NT, int WN, int TYPE = HQ_Q4_K, bool GATHER = false, bool SWIGLU = false>
__device__ __forceinline__ void q4k_gemm_tile(const GemmArgs& a, uint32_t m0, uint32_t n0) {
    static_assert(!SWIGLU || NT == 2, "gate and up are the wave's two weight tiles");
    constexpr int BMT = 32 * MT * (WAVES / WN);  // token rows of the workgroup tile: 256, or 64 for the small tiles
    constexpr int DMA_PER_WAVE = ActTileT<BMT>::kDma;
    constexpr bool Q5 = TYPE == HQ_Q5_K;
    constexpr uint32_t BYTES = Q5 ? Q5K_BYTES : Q4K_BYTES, QS = Q5 ? 48u : 16u;  // super-block size, offset of the nibbles
    const Workspace W = workspace_layout(a.lay_m, a.lay_n, a.k);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t l32 = lane & 31u, lg = lane >> 5;

    const uint32_t row_bytes = (a.k / 256) * BYTES;
    const uint32_t sb0 = a.sb0, sb1 = a.sb1;  // sb0 < sb1
    ActTileT<BMT, GATHER> at;
    at.init(a, W, m0, lane, wave);

    // ---- weights: this lane's two rows (one per 32-row tile of the wave), bytes 16*lg.. of each chunk ----
    const uint8_t* wrow[NT];
    float wdown[NT];  // power-of-two scale 2^-e of the lane's rows, from the pre-pass
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        uint32_t gn = SWIGLU ? n0 + wn * 32 + l32 : n0 + wn * (32 * NT) + nt * 32 + l32;
        gn = gn < a.n ? gn : a.n - 1u;
        wrow[nt] = (SWIGLU && nt == 1 ? a.w2 : a.w) + (size_t)gn * row_bytes;
        wdown[nt] = (SWIGLU && nt == 1 ? a.wscale2 : a.wscale)[a.wd_off + gn];
    }
    uint4 braw[4][NT];        // nibbles of stages s, s+1, s+2 in slots s%4 (a stage is a chunk of its super-block: slot = c)
    uint4 hdr[NT], hdrn[NT];  // super-block headers: current, next
    [[maybe_unused]] uint4 hq[NT], hqn[NT];  // Q5_K: qh bytes 16*lg.. of the current and the next super-block
    auto load_b = [&](uint32_t sblk, int c, int slot) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            braw[slot][nt] = ld16(wrow[nt] + (size_t)sblk * BYTES + QS + 32 * c + 16 * lg);
    };
    auto load_hdr = [&](uint32_t sblk, uint4* h, [[maybe_unused]] uint4* q) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            h[nt] = ld16(wrow[nt] + (size_t)sblk * BYTES);
            if constexpr (Q5) q[nt] = ld16(wrow[nt] + (size_t)sblk * BYTES + 16 + 16 * lg);
        }
    };

    f32x16_t acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // This lane's weight scales of a stage, chunk c of the super-block whose header is h: sub-blocks
    // 2c (low nibbles) and 2c+1 (high nibbles).
    auto scales_of = [&](const uint4* h, int c, float (*dsc)[2], float (*ndm)[2]) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            uint32_t sc0, sc1, mn0, mn1;
            q4k_scales(h[nt].y, h[nt].z, h[nt].w, c, sc0, sc1, mn0, mn1);
            const float d = f16_bits_to_f32(h[nt].x & 0xffffu) * wdown[nt];
            const float dmin = f16_bits_to_f32(h[nt].x >> 16) * wdown[nt];
            dsc[nt][0] = d * (float)sc0;
            dsc[nt][1] = d * (float)sc1;
            // the weights are formed from 1024 + q (see b_eighth): the offset goes into the constant term
            ndm[nt][0] = fmaf(-1024.f, dsc[nt][0], -dmin * (float)mn0);
            ndm[nt][1] = fmaf(-1024.f, dsc[nt][1], -dmin * (float)mn1);
        }
    };
    // Eighth e of k-step ks of a stage with nibbles b and scales dsc / ndm: two weights -> one
    // fragment word.  Quarter q = e/2 is one nibble word (nt = q/2, word pair half = q%2), masked
    // once and kept in mw for its second eighth.
    uint32_t mw[2 * NT];
    // (qv, cc: Q5_K only -- the qh bytes of the stage's super-block and the stage's chunk index in it)
    auto b_eighth = [&](const uint4* b, const float (*dsc)[2], const float (*ndm)[2], int ks, int e, uint4* bfw,
                        [[maybe_unused]] const uint4* qv, [[maybe_unused]] int cc) {
        const int q = e >> 1, part = e & 1, nt = q >> 1, half = q & 1;
        const int hi = ks >> 1;  // 0: low nibbles, 1: high nibbles
        if (part == 0) {
            const uint32_t w = (ks & 1) ? (half ? b[nt].w : b[nt].z) : (half ? b[nt].y : b[nt].x);
            uint32_t m = (hi ? w >> 4 : w) & 0x0f0f0f0fu;
            if constexpr (Q5) {
                const uint32_t h = (ks & 1) ? (half ? qv[nt].w : qv[nt].z) : (half ? qv[nt].y : qv[nt].x);
                m |= ((h >> (2 * cc + hi)) & 0x01010101u) << 4;
            }
            // opaque: the masked word is formed once, here, and both byte permutes below read this register
            asm volatile("" : "+v"(m));
            mw[q] = m;
        }
        const uint32_t m = mw[q];
        // d*sc*(1024 + q) + (-1024*d*sc - dmin*mn), see mix_pair
        const uint32_t r = mix_pair(m, part, dsc[nt][hi], ndm[nt][hi]);
        if (half == 0)
            (part == 0 ? bfw[nt].x : bfw[nt].y) = r;
        else
            (part == 0 ? bfw[nt].z : bfw[nt].w) = r;
    };
    constexpr int E = 4 * NT;            // eighths per k-step
    constexpr int kSteps = 4 * MT;       // MFMA steps per stage: k-step t / MT, row tile t % MT
    constexpr int PD = NT == 1 ? 3 : 1;  // steps an activation fragment is requested ahead (a step is NT MFMAs)
    static_assert(kSteps >= DMA_PER_WAVE && (E >= MT ? E % MT == 0 : MT % E == 0 && MT / E >= 2), "the spreading below assumes it");

    // ---- prologue: everything the first stage needs, and the second stage's nibbles ----
    load_hdr(sb0, hdr, hq);
    load_b(sb0, 0, 0);
    load_b(sb0, 1, 1);  // a super-block has four stages
    at.fetch_all(4 * sb0, 0);
    if (sb0 + 1 < sb1) load_hdr(sb0 + 1, hdrn, hqn);
    float dsc[NT][2], ndm[NT][2];      // scales of the stage being multiplied
    uint4 bfc[NT], bfn[NT];            // weight fragments: current k-step, next
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    scales_of(hdr, 0, dsc, ndm);
#pragma unroll
    for (int e = 0; e < E; ++e) b_eighth(braw[0], dsc, ndm, 0, e, bfc, hq, 0);
    __syncthreads();

    // The loop is software pipelined over stages as well: while the last k-step of stage s is
    // multiplied, the scales of stage s+1 and the fragments of its first k-step are formed, so a
    // stage begins with an MFMA and not with sixty VALU instructions that nothing overlaps.
    for (uint32_t sblk = sb0; sblk < sb1; ++sblk) {
        const bool next_sb = sblk + 1 < sb1;  // uniform
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t st = 4 * sblk + c;
            const uint32_t buf = c & 1;
            const bool has_next = c < 3 || next_sb;  // uniform: stage st + 1 belongs to this workgroup
            // The next stage's nibbles, requested a stage ago.  They are claimed here, before this
            // stage's activation fetches are issued: the compiler does not know about those, and the
            // wait it puts in front of the first use of these registers would otherwise cover them too.
            uint4 bnext[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                bnext[nt] = braw[(c + 1) & 3][nt];
                asm volatile("" : "+v"(bnext[nt].x), "+v"(bnext[nt].y), "+v"(bnext[nt].z), "+v"(bnext[nt].w));
            }
            if (c == 0 && sblk > sb0) {  // this super-block's header; request the next one
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    hdr[nt] = hdrn[nt];
                    if constexpr (Q5) hq[nt] = hqn[nt];
                }
                if (next_sb) load_hdr(sblk + 1, hdrn, hqn);
            }
            // nibbles of stage st + 2 (the header fetch of a super-block, issued a super-block ahead, has
            // already pulled most of its lines into cache)
            if (c < 2) {
                load_b(sblk, c + 2, (c + 2) & 3);
            } else if (next_sb) {
                load_b(sblk + 1, c - 2, (c + 2) & 3);
            }
            const bool fetch_a = has_next;

            auto a_frag = [&](int t) -> uint4 {
                const int ks = t / MT, mt = t % MT;
                // chunk index of this lane group's 8 activations inside the row's 64
                return at.frag(buf, wm * (32 * MT) + mt * 32 + l32, ks < 2 ? 2u * lg + ks : 4u + 2u * lg + (ks - 2));
            };
            float dscn[NT][2], ndmn[NT][2];  // scales of stage st + 1
            uint4 af[PD + 1];
#pragma unroll
            for (int t = 0; t < PD; ++t) af[t] = a_frag(t);
#pragma unroll
            for (int t = 0; t < kSteps; ++t) {
                const int ks = t / MT, mt = t % MT;
                if (t + PD < kSteps) af[(t + PD) % (PD + 1)] = a_frag(t + PD);
                // The next stage's activations go into the other buffer (free since the barrier that ended
                // the previous stage), one fetch per step at the start of the stage rather than all at once.
                if (t < DMA_PER_WAVE && fetch_a) at.fetch(st + 1, buf ^ 1u, t);
                const uint4 afc = af[t % (PD + 1)];
                acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_frag(bfc[0]), as_frag(afc), acc[mt][0], 0, 0, 0);
                // The next k-step's weights, spread evenly over this k-step's MFMAs (an MFMA hides about
                // four VALU instructions; what exceeds that delays the next MFMA).  In the last k-step
                // they are the next stage's first, preceded by that stage's scales.
                if (ks < 3) {
                    if constexpr (E >= MT) {
#pragma unroll
                        for (int e = 0; e < E / MT; ++e) b_eighth(braw[c], dsc, ndm, ks + 1, mt * (E / MT) + e, bfn, hq, c);
                    } else if (mt % (MT / E) == 0) {
                        b_eighth(braw[c], dsc, ndm, ks + 1, mt / (MT / E), bfn, hq, c);
                    }
                } else if (has_next) {
                    if (mt == 0) scales_of(c < 3 ? hdr : hdrn, (c + 1) & 3, dscn, ndmn);
                    if constexpr (E >= MT) {
                        // the scales come first, so the eighths of row tile 0 move to the last one's slot
                        if (mt > 0) {
#pragma unroll
                            for (int e = 0; e < E / MT; ++e)
                                b_eighth(bnext, dscn, ndmn, 0, (mt - 1) * (E / MT) + e, bfn, c < 3 ? hq : hqn, (c + 1) & 3);
                        }
                        if (mt == MT - 1) {
#pragma unroll
                            for (int e = 0; e < E / MT; ++e)
                                b_eighth(bnext, dscn, ndmn, 0, (MT - 1) * (E / MT) + e, bfn, c < 3 ? hq : hqn, (c + 1) & 3);
                        }
                    } else if (mt % (MT / E) == 1) {
                        b_eighth(bnext, dscn, ndmn, 0, mt / (MT / E), bfn, c < 3 ? hq : hqn, (c + 1) & 3);
                    }
                }
                if constexpr (NT == 2)
                    acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_frag(bfc[1]), as_frag(afc), acc[mt][1], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (mt == MT - 1) {
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) bfc[nt] = bfn[nt];
                }
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                dsc[nt][0] = dscn[nt][0], dsc[nt][1] = dscn[nt][1];
                ndm[nt][0] = ndmn[nt][0], ndm[nt][1] = ndmn[nt][1];
            }

            // The next stage's activations must have landed before anyone reads them.  They are the
            // youngest vector memory operations of this wave and such operations complete in order.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
    }

    if constexpr (SWIGLU)
        store_tile_swiglu<MT>(a, W, acc, m0 + wm * (32 * MT), n0 + wn * 32, l32, lg);
    else
        store_tile<MT, NT>(a, W, acc, m0 + wm * (32 * MT), n0 + wn * (32 * NT), l32, lg);
}

// One workgroup tile of Q8_0 weights (34-byte blocks: f16 d, 32 int8), four waves side by side, each
// 256 tokens x 32 weight rows.  A stage is 64 k = two blocks of a row; lane group lg = lane/32 takes
// block 2*st + lg whole, so its fragments of k-step ks are bytes 8*ks.. of the block and the
// activation chunk is 4*lg + ks.  The blocks are only 2-byte aligned: a lane whose blocks start at
// 4n reads the eight words of int8 from 4n (two bytes early) plus the two bytes that follow them,
// and shifts by two bytes when it forms a word (v_alignbyte); a lane whose blocks start at 4n + 2
// reads them from 4n + 4, aligned, and shifts by zero.  Since a stage advances every lane by 68
// bytes, a lane keeps its case.  w = d * q = d * ((q ^ 0x80) - 128) in fp32 (exact), one rounding
// to f16.
//
// TYPE = HQ_Q4_0 (18-byte blocks: f16 d, 16 bytes of nibbles; elements 0..15 are the low nibbles, 16..31 the
// high ones): the same frame with four words per block instead of eight; k-steps 0 and 1 take the low nibbles of
// words 0..1 and 2..3, k-steps 2 and 3 the high nibbles of the same words.  A stage advances a lane by 36 bytes,
// so it keeps its alignment case here too.  w = d * (q - 8).
template <int MT, int WN, int TYPE = HQ_Q8_0, bool GATHER = false>
__device__ __forceinline__ void q80_gemm_tile(const GemmArgs& a, uint32_t m0, uint32_t n0) {
    constexpr int BMT = 32 * MT * (WAVES / WN);  // token rows of the workgroup tile: 256, or 128 for the small tiles
    constexpr int DMA_PER_WAVE = ActTileT<BMT>::kDma;
    constexpr bool Q4 = TYPE == HQ_Q4_0;
    constexpr uint32_t BYTES = Q4 ? Q4_0_BYTES : Q8_0_BYTES;
    const Workspace W = workspace_layout(a.lay_m, a.lay_n, a.k);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t l32 = lane & 31u, lg = lane >> 5;
    // stages [st_first, nstages) of every row, an even number of them (k % 128 == 0; slices of k are whole 256s)
    const uint32_t st_first = 4u * a.sb0, nstages = a.sb1 * 4u < a.k / BK ? a.sb1 * 4u : a.k / BK;
    ActTileT<BMT, GATHER> at;
    at.init(a, W, m0, lane, wave);

    uint32_t gn = n0 + wn * 32 + l32;
    gn = gn < a.n ? gn : a.n - 1u;
    const uint8_t* blk0 = a.w + (size_t)gn * (a.k / 32) * BYTES + lg * BYTES;  // this lane's block of stage 0
    const float wdown = a.wscale[a.wd_off + gn];
    const bool early = (reinterpret_cast<uintptr_t>(blk0) & 2u) == 0;  // blocks at 4n: the int8 start two bytes into a word
    const uint32_t shift = early ? 2u : 0u;
    const uint8_t* win0 = early ? blk0 : blk0 + 2;                     // first of the eight aligned words
    // raw registers of a stage's block: d, eight words, and (early lanes) the two bytes behind them
    struct Raw { uint32_t d; uint4 lo, hi; uint32_t tail; };
    Raw braw[2];
    auto load_b = [&](uint32_t st, int slot) {
        const size_t off = (size_t)st * (2 * BYTES);
        braw[slot].d = *reinterpret_cast<const uint16_t*>(blk0 + off);
        braw[slot].lo = ld16_unaligned(win0 + off);  // 4-byte aligned
        if constexpr (!Q4) braw[slot].hi = ld16_unaligned(win0 + off + 16);
        // late lanes do not use it: they re-read their d, which is always inside the buffer
        braw[slot].tail = *reinterpret_cast<const uint16_t*>(early ? win0 + off + (Q4 ? 16 : 32) : blk0 + off);
    };

    f32x16_t acc[MT][1];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][0][v] = 0.f;

    constexpr int kSteps = 4 * MT;  // MFMA steps per stage: k-step t / MT, row tile t % MT
    constexpr int PD = 3;           // steps an activation fragment is requested ahead
    static_assert(MT % 4 == 0 && kSteps >= DMA_PER_WAVE, "four eighths per k-step, spread over the MT steps");

    load_b(st_first, 0);
    at.fetch_all(st_first, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    for (uint32_t st2 = st_first; st2 < nstages; st2 += 2) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const uint32_t st = st2 + c;
            const uint32_t buf = c;
            // This stage's block, requested a stage ago.  It is claimed here, before this stage's
            // activation fetches are issued: the compiler does not know about those, and the wait it
            // puts in front of the first use of these registers would otherwise cover them too.
            Raw cur = braw[c];
            if constexpr (Q4)
                asm volatile("" : "+v"(cur.d), "+v"(cur.tail), "+v"(cur.lo.x), "+v"(cur.lo.y), "+v"(cur.lo.z), "+v"(cur.lo.w));
            else
                asm volatile("" : "+v"(cur.d), "+v"(cur.tail), "+v"(cur.lo.x), "+v"(cur.lo.y), "+v"(cur.lo.z), "+v"(cur.lo.w),
                             "+v"(cur.hi.x), "+v"(cur.hi.y), "+v"(cur.hi.z), "+v"(cur.hi.w));
            const bool has_next = st + 1 < nstages;  // uniform
            if (has_next) load_b(st + 1, c ^ 1);
            // (the weights are formed from 1024 + q, see mix_pair: the constant term carries the -1024 as well; exact)
            const float dsc = f16_bits_to_f32(cur.d & 0xffffu) * wdown, ndm = (Q4 ? -1032.f : -1152.f) * dsc;
            uint32_t dw[9];
            dw[0] = cur.lo.x, dw[1] = cur.lo.y, dw[2] = cur.lo.z, dw[3] = cur.lo.w;
            if constexpr (Q4) {
                dw[4] = cur.tail;
            } else {
                dw[4] = cur.hi.x, dw[5] = cur.hi.y, dw[6] = cur.hi.z, dw[7] = cur.hi.w, dw[8] = cur.tail;
            }
            // Eighth e of k-step ks: two weights -> fragment word e.  Word 2*ks + e/2 of the block's int8
            // is formed (and its sign bits flipped) once and kept for its second eighth.
            uint32_t uw[2];
            auto b_eighth = [&](int ks, int e, uint4& bfw) {
                const int q = e >> 1, part = e & 1, i = 2 * (Q4 ? ks & 1 : ks) + q;
                if (part == 0) {
                    uint32_t u = __builtin_amdgcn_alignbyte(dw[i + 1], dw[i], shift);
                    if constexpr (Q4)
                        u = (ks >= 2 ? u >> 4 : u) & 0x0f0f0f0fu;
                    else
                        u ^= 0x80808080u;
                    // opaque: the word is formed once, here, and both byte permutes of mix_pair read this register
                    asm volatile("" : "+v"(u));
                    uw[q] = u;
                }
                const uint32_t r = mix_pair(uw[q], part, dsc, ndm);
                (e == 0 ? bfw.x : e == 1 ? bfw.y : e == 2 ? bfw.z : bfw.w) = r;
            };
            auto a_frag = [&](int t) -> uint4 {
                return at.frag(buf, wm * (32 * MT) + (t % MT) * 32 + l32, 4u * lg + (t / MT));
            };
            uint4 bfc, bfn;
#pragma unroll
            for (int e = 0; e < 4; ++e) b_eighth(0, e, bfc);
            uint4 af[PD + 1];
#pragma unroll
            for (int t = 0; t < PD; ++t) af[t] = a_frag(t);
#pragma unroll
            for (int t = 0; t < kSteps; ++t) {
                const int ks = t / MT, mt = t % MT;
                if (t + PD < kSteps) af[(t + PD) % (PD + 1)] = a_frag(t + PD);
                // next stage's activations into the other buffer (free since the barrier that ended the
                // previous stage), one fetch per step
                if (t < DMA_PER_WAVE && has_next) at.fetch(st + 1, buf ^ 1u, t);
                acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_frag(bfc), as_frag(af[t % (PD + 1)]), acc[mt][0], 0, 0, 0);
                if (ks < 3 && mt % (MT / 4) == 0) b_eighth(ks + 1, mt / (MT / 4), bfn);
                __builtin_amdgcn_sched_barrier(0);
                if (mt == MT - 1) bfc = bfn;
            }
            // The next stage's activations must have landed before anyone reads them; they are the
            // youngest vector memory operations of this wave and such operations complete in order.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
    }
    store_tile<MT, 1>(a, W, acc, m0 + wm * (32 * MT), n0 + wn * 32, l32, lg);
}

// One workgroup tile of Q6_K weights (210-byte super-blocks: ql[128], qh[64], int8 scales[16], f16
// d), four waves side by side, each 256 tokens x 32 weight rows.  A 128-element half h of a
// super-block is two stages that read the same bytes: elements 128h + 32*g + l (g = 0..3, l < 32)
// are nibble g/2 of ql[64h + 32*(g%2) + l] with bits 2g, 2g+1 of qh[32h + l] on top, scale
// 8h + 2g + l/16.  Stage s' = g/2 (low nibbles, then high), lane group lg = g%2: a lane fetches its 32
// ql bytes, the half's 32 qh bytes, eight scale bytes and d once per half, a half ahead.
// w = d*sc*(q - 32) in fp32 (d*sc exact), one rounding to f16.  The blocks are 2-byte aligned; the
// hardware takes the unaligned 16-byte loads.
template <int MT, int WN, bool GATHER = false>
__device__ __forceinline__ void q6k_gemm_tile(const GemmArgs& a, uint32_t m0, uint32_t n0) {
    constexpr int BMT = 32 * MT * (WAVES / WN);  // token rows of the workgroup tile: 256, or 128 for the small tiles
    constexpr int DMA_PER_WAVE = ActTileT<BMT>::kDma;
    const Workspace W = workspace_layout(a.lay_m, a.lay_n, a.k);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t l32 = lane & 31u, lg = lane >> 5;
    const uint32_t nsb = a.sb1, nstages = 4u * a.sb1;  // super-blocks [sb0, sb1) of every row
    ActTileT<BMT, GATHER> at;
    at.init(a, W, m0, lane, wave);

    uint32_t gn = n0 + wn * 32 + l32;
    gn = gn < a.n ? gn : a.n - 1u;
    const uint8_t* wrow = a.w + (size_t)gn * (a.k / 256) * Q6K_BYTES;
    const float wdown = a.wscale[a.wd_off + gn];
    struct Raw { uint4 l0, l1, h0, h1; uint2 sc; uint32_t d; };  // one half of a super-block, this lane's share
    Raw braw[2];
    auto load_half = [&](uint32_t sb, int h, int slot) {
        const uint8_t* blk = wrow + (size_t)sb * Q6K_BYTES;
        braw[slot].l0 = ld16_unaligned(blk + 64 * h + 32 * lg);
        braw[slot].l1 = ld16_unaligned(blk + 64 * h + 32 * lg + 16);
        braw[slot].h0 = ld16_unaligned(blk + 128 + 32 * h);
        braw[slot].h1 = ld16_unaligned(blk + 128 + 32 * h + 16);
        braw[slot].sc = ld8_unaligned(blk + 192 + 8 * h);
        braw[slot].d = ld2(blk + 208);
    };

    f32x16_t acc[MT][1];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][0][v] = 0.f;

    constexpr int kSteps = 4 * MT;  // MFMA steps per stage: k-step t / MT, row tile t % MT
    constexpr int PD = 3;           // steps an activation fragment is requested ahead
    static_assert(MT % 4 == 0 && kSteps >= DMA_PER_WAVE, "four eighths per k-step, spread over the MT steps");

    load_half(a.sb0, 0, 0);
    at.fetch_all(4u * a.sb0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    for (uint32_t sb = a.sb0; sb < nsb; ++sb) {
        const bool next_sb = sb + 1 < nsb;  // uniform
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int h = c >> 1, hi = c & 1;  // half of the super-block; low / high nibbles
            const uint32_t st = 4 * sb + c;
            const uint32_t buf = c & 1;
            // This half's bytes, requested a half ago.  They are claimed at the start of the half, before
            // its activation fetches are issued: the compiler does not know about those, and the wait it
            // puts in front of the first use of these registers would otherwise cover them too.
            Raw& cur = braw[h];
            if (hi == 0) {
                asm volatile("" : "+v"(cur.l0.x), "+v"(cur.l0.y), "+v"(cur.l0.z), "+v"(cur.l0.w), "+v"(cur.l1.x), "+v"(cur.l1.y),
                             "+v"(cur.l1.z), "+v"(cur.l1.w), "+v"(cur.h0.x), "+v"(cur.h0.y), "+v"(cur.h0.z), "+v"(cur.h0.w),
                             "+v"(cur.h1.x), "+v"(cur.h1.y), "+v"(cur.h1.z), "+v"(cur.h1.w), "+v"(cur.sc.x), "+v"(cur.sc.y),
                             "+v"(cur.d));
                if (h == 0) {
                    load_half(sb, 1, 1);
                } else if (next_sb) {
                    load_half(sb + 1, 0, 0);
                }
            }
            const bool has_next = st + 1 < nstages;  // uniform
            // the lane's two scales of this stage: bytes 4*hi + 2*lg, +1 of the half's eight
            const uint32_t scw = (hi ? cur.sc.y : cur.sc.x) >> (16 * lg);
            const float dw = f16_bits_to_f32(cur.d & 0xffffu) * wdown;
            const float dsc0 = dw * (float)(int)(int8_t)(scw & 0xffu), dsc1 = dw * (float)(int)(int8_t)((scw >> 8) & 0xffu);
            const float ndm0 = -1056.f * dsc0, ndm1 = -1056.f * dsc1;
            const uint32_t lw[8] = {cur.l0.x, cur.l0.y, cur.l0.z, cur.l0.w, cur.l1.x, cur.l1.y, cur.l1.z, cur.l1.w};
            const uint32_t hw[8] = {cur.h0.x, cur.h0.y, cur.h0.z, cur.h0.w, cur.h1.x, cur.h1.y, cur.h1.z, cur.h1.w};
            const uint32_t hshift = 4 * hi + 2 * lg;
            // Eighth e of k-step ks: two weights -> fragment word e.  Word 2*ks + e/2 of the lane's 6-bit
            // values is assembled once and kept for its second eighth.
            uint32_t uw[2];
            auto b_eighth = [&](int ks, int e, uint4& bfw) {
                const int q = e >> 1, part = e & 1, i = 2 * ks + q;
                if (part == 0) {
                    const uint32_t nib = (hi ? lw[i] >> 4 : lw[i]) & 0x0f0f0f0fu;
                    uint32_t u = (((hw[i] >> hshift) & 0x03030303u) << 4) | nib;
                    // opaque: the word is formed once, here, and both byte permutes of mix_pair read this register
                    asm volatile("" : "+v"(u));
                    uw[q] = u;
                }
                // elements 8*ks.. of 32: scale ks / 2; d*sc*(1024 + q) - 1056*d*sc (the format's 32 and mix_pair's 1024)
                const uint32_t r = mix_pair(uw[q], part, ks < 2 ? dsc0 : dsc1, ks < 2 ? ndm0 : ndm1);
                (e == 0 ? bfw.x : e == 1 ? bfw.y : e == 2 ? bfw.z : bfw.w) = r;
            };
            auto a_frag = [&](int t) -> uint4 {
                return at.frag(buf, wm * (32 * MT) + (t % MT) * 32 + l32, 4u * lg + (t / MT));
            };
            uint4 bfc, bfn;
#pragma unroll
            for (int e = 0; e < 4; ++e) b_eighth(0, e, bfc);
            uint4 af[PD + 1];
#pragma unroll
            for (int t = 0; t < PD; ++t) af[t] = a_frag(t);
#pragma unroll
            for (int t = 0; t < kSteps; ++t) {
                const int ks = t / MT, mt = t % MT;
                if (t + PD < kSteps) af[(t + PD) % (PD + 1)] = a_frag(t + PD);
                // next stage's activations into the other buffer (free since the barrier that ended the
                // previous stage), one fetch per step
                if (t < DMA_PER_WAVE && has_next) at.fetch(st + 1, buf ^ 1u, t);
                acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_frag(bfc), as_frag(af[t % (PD + 1)]), acc[mt][0], 0, 0, 0);
                if (ks < 3 && mt % (MT / 4) == 0) b_eighth(ks + 1, mt / (MT / 4), bfn);
                __builtin_amdgcn_sched_barrier(0);
                if (mt == MT - 1) bfc = bfn;
            }
            // The next stage's activations must have landed before anyone reads them; they are the
            // youngest vector memory operations of this wave and such operations complete in order.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
    }
    store_tile<MT, 1>(a, W, acc, m0 + wm * (32 * MT), n0 + wn * 32, l32, lg);
}

// Tile order: workgroups go to the 8 XCDs round-robin and every XCD has its own L2, so workgroup i
// runs on XCD i % 8.  The tiles, counted along the weight rows first, are cut into eight equal runs and
// XCD x takes run x: its workgroups share one activation tile (or two, at a seam) that stays in that XCD's L2 while
// they sweep the weight tiles -- and every XCD has work whatever the number of token tiles is (with whole rows of
// tiles per XCD, 512 .. 1792 tokens kept two to seven of the eight XCDs busy and took the time of 2048).
// The grid is padded to 8 * ceil(tiles / 8).
__device__ __forceinline__ bool tile_of(uint32_t b, uint32_t tiles_m, uint32_t tiles_n, uint32_t bn, uint32_t& m0, uint32_t& n0) {
    const uint32_t total = tiles_m * tiles_n, run = (total + 7u) / 8u;
    const uint32_t xcd = b & 7u, idx = b >> 3;
    const uint32_t flat = xcd * run + idx;
    if (idx >= run || flat >= total) return false;
    m0 = (flat / tiles_n) * BM;
    n0 = (flat % tiles_n) * bn;
    return true;
}
// Workgroups of a launch whose tiles tile_of() hands out.
inline uint32_t tile_grid(uint32_t tiles_m, uint32_t tiles_n) { return 8u * ((tiles_m * tiles_n + 7u) / 8u); }

// Weight rows [0, n_wide) in tiles of 128 (the first grid_wide workgroups), the rest in tiles of 64.
template <int TYPE>
__global__ __launch_bounds__(64 * WAVES, 2) void q4k_gemm_kernel(GemmArgs a, uint32_t n_wide, uint32_t grid_wide) {
    const uint32_t tiles_m = (a.m + BM - 1) / BM;
    uint32_t m0, n0;
    if (blockIdx.x < grid_wide) {
        if (!tile_of(blockIdx.x, tiles_m, n_wide / BN_WIDE, BN_WIDE, m0, n0)) return;
        q4k_gemm_tile<8, 1, 4, TYPE>(a, m0, n0);
    } else {
        if (!tile_of(blockIdx.x - grid_wide, tiles_m, (a.n - n_wide + BN_NARROW - 1) / BN_NARROW, BN_NARROW, m0, n0)) return;
        q4k_gemm_tile<4, 1, 2, TYPE>(a, m0, n_wide + n0);
    }
}

// Up to 128 token rows of Q4_K / Q5_K: one token tile of 64 rows (m <= 64) or of 128, x 128 weight rows (four waves side by
// side, each 64 or 128 x 32, so every weight is dequantised once), so that a few rows do not pay for 256.  Where the tiles alone are
// fewer workgroups than the device has CUs, k is cut into `splits` slices of sb_per super-blocks, each with workgroups of
// its own that store their products into slice `s` of `partial` ([splits][m][n] floats, same scaling as y);
// split_sum_kernel then adds the slices in order.
template <int TYPE, int MTS>  // MTS = 2: 64 token rows per tile (m <= 64); 4: 128; 8: 256
__global__ __launch_bounds__(64 * WAVES, 2) void q4k_gemm_small_kernel(GemmArgs a, uint32_t splits, uint32_t sb_per,
                                                                       float* __restrict__ partial) {
    constexpr uint32_t BMS = 32 * MTS;
    // consecutive workgroups (which the hardware deals to the XCDs in turn) take consecutive weight-row tiles
    const uint32_t tiles_n = (a.n + BN_WIDE - 1) / BN_WIDE, tiles_m = (a.m + BMS - 1) / BMS;
    const uint32_t s = blockIdx.x / (tiles_n * tiles_m), t = blockIdx.x % (tiles_n * tiles_m);
    if (splits > 1) {
        a.sb0 = s * sb_per;
        a.sb1 = a.sb0 + sb_per < a.sb1 ? a.sb0 + sb_per : a.sb1;
        a.y = partial + (size_t)s * a.m * a.n;
    }
    q4k_gemm_tile<MTS, 1, 4, TYPE>(a, (t / tiles_n) * BMS, (t % tiles_n) * BN_WIDE);
}

// y = silu(x . Wg^T) * (x . Wu^T) for Q4_K / Q5_K: one workgroup per (tile of 32 * MTS token rows, 128 output columns), a
// wave the same 32 weight rows of both matrices (see q4k_gemm_tile's SWIGLU form).  No slices of k: the result is not
// linear in the partial products.
template <int TYPE, int MTS>
__global__ __launch_bounds__(64 * WAVES, 2) void q4k_swiglu_kernel(GemmArgs a) {
    constexpr uint32_t BMS = 32 * MTS;
    const uint32_t tiles_n = (a.n + BN_WIDE - 1) / BN_WIDE;
    q4k_gemm_tile<MTS, 2, 4, TYPE, false, true>(a, (blockIdx.x / tiles_n) * BMS, (blockIdx.x % tiles_n) * BN_WIDE);
}

// y[i] = partial[0][i] + partial[1][i] + ... in this order, whatever order the slices were written in.
__global__ __launch_bounds__(256) void split_sum_kernel(const float* __restrict__ partial, float* __restrict__ y, uint32_t count,
                                                        uint32_t splits) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= count) return;
    float v = partial[i];
    for (uint32_t s = 1; s < splits; ++s) v += partial[(size_t)s * count + i];
    y[i] = v;
}

// Slices of k for the small tiles (bm token rows x bn weight rows): doubled while the grid has fewer workgroups than
// the device has CUs (256) and a slice keeps at least four 256-element runs (sixteen stages, so that its prologue and
// epilogue stay a fraction of its work), up to eight slices; k must be whole runs for that.
// The slices actually cut are ceil(nsb / sb_per) with sb_per = ceil(nsb / s): for nsb that s does not divide this can be
// fewer than s (33 runs in eight slices of five: seven slices), and every slice then starts inside k, so no tile is
// handed an empty or negative range of super-blocks.
struct KSlices {
    uint32_t splits, sb_per;
};
inline KSlices small_tile_splits(uint32_t m, uint32_t n, uint32_t k, uint32_t bm, uint32_t bn) {
    const uint64_t tiles = (uint64_t)((m + bm - 1) / bm) * ((n + bn - 1) / bn);
    const uint32_t nsb = (k + 255u) / 256u;
    uint32_t s = 1;
    if (k % 256) return KSlices{1u, nsb};
    while (s < 8 && tiles * s < 256 && nsb / (2 * s) >= 4) s *= 2;
    const uint32_t sb_per = (nsb + s - 1) / s;
    return KSlices{(nsb + sb_per - 1) / sb_per, sb_per};  // (splits - 1) * sb_per < nsb
}

// The same for Q6_K and Q8_0 / Q4_0, up to 128 token rows: tiles of 128 token rows x 128 weight rows (four waves side by
// side, each 128 x 32; these tile bodies spread a k-step's four fragment words over MT >= 4 row tiles).
template <int TYPE, int MTS>  // MTS = 4: 128 token rows per tile (m <= 128); 8: 256
__global__ __launch_bounds__(64 * WAVES, 2) void mid_gemm_small_kernel(GemmArgs a, uint32_t splits, uint32_t sb_per,
                                                                       float* __restrict__ partial) {
    constexpr uint32_t BMS = 32 * MTS;
    const uint32_t tiles_n = (a.n + BN_WIDE - 1) / BN_WIDE, tiles_m = (a.m + BMS - 1) / BMS;
    const uint32_t s = blockIdx.x / (tiles_n * tiles_m), t = blockIdx.x % (tiles_n * tiles_m);
    if (splits > 1) {
        a.sb0 = s * sb_per;
        a.sb1 = a.sb0 + sb_per < a.sb1 ? a.sb0 + sb_per : a.sb1;
        a.y = partial + (size_t)s * a.m * a.n;
    }
    if constexpr (TYPE == HQ_Q6_K)
        q6k_gemm_tile<MTS, 4>(a, (t / tiles_n) * BMS, (t % tiles_n) * BN_WIDE);
    else
        q80_gemm_tile<MTS, 4, TYPE>(a, (t / tiles_n) * BMS, (t % tiles_n) * BN_WIDE);
}

__global__ __launch_bounds__(64 * WAVES, 2) void q6k_gemm_kernel(GemmArgs a) {
    const uint32_t tiles_m = (a.m + BM - 1) / BM;
    uint32_t m0, n0;
    if (!tile_of(blockIdx.x, tiles_m, (a.n + BN_WIDE - 1) / BN_WIDE, BN_WIDE, m0, n0)) return;
    q6k_gemm_tile<8, 4>(a, m0, n0);
}

template <int TYPE>
__global__ __launch_bounds__(64 * WAVES, 2) void q80_gemm_kernel(GemmArgs a) {
    const uint32_t tiles_m = (a.m + BM - 1) / BM;
    uint32_t m0, n0;
    if (!tile_of(blockIdx.x, tiles_m, (a.n + BN_WIDE - 1) / BN_WIDE, BN_WIDE, m0, n0)) return;
    q80_gemm_tile<8, 4, TYPE>(a, m0, n0);
}

// ---- grouped (expert) form -------------------------------------------------------------------
// Routed rows are sorted by expert; every expert's run of rows is cut into tiles of BM rows, and a
// workgroup multiplies one such tile with BN_WIDE weight rows of that expert.  Workspace beyond the
// dense layout (for P routed rows and n_experts * n weight rows): row_map[P], the tile table (one
// uint4 per tile: expert, first row, end of the expert's rows) and the tile count.
struct GroupedLayout {
    Workspace base;
    size_t row_map, tiles, count, total;
    uint32_t max_tiles;
};
// n_tokens converted activation rows (the tiles gather their routed rows' tokens from them), the scales of w_rows
// weight rows (n_experts * n, twice that for the SwiGLU form's two stacks), the permutation of the routed rows, the tiles.
__host__ __device__ inline GroupedLayout grouped_layout(uint32_t n_tokens, uint32_t pairs, uint32_t n_experts, uint32_t w_rows, uint32_t k) {
    GroupedLayout g;
    g.base = workspace_layout(n_tokens, w_rows, k);
    g.max_tiles = pairs / BM_SMALL + n_experts;  // enough for tiles of 64 rows or more
    g.row_map = g.base.total;
    g.tiles = g.row_map + (((size_t)pairs * 4 + 255) & ~(size_t)255);
    g.count = g.tiles + (((size_t)g.max_tiles * 16 + 255) & ~(size_t)255);
    g.total = g.count + 256;
    return g;
}

constexpr uint32_t BUCKET_MAX_EXPERTS = 1024;  // one expert per thread of the sort kernel (hq_moe_softmax_topk's limit too)

// One workgroup: counting sort of the routed rows by expert.  Rows whose id is not an expert get NaN
// outputs here and take no part in the product.  The order of the rows inside an expert's run depends
// on the order in which the atomics land; every output row is computed on its own, so the results do not.
// `stage` (LDS, `pairs` words, or null): the permutation is put together there and copied out in 16-byte pieces --
// one CU writes about one cache line per clock, and 16384 scattered 4-byte stores took 5.7 of this sort's 10.3 us.
constexpr uint32_t BUCKET_STAGE_MAX_PAIRS = 16384;  // 64 KB of LDS
struct BucketArgs {
    const uint32_t* ids;
    uint32_t pairs, n_experts;
    uint32_t* row_map;
    uint4* tiles;
    uint32_t* n_tiles;
    float* y;
    uint32_t n, bm;
    uint32_t half_tiles;  // a tile of at most bm / 2 rows is marked (tiles[].w = 1): the tile kernel runs it at half height
};
__device__ __forceinline__ void moe_bucket_sort(const BucketArgs& b, uint32_t* stage) {
    const uint32_t* __restrict__ ids = b.ids;
    uint32_t* __restrict__ row_map = b.row_map;
    uint4* __restrict__ tiles = b.tiles;
    uint32_t* __restrict__ n_tiles = b.n_tiles;
    float* __restrict__ y = b.y;
    const uint32_t pairs = b.pairs, n_experts = b.n_experts, n = b.n, bm = b.bm;
    __shared__ uint32_t cnt[BUCKET_MAX_EXPERTS], cur[BUCKET_MAX_EXPERTS];
    const uint32_t tid = threadIdx.x;
    for (uint32_t e = tid; e < n_experts; e += 1024) cnt[e] = 0;
    __syncthreads();
    // The ids are walked in batches of 16 per thread, four 16-byte loads in flight at once (one trip to memory per
    // 16384 ids instead of sixteen); ids that are not 16-byte aligned or not a multiple of four take single loads.
    const bool vec = pairs % 4u == 0 && (reinterpret_cast<uintptr_t>(ids) & 15u) == 0;
    auto for_each_id = [&](auto&& f) {  // f(position p, expert id)
        if (vec) {
            const uint4* ids4 = reinterpret_cast<const uint4*>(ids);
            const uint32_t quads = pairs / 4u;
            for (uint32_t q0 = 0; q0 < quads; q0 += 4096u) {
                uint4 v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t q = q0 + tid + 1024u * j;
                    v[j] = ids4[q < quads ? q : quads - 1u];
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t q = q0 + tid + 1024u * j;
                    if (q < quads) {
                        f(4u * q, v[j].x);
                        f(4u * q + 1u, v[j].y);
                        f(4u * q + 2u, v[j].z);
                        f(4u * q + 3u, v[j].w);
                    }
                }
            }
        } else {
            for (uint32_t p = tid; p < pairs; p += 1024) f(p, ids[p]);
        }
    };
    for_each_id([&](uint32_t, uint32_t e) {
        if (e < n_experts) atomicAdd(&cnt[e], 1u);
    });
    __syncthreads();
    // Exclusive prefix sums over the experts of (rows, tiles), one expert per thread (n_experts <= 1024 = the
    // workgroup): inside a wave by shuffles, across the sixteen waves through LDS.  Expert e then writes its own tiles.
    __shared__ uint32_t wave_rows[16], wave_tiles[16];
    const uint32_t my_rows = tid < n_experts ? cnt[tid] : 0u, my_tiles = (my_rows + bm - 1) / bm;
    uint32_t inc_rows = my_rows, inc_tiles = my_tiles;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t r = __shfl_up(inc_rows, d), t = __shfl_up(inc_tiles, d);
        if ((tid & 63u) >= (uint32_t)d) inc_rows += r, inc_tiles += t;
    }
    if ((tid & 63u) == 63u) wave_rows[tid >> 6] = inc_rows, wave_tiles[tid >> 6] = inc_tiles;
    __syncthreads();
    uint32_t off = inc_rows - my_rows, first_tile = inc_tiles - my_tiles, total_rows = 0, total_tiles = 0;
#pragma unroll
    for (uint32_t w = 0; w < 16; ++w) {
        if (w < (tid >> 6)) off += wave_rows[w], first_tile += wave_tiles[w];
        total_rows += wave_rows[w], total_tiles += wave_tiles[w];
    }
    if (tid < n_experts) {
        cur[tid] = off;
        for (uint32_t r = 0; r < my_rows; r += bm)
            tiles[first_tile + r / bm] = make_uint4(tid, off + r, off + my_rows, b.half_tiles && my_rows - r <= bm / 2u ? 1u : 0u);
    }
    if (tid == 0) *n_tiles = total_tiles;
    __syncthreads();
    for_each_id([&](uint32_t p, uint32_t e) {
        if (e < n_experts) {
            (stage ? stage : row_map)[atomicAdd(&cur[e], 1u)] = p;
        } else {
            for (uint32_t c = 0; c < n; ++c) y[(size_t)p * n + c] = __uint_as_float(0x7fc00000u);
        }
    });
    if (stage) {  // row_map is 16-byte aligned (an offset of the 256-byte aligned workspace that is a multiple of 256)
        __syncthreads();
        for (uint32_t r = 4u * tid; r < total_rows; r += 4096u) {
            if (r + 4u <= total_rows) {
                *reinterpret_cast<uint4*>(row_map + r) = *reinterpret_cast<const uint4*>(stage + r);
            } else {
                for (uint32_t i = r; i < total_rows; ++i) row_map[i] = stage[i];
            }
        }
    }
    // rows of the workspace past the sorted ones (invalid ids leave a gap at the end) point at row 0
    for (uint32_t r = total_rows + tid; r < pairs; r += 1024) row_map[r] = 0;
}

// The grouped form's pre-pass as ONE launch of 1024-thread workgroups: workgroup 0 sorts the routed rows by expert,
// the next ones convert the activation rows (one per token; four rows per workgroup, or sixteen, a wave each, when a
// row is at most 1024 values), the rest scan the scales of 1024 / weight_scan_lanes(k) weight rows each.  The sort is
// a single workgroup's work of about 13 us; beside the other two it costs nothing.
__host__ __device__ __forceinline__ uint32_t grouped_prep_rows_per_wg(uint32_t k) { return k <= 1024u ? 16u : 4u; }

template <bool X_BF16, int TYPE>
__global__ __launch_bounds__(1024) void grouped_prep_kernel(BucketArgs b, const void* __restrict__ x, const uint8_t* __restrict__ w,
                                                            const uint8_t* __restrict__ w2, uint8_t* __restrict__ ws, uint32_t m,
                                                            uint32_t n_rows, uint32_t k, uint32_t stage_words) {
    extern __shared__ __align__(16) uint32_t sort_stage[];  // b.pairs words for workgroup 0 when the launch brings them
    if (blockIdx.x == 0) {
        moe_bucket_sort(b, stage_words ? sort_stage : nullptr);
        return;
    }
    __shared__ float red[16];
    // (w2: a second stack of n_rows rows, scanned by workgroups of its own after the first stack's; its scales follow)
    const Workspace L = workspace_layout(m, w2 ? 2u * n_rows : n_rows, k);
    const uint32_t per_wg = grouped_prep_rows_per_wg(k), row_wgs = (m + per_wg - 1u) / per_wg, wg = blockIdx.x - 1u;
    if (wg < row_wgs) {
        if (per_wg == 16u)
            prep_activation_row<X_BF16, 64>(x, ws, L, m, k, 0u, wg * 16u + (threadIdx.x >> 6), threadIdx.x & 63u, red);
        else
            prep_activation_row<X_BF16, 256>(x, ws, L, m, k, 0u, wg * 4u + (threadIdx.x >> 8), threadIdx.x & 255u,
                                             red + 4u * (threadIdx.x >> 8));
    } else {
        const uint32_t lanes = weight_scan_lanes<TYPE>(k), per_scan_wg = 1024u / lanes;
        const uint32_t stack_wgs = (n_rows + per_scan_wg - 1u) / per_scan_wg;
        const uint32_t sw = wg - row_wgs, second = sw >= stack_wgs ? 1u : 0u;
        prep_weight_rows<TYPE>(second ? w2 : w, reinterpret_cast<float*>(ws + L.wdown) + second * n_rows, n_rows, k,
                               ((sw - second * stack_wgs) * 4u + (threadIdx.x >> 8)) * (256u / lanes), threadIdx.x & 255u, lanes);
    }
}

// A tile is 32 * MT routed rows (MT 8: 256 rows; 4: 128; 2: 64, Q4_K / Q5_K only) x 128 weight rows, a wave all its rows x 32.
template <int TYPE, int MT, bool SWIGLU = false>
__global__ __launch_bounds__(64 * WAVES, 2) void grouped_gemm_kernel(GemmArgs a, const uint4* __restrict__ tiles,
                                                                      const uint32_t* __restrict__ n_tiles, uint32_t tiles_n,
                                                                      uint64_t expert_stride) {
    // Workgroups go to the XCDs in turn (workgroup b to XCD b % 8), and every XCD has an L2 of its own: the tiles_n
    // workgroups that multiply the same routed rows with different weight rows are b = 8 (tiles_n q + i) + x for
    // i = 0 .. tiles_n - 1, all on XCD x and dispatched together, so the gathered activation rows cross the fabric
    // once instead of once per weight-row tile.
    const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
    const uint32_t t = (slot / tiles_n) * 8u + xcd, n0 = (slot % tiles_n) * BN_WIDE;
    if (t >= *n_tiles) return;
    const uint4 tt = tiles[t];
    a.w += (size_t)tt.x * expert_stride;
    a.wd_off = tt.x * a.n;
    a.m = tt.z;  // rows past the expert's run repeat its last row and are not stored
    if constexpr (SWIGLU) {  // Q4_K / Q5_K: gate and up of the same 32 weight rows per wave, silu(gate) * up stored
        a.w2 += (size_t)tt.x * expert_stride;
        q4k_gemm_tile<MT, 2, 4, TYPE, true, true>(a, tt.y, n0);
    } else if constexpr (TYPE == HQ_Q4_K || TYPE == HQ_Q5_K) {
        // the last tile of an expert, when at most half full, at half height (64 rows of 128: half of the MFMA work)
        if constexpr (MT == 4) {
            if (tt.w) {
                q4k_gemm_tile<2, 1, 4, TYPE, true>(a, tt.y, n0);
                return;
            }
        }
        q4k_gemm_tile<MT, 1, 4, TYPE, true>(a, tt.y, n0);
    } else if constexpr (TYPE == HQ_Q6_K)
        q6k_gemm_tile<MT, 4, true>(a, tt.y, n0);
    else
        q80_gemm_tile<MT, 4, TYPE, true>(a, tt.y, n0);
}

}  // namespace

// One token tile (m <= 256) takes the form whose k may be cut into slices: a single row of tiles seldom fills the device.
bool gemm_f16_small_tiles(hq_ggml_type t, uint32_t m) { return m <= (uint32_t)BM; }

// Slices of k the small tiles of type t cut the product into (1: none).
static KSlices small_slices_of(hq_ggml_type t, uint32_t m, uint32_t n, uint32_t k) {
    const uint32_t bm = (t == HQ_Q4_K || t == HQ_Q5_K) && m <= (uint32_t)BM_SMALL ? BM_SMALL : m <= (uint32_t)BM_MID ? BM_MID : BM;
    return small_tile_splits(m, n, k, bm, BN_WIDE);
}
static uint32_t small_splits_of(hq_ggml_type t, uint32_t m, uint32_t n, uint32_t k) { return small_slices_of(t, m, n, k).splits; }

void gemm_f16_small_tile_slices(hq_ggml_type t, uint32_t m, uint32_t n, uint32_t k, uint32_t* splits, uint32_t* sb_per) {
    const KSlices ks = small_slices_of(t, m, n, k);
    *splits = ks.splits;
    *sb_per = ks.sb_per;
}

bool gemm_f16_tile_gated_supported(hq_ggml_type t, uint32_t m, uint32_t n, uint32_t k) {
    return gemm_f16_tile_supported(t, k) && !(gemm_f16_small_tiles(t, m) && small_splits_of(t, m, n, k) > 1);
}

size_t gemm_f16_tile_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t) {
    size_t total = workspace_layout(m, n, k).total;
    if (gemm_f16_small_tiles(t, m)) {  // partial sums of the slices of k
        const uint32_t splits = small_splits_of(t, m, n, k);
        if (splits > 1) total += (size_t)splits * m * n * 4;
    }
    return total;
}

bool gemm_f16_grouped_supported(hq_ggml_type t, uint32_t n, uint32_t k, uint32_t n_experts, uint64_t expert_stride, uint64_t pairs) {
    if (!gemm_f16_tile_supported(t, k) || n_experts > BUCKET_MAX_EXPERTS || pairs > 0x7fffffffull / 4) return false;
    const uint64_t row_bytes = t == HQ_Q4_K   ? (uint64_t)(k / 256) * Q4K_BYTES
                               : t == HQ_Q5_K ? (uint64_t)(k / 256) * Q5K_BYTES
                               : t == HQ_Q6_K ? (uint64_t)(k / 256) * Q6K_BYTES
                               : t == HQ_Q4_0 ? (uint64_t)(k / 32) * Q4_0_BYTES
                                              : (uint64_t)(k / 32) * Q8_0_BYTES;
    // the pre-pass walks the stack as one matrix of n_experts * n rows
    return expert_stride == (uint64_t)n * row_bytes && (uint64_t)n_experts * n <= 0x7fffffffull;
}

size_t gemm_f16_grouped_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t n_experts, uint32_t n, uint32_t k,
                                        uint32_t stacks) {
    return grouped_layout(n_tokens, n_tokens * top_k, n_experts, stacks * n_experts * n, k).total;
}

// The SwiGLU form (two stacks, silu(gate) * up stored) exists for the Q4_K / Q5_K tiles, whose waves take two weight
// tiles side by side.
bool gemm_f16_grouped_swiglu_supported(hq_ggml_type t) { return t == HQ_Q4_K || t == HQ_Q5_K; }

template <int TYPE>
static int launch_prep(hipStream_t s, const void* x, hq_act_dtype xdt, const uint8_t* wb, uint8_t* ws, uint32_t m,
                       uint32_t n, uint32_t k, uint32_t perm_hd, bool scan_weights, const uint8_t* wb2 = nullptr) {
    const uint32_t rows_per_wg = 256u / weight_scan_lanes<TYPE>(k);
    const uint32_t scan_wgs = scan_weights ? (wb2 ? 2u : 1u) * ((n + rows_per_wg - 1u) / rows_per_wg) : 0u;
    const dim3 prep_grid(scan_wgs + m);
    if (xdt == HQ_BF16)
        hipLaunchKernelGGL((tile_prep_kernel<true, TYPE>), prep_grid, dim3(256), 0, s, x, wb, wb2, ws, m, n, k, perm_hd, scan_wgs);
    else
        hipLaunchKernelGGL((tile_prep_kernel<false, TYPE>), prep_grid, dim3(256), 0, s, x, wb, wb2, ws, m, n, k, perm_hd, scan_wgs);
    return check_launch("tile gemm pre-pass launch");
}

template <int TYPE>
static int launch_grouped_t(hipStream_t s, const void* x, hq_act_dtype xdt, const uint8_t* wb, const uint32_t* ids, float* y,
                            uint8_t* ws, uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k, uint32_t n_experts,
                            uint64_t expert_stride, const float* w_scales, const uint8_t* wb2, const float* w_scales2) {
    // wb2: the SwiGLU form, y = silu(W[ids] . x) * (W2[ids] . x); Q4_K / Q5_K only (the caller has checked)
    const uint32_t pairs = n_tokens * top_k;
    const GroupedLayout G = grouped_layout(n_tokens, pairs, n_experts, (wb2 ? 2u : 1u) * n_experts * n, k);
    uint32_t* row_map = reinterpret_cast<uint32_t*>(ws + G.row_map);
    uint4* tiles = reinterpret_cast<uint4*>(ws + G.tiles);
    uint32_t* n_tiles = reinterpret_cast<uint32_t*>(ws + G.count);
    // Experts with few rows each take smaller tiles (Qwen3.6-35B-A3B: 2048 tokens x top-8 over 256 experts = 64 rows per
    // expert on average, tiles of 128 routed rows: the 256-row tiles would run a quarter full, and half of the experts
    // would need two 64-row tiles); at 40 rows per expert or fewer the Q4_K / Q5_K tiles of 64 rows.
    constexpr bool HAS_64 = TYPE == HQ_Q4_K || TYPE == HQ_Q5_K;
    // (the SwiGLU form keeps two accumulator tiles per row tile: 128 rows is the most a wave's registers hold, and with
    // Q5_K's high-bit words beside them 64 rows -- its 128-row form spills 42 registers)
    const int mt = (HAS_64 && (uint64_t)pairs <= (uint64_t)n_experts * 40u) || (wb2 && TYPE == HQ_Q5_K) ? 2
                   : (uint64_t)pairs < (uint64_t)n_experts * 160u || wb2                              ? 4
                                                                                                      : 8;
    const uint32_t bm = 32u * (uint32_t)mt, bn = BN_WIDE;
    // sort by expert + one converted activation row per token (the tiles gather the rows of their routed rows from
    // them) + the weight rows' scales, in one launch
    const BucketArgs b{ids, pairs, n_experts, row_map, tiles, n_tiles, y, n, bm, HAS_64 && mt == 4 && !wb2 ? 1u : 0u};
    const uint32_t n_rows = n_experts * n;
    const uint32_t act_per_wg = grouped_prep_rows_per_wg(k), w_per_wg = 1024u / weight_scan_lanes<TYPE>(k);
    const dim3 prep_grid(1u + (n_tokens + act_per_wg - 1u) / act_per_wg +
                         (w_scales ? 0u : (wb2 ? 2u : 1u) * ((n_rows + w_per_wg - 1u) / w_per_wg)));  // the weight workgroups come last
    // up to 16384 routed rows: the sort stages its permutation in LDS (two workgroups of this launch still share a CU)
    const uint32_t stage_words = pairs <= BUCKET_STAGE_MAX_PAIRS ? (pairs + 3u) & ~3u : 0u;
    void (*prep)(BucketArgs, const void*, const uint8_t*, const uint8_t*, uint8_t*, uint32_t, uint32_t, uint32_t, uint32_t) =
        xdt == HQ_BF16 ? grouped_prep_kernel<true, TYPE> : grouped_prep_kernel<false, TYPE>;
    // (the kernel's static LDS, under 16 KB, counts towards the 64 KB a launch may use without the attribute)
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(prep), stage_words ? (size_t)stage_words * 4 + 16384 : 0,
                                  "hipFuncSetAttribute(grouped pre-pass LDS)"))
        return rc;
    hipLaunchKernelGGL(prep, prep_grid, dim3(1024), stage_words * 4, s, b, x, wb, wb2, ws, n_tokens, n_rows, k, stage_words);
    if (int rc = check_launch("grouped gemm pre-pass launch")) return rc;
    const int lds = 2 * (mt == 2 ? ActTileT<BM_SMALL>::kTile : mt == 4 ? ActTileT<BM_MID>::kTile : ActTile::kTile);
    void (*kern)(GemmArgs, const uint4*, const uint32_t*, uint32_t, uint64_t) = grouped_gemm_kernel<TYPE, 8>;
    if (mt == 4) kern = grouped_gemm_kernel<TYPE, 4>;
    if constexpr (HAS_64) {
        if (mt == 2) kern = grouped_gemm_kernel<TYPE, 2>;
        if (wb2) {
            kern = grouped_gemm_kernel<TYPE, 2, true>;
            if constexpr (TYPE == HQ_Q4_K)
                if (mt == 4) kern = grouped_gemm_kernel<TYPE, 4, true>;
        }
    }
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), (size_t)lds, "hipFuncSetAttribute(grouped gemm LDS)"))
        return rc;
    const float* ws_scales = reinterpret_cast<const float*>(ws + G.base.wdown);  // the pre-pass's: first stack, then second
    GemmArgs a{ws, wb, y, pairs, n, k, n_tokens, (wb2 ? 2u : 1u) * n_rows, 0u, row_map, 0u, (k + 255u) / 256u, top_k,
               w_scales ? w_scales : ws_scales, wb2, wb2 ? (w_scales ? w_scales2 : ws_scales + n_rows) : nullptr};
    const uint32_t tiles_n = (n + bn - 1) / bn;
    const uint32_t max_tiles = pairs / bm + n_experts;
    hipLaunchKernelGGL(kern, dim3(((max_tiles + 7u) & ~7u) * tiles_n), dim3(64 * WAVES), lds, s, a, tiles, n_tiles, tiles_n, expert_stride);
    return check_launch("grouped gemm kernel launch");
}

int launch_weight_row_scales(hipStream_t s, const void* w, float* scales, uint32_t n_rows, uint32_t k, hq_ggml_type t) {
    const uint8_t* wb = static_cast<const uint8_t*>(w);
    auto go = [&](auto tag) {
        constexpr int TYPE = decltype(tag)::value;
        const uint32_t per_wg = 256u / weight_scan_lanes<TYPE>(k);
        hipLaunchKernelGGL((weight_scales_kernel<TYPE>), dim3((n_rows + per_wg - 1u) / per_wg), dim3(256), 0, s, wb, scales, n_rows, k);
        return check_launch("weight row scales launch");
    };
    switch (t) {
        case HQ_Q4_K: return go(std::integral_constant<int, HQ_Q4_K>{});
        case HQ_Q5_K: return go(std::integral_constant<int, HQ_Q5_K>{});
        case HQ_Q6_K: return go(std::integral_constant<int, HQ_Q6_K>{});
        case HQ_Q8_0: return go(std::integral_constant<int, HQ_Q8_0>{});
        case HQ_Q4_0: return go(std::integral_constant<int, HQ_Q4_0>{});
    }
    return fail(HQ_ERR_UNSUPPORTED, "weight row scales: ggml type %d", (int)t);
}

int launch_gemm_f16_grouped(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_stack, const uint32_t* ids, float* y,
                            void* workspace, uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k, uint32_t n_experts,
                            uint64_t expert_stride, hq_ggml_type t, const float* w_scales, const void* w_stack2,
                            const float* w_scales2) {
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    const uint8_t* wb2 = static_cast<const uint8_t*>(w_stack2);
    if (wb2 && !gemm_f16_grouped_swiglu_supported(t)) return fail(HQ_ERR_UNSUPPORTED, "grouped gemm, SwiGLU form: ggml type %d", (int)t);
    const uint8_t* wb = static_cast<const uint8_t*>(w_stack);
    switch (t) {
        case HQ_Q4_K: return launch_grouped_t<HQ_Q4_K>(s, x, xdt, wb, ids, y, ws, n_tokens, top_k, n, k, n_experts, expert_stride, w_scales, wb2, w_scales2);
        case HQ_Q5_K: return launch_grouped_t<HQ_Q5_K>(s, x, xdt, wb, ids, y, ws, n_tokens, top_k, n, k, n_experts, expert_stride, w_scales, wb2, w_scales2);
        case HQ_Q6_K: return launch_grouped_t<HQ_Q6_K>(s, x, xdt, wb, ids, y, ws, n_tokens, top_k, n, k, n_experts, expert_stride, w_scales, nullptr, nullptr);
        case HQ_Q8_0: return launch_grouped_t<HQ_Q8_0>(s, x, xdt, wb, ids, y, ws, n_tokens, top_k, n, k, n_experts, expert_stride, w_scales, nullptr, nullptr);
        case HQ_Q4_0: return launch_grouped_t<HQ_Q4_0>(s, x, xdt, wb, ids, y, ws, n_tokens, top_k, n, k, n_experts, expert_stride, w_scales, nullptr, nullptr);
    }
    return fail(HQ_ERR_UNSUPPORTED, "grouped gemm: ggml type %d", (int)t);
}

bool gemm_f16_tile_supported(hq_ggml_type t, uint32_t k) {
    return ((t == HQ_Q4_K || t == HQ_Q5_K || t == HQ_Q6_K) && k % 256 == 0) || ((t == HQ_Q8_0 || t == HQ_Q4_0) && k % 128 == 0);
}

size_t gemm_f16_swiglu_workspace_bytes(uint32_t m, uint32_t n, uint32_t k) { return workspace_layout(m, 2u * n, k).total; }

// y[m, n] = silu(x . Wg^T) * (x . Wu^T), Q4_K / Q5_K, k % 256 == 0: the activation pre-pass once (with both matrices'
// row scales unless the caller brings them) and one launch of tiles that multiply the same activation rows with both
// matrices.  Tiles of 64 token rows while those leave CUs idle, of 128 beyond.
int launch_gemm_f16_swiglu(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up, float* y, uint32_t m,
                           uint32_t n, uint32_t k, hq_ggml_type t, void* workspace, const float* gate_scales, const float* up_scales) {
    if (t != HQ_Q4_K && t != HQ_Q5_K) return fail(HQ_ERR_UNSUPPORTED, "tile gemm, SwiGLU form: ggml type %d", (int)t);
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    const uint8_t *wg = static_cast<const uint8_t*>(w_gate), *wu = static_cast<const uint8_t*>(w_up);
    if (int rc = t == HQ_Q5_K ? launch_prep<HQ_Q5_K>(s, x, xdt, wg, ws, m, n, k, 0, !gate_scales, wu)
                              : launch_prep<HQ_Q4_K>(s, x, xdt, wg, ws, m, n, k, 0, !gate_scales, wu))
        return rc;
    const float* ws_scales = reinterpret_cast<const float*>(ws + workspace_layout(m, 2u * n, k).wdown);
    GemmArgs a{ws, wg, y, m, n, k, m, 2u * n, 0u, nullptr, 0u, (k + 255u) / 256u, 0u,
               gate_scales ? gate_scales : ws_scales, wu, gate_scales ? up_scales : ws_scales + n};
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    const uint32_t tiles_n = (n + BN_WIDE - 1) / BN_WIDE;
    const bool small = t == HQ_Q5_K || (uint64_t)((m + BM_MID - 1) / BM_MID) * tiles_n < cus;  // (Q5_K's 128-row form spills)
    void (*kern)(GemmArgs) = t == HQ_Q5_K ? q4k_swiglu_kernel<HQ_Q5_K, 2>
                                          : (small ? q4k_swiglu_kernel<HQ_Q4_K, 2> : q4k_swiglu_kernel<HQ_Q4_K, 4>);
    const uint32_t bm = small ? BM_SMALL : BM_MID;
    const int lds = 2 * (small ? ActTileT<BM_SMALL>::kTile : ActTileT<BM_MID>::kTile);
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), (size_t)lds, "hipFuncSetAttribute(swiglu gemm LDS)")) return rc;
    hipLaunchKernelGGL(kern, dim3(((m + bm - 1) / bm) * tiles_n), dim3(64 * WAVES), lds, s, a);
    return check_launch("swiglu gemm kernel launch");
}

int launch_gemm_f16_tile(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m,
                         uint32_t n, uint32_t k, hq_ggml_type t, void* workspace, uint32_t perm_hd, const float* w_scales,
                         const float* gate_in) {
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    const uint8_t* wb = static_cast<const uint8_t*>(w);
    GemmArgs a{ws, wb, y, m, n, k, m, n, 0u, nullptr, 0u, (k + 255u) / 256u, 0u,
               w_scales ? w_scales : reinterpret_cast<const float*>(ws + workspace_layout(m, n, k).wdown), nullptr, nullptr, gate_in};
    // (the forms that cut k into slices add partial products: the gating cannot go into their epilogue)
    if (gate_in && gemm_f16_small_tiles(t, m) && small_splits_of(t, m, n, k) > 1)
        return fail(HQ_ERR_UNSUPPORTED, "tile gemm with a gated epilogue: this shape is cut into slices of k");
    constexpr int lds = 2 * ActTile::kTile;
    const uint32_t tiles_m = (m + BM - 1) / BM, cols_wide = (n + BN_WIDE - 1) / BN_WIDE;
    // up to 256 token rows of Q6_K / Q8_0 / Q4_0: one token tile of 128 or 256 rows x 128 weight rows, k in slices where
    // that leaves CUs idle
    auto launch_mid_small = [&](void (*k128)(GemmArgs, uint32_t, uint32_t, float*),
                                void (*k256)(GemmArgs, uint32_t, uint32_t, float*)) -> int {
        const bool one128 = m <= (uint32_t)BM_MID;
        void (*kern)(GemmArgs, uint32_t, uint32_t, float*) = one128 ? k128 : k256;
        const uint32_t tn = (n + BN_WIDE - 1) / BN_WIDE;
        const KSlices ks = small_slices_of(t, m, n, k);
        const uint32_t splits = ks.splits, sb_per = ks.sb_per;
        float* partial = reinterpret_cast<float*>(ws + workspace_layout(m, n, k).total);
        const int lds_small = 2 * (one128 ? ActTileT<BM_MID>::kTile : ActTile::kTile);
        if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), (size_t)lds_small, "hipFuncSetAttribute(small gemm LDS)"))
            return rc;
        hipLaunchKernelGGL(kern, dim3(tn * splits), dim3(64 * WAVES), lds_small, s, a, splits, sb_per, partial);
        if (int rc = check_launch("small gemm kernel launch")) return rc;
        if (splits == 1) return HQ_OK;
        const uint32_t count = m * n;  // m <= 256
        hipLaunchKernelGGL(split_sum_kernel, dim3((count + 255u) / 256u), dim3(256), 0, s, partial, y, count, splits);
        return check_launch("split sum kernel launch");
    };
    if (t == HQ_Q6_K) {
        if (int rc = launch_prep<HQ_Q6_K>(s, x, xdt, wb, ws, m, n, k, perm_hd, !w_scales)) return rc;
        if (gemm_f16_small_tiles(t, m)) return launch_mid_small(mid_gemm_small_kernel<HQ_Q6_K, 4>, mid_gemm_small_kernel<HQ_Q6_K, 8>);
        if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(q6k_gemm_kernel), (size_t)lds, "hipFuncSetAttribute(q6_k gemm LDS)"))
            return rc;
        hipLaunchKernelGGL(q6k_gemm_kernel, dim3(tile_grid(tiles_m, cols_wide)), dim3(64 * WAVES), lds, s, a);
        return check_launch("q6_k gemm kernel launch");
    }
    if (t == HQ_Q8_0 || t == HQ_Q4_0) {
        void (*kern)(GemmArgs) = t == HQ_Q4_0 ? q80_gemm_kernel<HQ_Q4_0> : q80_gemm_kernel<HQ_Q8_0>;
        if (int rc = t == HQ_Q4_0 ? launch_prep<HQ_Q4_0>(s, x, xdt, wb, ws, m, n, k, perm_hd, !w_scales)
                                  : launch_prep<HQ_Q8_0>(s, x, xdt, wb, ws, m, n, k, perm_hd, !w_scales))
            return rc;
        if (gemm_f16_small_tiles(t, m))
            return t == HQ_Q4_0 ? launch_mid_small(mid_gemm_small_kernel<HQ_Q4_0, 4>, mid_gemm_small_kernel<HQ_Q4_0, 8>)
                                : launch_mid_small(mid_gemm_small_kernel<HQ_Q8_0, 4>, mid_gemm_small_kernel<HQ_Q8_0, 8>);
        if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), (size_t)lds, "hipFuncSetAttribute(q8_0 gemm LDS)"))
            return rc;
        hipLaunchKernelGGL(kern, dim3(tile_grid(tiles_m, cols_wide)), dim3(64 * WAVES), lds, s, a);
        return check_launch("q8_0 gemm kernel launch");
    }
    if (int rc = t == HQ_Q5_K ? launch_prep<HQ_Q5_K>(s, x, xdt, wb, ws, m, n, k, perm_hd, !w_scales)
                              : launch_prep<HQ_Q4_K>(s, x, xdt, wb, ws, m, n, k, perm_hd, !w_scales))
        return rc;
    if (gemm_f16_small_tiles(t, m)) {  // Q4_K / Q5_K: one token tile of 64, 128 or 256 rows, tiles of 128 weight rows
        const int mts = m <= (uint32_t)BM_SMALL ? 2 : m <= (uint32_t)BM_MID ? 4 : 8;
        void (*ksmall)(GemmArgs, uint32_t, uint32_t, float*) =
            t == HQ_Q5_K ? (mts == 2 ? q4k_gemm_small_kernel<HQ_Q5_K, 2> : mts == 4 ? q4k_gemm_small_kernel<HQ_Q5_K, 4> : q4k_gemm_small_kernel<HQ_Q5_K, 8>)
                         : (mts == 2 ? q4k_gemm_small_kernel<HQ_Q4_K, 2> : mts == 4 ? q4k_gemm_small_kernel<HQ_Q4_K, 4> : q4k_gemm_small_kernel<HQ_Q4_K, 8>);
        const uint32_t tn = (n + BN_WIDE - 1) / BN_WIDE;
        const KSlices ks = small_slices_of(t, m, n, k);
        const uint32_t splits = ks.splits, sb_per = ks.sb_per;
        float* partial = reinterpret_cast<float*>(ws + workspace_layout(m, n, k).total);
        const int lds_small = 2 * (mts == 2 ? ActTileT<BM_SMALL>::kTile : mts == 4 ? ActTileT<BM_MID>::kTile : ActTile::kTile);
        if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(ksmall), (size_t)lds_small, "hipFuncSetAttribute(q4k small gemm LDS)"))
            return rc;
        hipLaunchKernelGGL(ksmall, dim3(tn * splits), dim3(64 * WAVES), lds_small, s, a, splits, sb_per, partial);
        if (int rc = check_launch("q4k small gemm kernel launch")) return rc;
        if (splits == 1) return HQ_OK;
        const uint32_t count = m * n;  // m <= 256
        hipLaunchKernelGGL(split_sum_kernel, dim3((count + 255u) / 256u), dim3(256), 0, s, partial, y, count, splits);
        return check_launch("split sum kernel launch");
    }
    void (*kern)(GemmArgs, uint32_t, uint32_t) = t == HQ_Q5_K ? q4k_gemm_kernel<HQ_Q5_K> : q4k_gemm_kernel<HQ_Q4_K>;
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), (size_t)lds, "hipFuncSetAttribute(q4k gemm LDS)"))
        return rc;
    // Tiles of 128 weight rows; tiles of 64 when the wide ones would occupy at most half of the CUs.
    // (Cutting only the last, partly filled round of a large problem into narrow tiles was measured:
    // no gain, the narrow tiles pay the double dequantisation.)
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    const uint32_t cols_narrowed = (uint64_t)tiles_m * cols_wide <= cus / 2 ? cols_wide : 0;  // columns cut in two
    const uint32_t n_wide = (cols_wide - cols_narrowed) * BN_WIDE;  // < n whenever cols_narrowed > 0
    const uint32_t cols_narrow = n_wide < n ? (n - n_wide + BN_NARROW - 1) / BN_NARROW : 0;
    const uint32_t grid_wide = tile_grid(tiles_m, cols_wide - cols_narrowed), grid_narrow = tile_grid(tiles_m, cols_narrow);
    hipLaunchKernelGGL(kern, dim3(grid_wide + grid_narrow), dim3(64 * WAVES), lds, s, a, n_wide, grid_wide);
    return check_launch("q4k gemm kernel launch");
}

}  // namespace hq

// Dequant-fused product for 2..8 activation rows over the 32-weight-block types (Q8_0, Q4_0):
// y[m, n] = sum_k x[m, k] * W[n, k] with every weight fetched once for all rows, where the GEMV kernel would fetch
// it once per row.  Every product is exact, as in the GEMV (v_cvt of the integer weight, v_fma in fp32).
//
// One workgroup of 16 waves per CU.  k is walked in chunks of 2048 activations = 64 blocks of a row, one block per
// lane.  For a chunk, the workgroup stages all rows of x in LDS as f32 (bf16 input is widened, which is exact), each
// lane's 32 activations of a row in a 144-byte slot: the 16-byte pad makes the slots of 16 consecutive lanes start
// in 16 different bank groups, so the 16-byte reads of a wave are conflict-free.  Then every wave walks its weight
// rows, row (i * 16 + wave) * grid + block, with one block per lane in flight; the integer-to-float conversion of a
// block is shared by the activation rows, the multiply-adds are per row.  A row's partial sum over the chunk is
// reduced across the 64 lanes and added to y by lane 0: stored for the first chunk, added (hardware float atomic,
// the only writer of that address, in chunk order: deterministic) for the later ones.
#include "gemv_pieces.h"

namespace hq {

namespace {

struct R32Args {
    const void* x;
    const uint8_t* w;
    float* y;
    uint32_t m, n, k;
};

constexpr uint32_t R32_WAVES = 16;
constexpr uint32_t R32_KC = 2048;                  // activations of a row per staged chunk: 64 blocks
constexpr uint32_t R32_SLOT = 9;                   // float4 per (row, lane) slot: 8 of data + 1 of pad
constexpr uint32_t R32_ROW4 = 64 * R32_SLOT;       // float4 per staged row

template <int R>
constexpr uint32_t kR32LdsBytes = R * R32_ROW4 * 16 + R * 64 * 4;  // activations, then the per-block sums

template <int TYPE, bool X_BF16, int R>
__global__ __launch_bounds__(64 * R32_WAVES) void rows32_kernel(R32Args a) {
    constexpr uint32_t BB = kBlockBytes<TYPE>;
    constexpr uint32_t NT = 64 * R32_WAVES;
    extern __shared__ float4 r32_smem[];
    float4* xs = r32_smem;
    float* ss = reinterpret_cast<float*>(xs + R * R32_ROW4);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wv = tid >> 6;
    const uint32_t nblk = a.k / 32u, rowb = nblk * BB;
    const uint32_t nch = (a.k + R32_KC - 1u) / R32_KC;
    const uint32_t stride = R32_WAVES * gridDim.x;
    const uint32_t row_first = wv * gridDim.x + blockIdx.x;
    const uint32_t rows_mine = row_first < a.n ? (a.n - row_first + stride - 1u) / stride : 0u;

    Piece<TYPE> pc;
    auto fetch = [&](uint32_t row, uint32_t ch) {
        // blocks past the end of a short last chunk read the row's last block; their activations are staged as zeros
        const uint32_t b = ch * 64u + lane;
        pc.load(a.w + (size_t)row * rowb + (size_t)(b < nblk ? b : nblk - 1u) * BB, 0);
    };

    for (uint32_t ch = 0; ch < nch; ++ch) {
        if (rows_mine) fetch(row_first, ch);  // in flight while the chunk is staged
        if (ch) __syncthreads();              // every wave is done with the previous chunk's activations
        // ---- stage: thread f of a pass takes four consecutive activations (lane slot f / 8, part f % 8) of row r ----
#pragma unroll
        for (uint32_t it = 0; it < (R * 512u + NT - 1u) / NT; ++it) {
            const uint32_t idx = it * NT + tid;           // < R * 512 where it matters
            const uint32_t r = idx >> 9, f = idx & 511u;  // row, float4 within the chunk
            const uint32_t e0 = ch * R32_KC + 4u * f;     // first of the four activations
            // no branch around the load: rows past m and activations past k read a valid address and are zeroed
            const bool live = r < a.m && e0 < a.k && idx < R * 512u;
            const uint32_t rr = r < a.m ? r : a.m - 1u, ee = e0 < a.k ? e0 : 0u;
            const uint32_t keep = live ? 0xffffffffu : 0u;
            float4 v;
            if constexpr (X_BF16) {
                const uint2 u = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(a.x) + (size_t)rr * a.k + ee);
                v = make_float4(__uint_as_float((u.x << 16) & keep), __uint_as_float((u.x & 0xffff0000u) & keep),
                                __uint_as_float((u.y << 16) & keep), __uint_as_float((u.y & 0xffff0000u) & keep));
            } else {
                const uint4 u = *reinterpret_cast<const uint4*>(static_cast<const float*>(a.x) + (size_t)rr * a.k + ee);
                v = make_float4(__uint_as_float(u.x & keep), __uint_as_float(u.y & keep), __uint_as_float(u.z & keep),
                                __uint_as_float(u.w & keep));
            }
            if (idx < R * 512u) xs[r * R32_ROW4 + (f >> 3) * R32_SLOT + (f & 7u)] = v;
            if constexpr (TYPE == HQ_Q4_0) {
                // sum of a block's 32 activations (for the -8 d sum x term): four here, then across the eight threads
                // of the block
                float s = (v.x + v.y) + (v.z + v.w);
                s = dpp_add<0xB1>(s);
                s = dpp_add<0x4E>(s);
                s = dpp_add<0x141>(s);
                if ((f & 7u) == 0 && idx < R * 512u) ss[r * 64u + (f >> 3)] = s;
            }
        }
        __syncthreads();

        // ---- this wave's rows over the chunk ----
        uint32_t row = row_first;
        for (uint32_t i = 0; i < rows_mine; ++i, row += stride) {
            float part[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float xf[32], sx[2] = {0.f, 0.f};
                const float4* src = xs + r * R32_ROW4 + lane * R32_SLOT;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float4 t = src[j];
                    xf[4 * j] = t.x, xf[4 * j + 1] = t.y, xf[4 * j + 2] = t.z, xf[4 * j + 3] = t.w;
                }
                if constexpr (TYPE == HQ_Q4_0) sx[0] = ss[r * 64u + lane];
                part[r] = dot_f32(pc, 0, xf, sx);
            }
            if (i + 1 < rows_mine) {
#pragma unroll
                for (int r = 0; r < R; ++r) asm volatile("" : "+v"(part[r]));  // the refill follows the arithmetic
                fetch(row + stride, ch);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float v = group_sum(part[r], 6);
                if (lane == 0 && (uint32_t)r < a.m) {
                    float* dst = a.y + (size_t)r * a.n + row;
                    if (ch == 0)
                        *dst = v;
                    else
                        unsafeAtomicAdd(dst, v);
                }
            }
        }
    }
}

template <int TYPE, bool X_BF16>
int launch_r32_t(hipStream_t s, const R32Args& a) {
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    const uint32_t groups = (a.n + R32_WAVES - 1u) / R32_WAVES;
    const dim3 grid(groups < cus ? groups : cus);
    void (*kern)(R32Args);
    size_t lds;
    if (a.m <= 2) {
        kern = rows32_kernel<TYPE, X_BF16, 2>;
        lds = kR32LdsBytes<2>;
    } else if (a.m <= 4) {
        kern = rows32_kernel<TYPE, X_BF16, 4>;
        lds = kR32LdsBytes<4>;
    } else {
        kern = rows32_kernel<TYPE, X_BF16, 8>;
        lds = kR32LdsBytes<8>;
    }
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, "hipFuncSetAttribute(rows kernel LDS)")) return rc;
    hipLaunchKernelGGL(kern, grid, dim3(64 * R32_WAVES), lds, s, a);
    return check_launch("rows kernel launch (32-weight blocks)");
}

}  // namespace

// Q8_0 / Q4_0, 2 <= m <= 8, any k (a multiple of the block size).
bool gemv_rows32_supported(hq_ggml_type t, uint32_t m, uint32_t k) {
    return (t == HQ_Q8_0 || t == HQ_Q4_0) && m >= 2 && m <= 8 && k % 32 == 0 && k >= 32;
}

int launch_gemv_rows32(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w, float* y, uint32_t m, uint32_t n,
                       uint32_t k, hq_ggml_type t) {
    const R32Args a{x, static_cast<const uint8_t*>(w), y, m, n, k};
    const bool bf = xdt == HQ_BF16;
    if (t == HQ_Q8_0) return bf ? launch_r32_t<HQ_Q8_0, true>(s, a) : launch_r32_t<HQ_Q8_0, false>(s, a);
    return bf ? launch_r32_t<HQ_Q4_0, true>(s, a) : launch_r32_t<HQ_Q4_0, false>(s, a);
}

}  // namespace hq

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
#include <mutex>

#include "hq_internal.h"
#include "moe_topk.h"
#include "gemv_pieces.h"
#include "gemv_walk.h"

namespace hq {

namespace {

// Tasks (row slot x step) per CU from which the queue kernel takes over.
constexpr uint32_t QUEUE_MIN_TASKS_PER_CU = 96;

struct KArgs {
    const void* x;
    const void* x2;  // f32 only, may be null: the activations are silu(x) * x2
    const uint8_t* w;
    const uint32_t* ids;
    const float* route_logits;  // see GemvArgs
    uint32_t* route_ids;
    float* route_w;
    float* y;
    uint32_t top_k, n, k, n_experts;
    uint64_t expert_stride;
    uint32_t log_l;   // log2 of the lanes that share one row
    uint32_t groups;  // row groups (one group = the rows a workgroup covers in one pass)
    uint32_t pairs;   // activation-row / output-row pairs (grid.y of the job)
    uint32_t xpad;    // zeros staged behind the activations (elements): what the lanes past a row's last piece multiply with
    // Bit masks of the nibble -> bf16 conversion.  They are passed as arguments and
    // not written as literals so that the compiler keeps them in registers and
    // forms the three-operand v_and_or_b32 (gfx9 VOP3 takes no literals; with
    // literals it emits v_and + v_or instead).
    uint32_t m4, m2, magic;
};

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

// ---- the per-wave walk ------------------------------------------------------
// A wave owns NR "row slots" (a slot = the 64/L rows its lanes cover at once) of a
// wave group and walks the (step, slot) tasks in step-major order with D weight
// fetches in flight: the fetch for task t+D is issued right after task t has
// consumed its registers, and the ring runs on into the wave's next wave group,
// so the stream of fetches does not drain between groups.  The activations of a
// step stay in registers for all NR slots.  NR % D == 0 keeps every buffer index
// static.  Rows past the end are clamped to the last row (always a valid read;
// its result is not stored).
template <int TYPE, bool X_BF16, bool PAIR, int NR, int D>
struct Walk {
    static_assert(NR % D == 0, "buffer rotation must repeat per step");
    static constexpr int EPL = Lane<TYPE>::kElems;
    static constexpr uint32_t BYTES = kBlockBytes<TYPE>;
    static constexpr int XW = PAIR ? EPL / 2 : EPL;  // LDS words per piece

    const uint8_t* w;  // weight base + this lane's piece offset at step 0
    const uint32_t* lds_x;
    const float* lds_s;
    uint32_t n, log_l, rpw, lane, li, steps, row_bytes, bstep, lane_row, pieces, nblk, blk0;
    int c;
    uint32_t m4, m2, magic;
    Piece<TYPE> buf[D];

    __device__ __forceinline__ void init(const KArgs& a, const uint8_t* wbase, const uint32_t* lx, const float* ls) {
        lane = threadIdx.x & 63u;
        n = a.n;
        log_l = a.log_l;
        const uint32_t L = 1u << log_l;
        rpw = 64u >> log_l;
        li = lane & (L - 1u);
        lane_row = lane >> log_l;
        // pieces per row / L, rounded up: in the last step of a row whose pieces L does not divide, the lanes past the end fetch
        // the row's last block again and multiply it with the zeros staged behind the activations
        pieces = a.k / EPL;
        steps = (pieces + L - 1u) >> log_l;
        nblk = a.k / (kBlock32<TYPE> ? 32 : 256);
        row_bytes = nblk * BYTES;
        // L >= 4 for the K-quants (k >= 256), so a lane keeps the same sub-piece index c on every step
        c = kBlock32<TYPE> ? 0 : (int)(li & 3u);
        bstep = kBlock32<TYPE> ? L : L >> 2;  // blocks of a row one step covers
        blk0 = kBlock32<TYPE> ? li : li >> 2;
        w = wbase;
        lds_x = lx;
        lds_s = ls;
    }

    // The conversion masks must sit in VGPRs for v_and_or_b32 (one scalar operand
    // at most per VALU op on gfx9); the copy is opaque so they stay there.
    __device__ __forceinline__ void load_masks(const KArgs& a) {
        asm volatile("v_mov_b32 %0, %3\n\tv_mov_b32 %1, %4\n\tv_mov_b32 %2, %5"
                     : "=v"(m4), "=v"(m2), "=v"(magic)
                     : "s"(a.m4), "s"(a.m2), "s"(a.magic));
    }

    // Issues the fetch of task (rowbase, slot u, step s) into f, ordered after the
    // value `tie` names.
    __device__ __forceinline__ void fetch(Piece<TYPE>& f, uint32_t rowbase, int u, uint32_t s, float tie) {
        uint32_t r = rowbase + (uint32_t)u * rpw + lane_row;
        r = r < n ? r : n - 1u;
        uint32_t blk = blk0 + s * bstep;
        blk = blk < nblk ? blk : nblk - 1u;
        const uint8_t* ptr = w + (size_t)r * row_bytes + (size_t)blk * BYTES;
        asm volatile("" : "+v"(ptr) : "v"(tie));
        f.load(ptr, c);
    }

    __device__ __forceinline__ void prime(uint32_t rowbase) {
#pragma unroll
        for (int u = 0; u < D; ++u) fetch(buf[u], rowbase, u, 0, 0.f);
    }

    // All tasks of one wave group; stores its NR slots of results.  next_rowbase /
    // has_next: where the fetch ring continues after this group.
    __device__ __forceinline__ void group(uint32_t rowbase, uint32_t next_rowbase, bool has_next, float* yrow,
                                          bool valid) {
        float acc[NR];
#pragma unroll
        for (int u = 0; u < NR; ++u) acc[u] = 0.f;

        for (uint32_t s = 0; s < steps; ++s) {
            uint32_t xr[XW];
            float sx[4];
            const uint32_t pc = li + s * (1u << log_l);
            load_x_piece<TYPE, PAIR, XW>(lds_x, lds_s, pc < pieces ? pc : pieces + (uint32_t)c, c, xr, sx);
            const bool more = s + 1 < steps;  // uniform
#pragma unroll
            for (int u = 0; u < NR; ++u) {
                Piece<TYPE>& b = buf[u % D];
                if constexpr (PAIR)
                    acc[u] += dot_pair(b, c, xr, sx, m4, m2, magic);
                else
                    acc[u] += dot_f32(b, c, reinterpret_cast<const float*>(xr), sx);
                // refill with the task D ahead: same step while slots remain, else the
                // first slots of the next step, else of the next wave group.  The fetch is
                // tied to this task's result: otherwise the compiler hoists every refill
                // above the arithmetic into fresh registers, which doubles the buffers
                // and halves occupancy.
                if (u + D < NR || more || has_next)
                    fetch(b, u + D < NR || more ? rowbase : next_rowbase, u + D < NR ? u + D : u + D - NR,
                          u + D < NR ? s : more ? s + 1 : 0u, acc[u]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

#pragma unroll
        for (int u = 0; u < NR; ++u) {
            const float v = group_sum(acc[u], log_l);
            const uint32_t r = rowbase + (uint32_t)u * rpw + lane_row;
            if (li == 0 && r < n) yrow[r] = valid ? v : __builtin_nanf("");
        }
    }
};

// LDS layout of both kernels: activations | per-16 sums | queue counter (16 bytes).
//
// Small and medium problems, and every mul_mat_id launch: one workgroup of four
// waves per four wave groups, blockIdx.y = the (token, slot) pair.  The
// activations are requested first (vector loads return in order: behind a queue
// of weight fetches they would hold the workgroup at its barrier), then the
// first weight fetches go out so that their latency overlaps the staging.
// The zeros behind the activations and behind their sums (rows whose pieces the lanes per row do not divide).
template <bool PAIR>
__device__ __forceinline__ void stage_zero_pad(const KArgs& a, uint32_t* lds_x, float* lds_s, uint32_t tid, uint32_t threads) {
    if (!a.xpad) return;
    const uint32_t xw = PAIR ? a.k / 2 : a.k, pw = PAIR ? a.xpad / 2 : a.xpad;
    for (uint32_t i = tid; i < pw; i += threads) lds_x[xw + i] = 0u;
    for (uint32_t i = tid; i < a.xpad / 16u; i += threads) lds_s[a.k / 16u + i] = 0.f;
}

template <int TYPE, bool X_BF16, bool PAIR, int NR, int D>
__device__ __forceinline__ void gemv_body(const KArgs& a, uint32_t bx, uint32_t p) {
    extern __shared__ uint4 smem[];
    uint32_t* lds_x = reinterpret_cast<uint32_t*>(smem);
    float* lds_s = reinterpret_cast<float*>(lds_x + (PAIR ? (a.k + a.xpad) / 2 : a.k + a.xpad));

    const size_t xoff = (size_t)(p / a.top_k) * a.k * (X_BF16 ? 2 : 4);
    const uint8_t* xrow = static_cast<const uint8_t*>(a.x) + xoff;
    const uint32_t xchunks = a.k / 16;
    bool swiglu = false;
    if constexpr (!X_BF16) swiglu = a.x2 != nullptr;
    [[maybe_unused]] const uint8_t* urow = nullptr;
    XRaw<X_BF16> xraw;
    [[maybe_unused]] SwigluRaw sraw;
    if (!swiglu) {
        if (threadIdx.x < xchunks) xraw.fetch(xrow, threadIdx.x);
    } else if constexpr (!X_BF16) {
        urow = static_cast<const uint8_t*>(a.x2) + xoff;
        if (threadIdx.x < a.k / 4) sraw.fetch(xrow, urow, threadIdx.x);
    }

    const uint8_t* w = a.w;
    bool valid = true;
    if (a.ids) {
        const uint32_t e = a.ids[p];
        valid = e < a.n_experts;
        w += (size_t)(valid ? e : 0u) * a.expert_stride;
    } else if (a.route_logits) {
        // every wave works the token's routing out for itself (no barrier before the first weight fetch); one
        // wave of the launch per token also writes it down
        const uint32_t tok = p / a.top_k, slot = p % a.top_k, lane = threadIdx.x & 63u;
        uint32_t id;
        float wt;
        softmax_topk_lane<4>(a.route_logits + (size_t)tok * a.n_experts, a.n_experts, a.top_k, lane, id, wt);
        if (a.route_ids && bx == 0 && slot == 0 && threadIdx.x < a.top_k) {
            a.route_ids[(size_t)tok * a.top_k + lane] = id;
            a.route_w[(size_t)tok * a.top_k + lane] = wt;
        }
        w += (size_t)__shfl(id, slot) * a.expert_stride;
    }

    Walk<TYPE, X_BF16, PAIR, NR, D> wk;
    wk.init(a, w, lds_x, lds_s);
    const uint32_t rowbase = (bx * 4u + (threadIdx.x >> 6)) * wk.rpw * NR;
    wk.prime(rowbase);

    if (!swiglu) {
        if (threadIdx.x < xchunks) stage_store<X_BF16, PAIR>(xraw, threadIdx.x, lds_x, lds_s);
        for (uint32_t i = threadIdx.x + 256u; i < xchunks; i += 256u) {
            xraw.fetch(xrow, i);
            stage_store<X_BF16, PAIR>(xraw, i, lds_x, lds_s);
        }
    } else if constexpr (!X_BF16) {
        // k is a multiple of 16, so the four lanes of a quad enter and leave together
        if (threadIdx.x < a.k / 4) stage_swiglu(sraw, threadIdx.x, lds_x, lds_s);
        for (uint32_t i = threadIdx.x + 256u; i < a.k / 4; i += 256u) {
            sraw.fetch(xrow, urow, i);
            stage_swiglu(sraw, i, lds_x, lds_s);
        }
    }
    stage_zero_pad<PAIR>(a, lds_x, lds_s, threadIdx.x, 256u);
    wk.load_masks(a);
    __syncthreads();

    wk.group(rowbase, 0u, false, a.y + (size_t)p * a.n, valid);
}

template <int TYPE, bool X_BF16, bool PAIR, int NR, int D>
__global__ __launch_bounds__(256) void gemv_kernel(KArgs a) {
    gemv_body<TYPE, X_BF16, PAIR, NR, D>(a, blockIdx.x, blockIdx.y);
}

// Several independent GEMVs in one launch: blockIdx.z selects the job, the grid
// spans the largest job and the workgroups outside a smaller one leave at once.
constexpr uint32_t MAX_JOBS = 4;
struct KJobs {
    KArgs j[MAX_JOBS];
};

template <int TYPE, bool X_BF16, bool PAIR, int NR, int D>
__global__ __launch_bounds__(256) void gemv_jobs_kernel(KJobs js) {
    const KArgs& a = js.j[blockIdx.z];
    const uint32_t rows_per_wg = 4u * (64u >> a.log_l) * NR;
    if (blockIdx.y >= a.pairs || blockIdx.x * rows_per_wg >= a.n) return;
    gemv_body<TYPE, X_BF16, PAIR, NR, D>(a, blockIdx.x, blockIdx.y);
}

// Dense GEMV for matrices with many wave groups per CU: one workgroup of WAVES
// waves per CU (the launch asks for more than half of the CU's LDS, so two never
// share a CU), each CU owning an equal share of the wave groups.
// Inside the CU the waves take wave groups from a counter in LDS instead of a
// fixed split: the SIMD's issue arbitration favours its oldest wave, so with a
// fixed split the youngest wave of every SIMD finishes long after the others and
// the CU idles meanwhile.  A wave knows its next wave group one group ahead, so
// the fetch ring runs across group boundaries.
template <int TYPE, bool X_BF16, bool PAIR, int NR, int D, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemv_queue_kernel(KArgs a) {
    constexpr uint32_t THREADS = 64 * WAVES;
    extern __shared__ uint4 smem[];
    uint32_t* lds_x = reinterpret_cast<uint32_t*>(smem);
    float* lds_s = reinterpret_cast<float*>(lds_x + (PAIR ? (a.k + a.xpad) / 2 : a.k + a.xpad));
    uint32_t* lds_q = reinterpret_cast<uint32_t*>(lds_s + (a.k + a.xpad) / 16);

    const uint8_t* xrow = static_cast<const uint8_t*>(a.x);
    const uint32_t xchunks = a.k / 16;
    XRaw<X_BF16> xraw;
    if (threadIdx.x < xchunks) xraw.fetch(xrow, threadIdx.x);

    Walk<TYPE, X_BF16, PAIR, NR, D> wk;
    wk.init(a, a.w, lds_x, lds_s);

    // this CU's share of the wave groups: blockIdx.x, blockIdx.x + gridDim.x, ... (its i-th group is group_of(i)).
    // All CUs so walk the matrix front to back together and the fetches in flight at any moment cover one
    // dense window of it; with a contiguous share per CU they would come from gridDim.x distant places
    // (measured 3 % slower).
    const uint32_t count = (a.groups + gridDim.x - 1u - blockIdx.x) / gridDim.x;
    const uint32_t rows_per_group = wk.rpw * NR;
    auto group_of = [&](uint32_t i) -> uint32_t { return i * gridDim.x + blockIdx.x; };

    // the first WAVES wave groups are claimed by wave index, the rest from the counter
    uint32_t cur = threadIdx.x >> 6;
    if (cur < count) wk.prime(group_of(cur) * rows_per_group);

    if (threadIdx.x == 0) *lds_q = WAVES;
    if (threadIdx.x < xchunks) stage_store<X_BF16, PAIR>(xraw, threadIdx.x, lds_x, lds_s);
    for (uint32_t i = threadIdx.x + THREADS; i < xchunks; i += THREADS) {
        xraw.fetch(xrow, i);
        stage_store<X_BF16, PAIR>(xraw, i, lds_x, lds_s);
    }
    stage_zero_pad<PAIR>(a, lds_x, lds_s, threadIdx.x, THREADS);
    wk.load_masks(a);
    __syncthreads();

    auto grab = [&]() -> uint32_t {
        uint32_t v = 0;
        if (wk.lane == 0) v = __hip_atomic_fetch_add(lds_q, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return v;
    };
    uint32_t nxt = __builtin_amdgcn_readfirstlane(grab());
    while (cur < count) {
        const uint32_t after = grab();  // claimed now, read when this group is done
        wk.group(group_of(cur) * rows_per_group, group_of(nxt) * rows_per_group, nxt < count, a.y, true);
        cur = nxt;
        nxt = __builtin_amdgcn_readfirstlane(after);
    }
}


// Dense single-row GEMV over K-quants with bf16 activations and k % 4096 == 0 (64 lanes per row step): one
// workgroup of W waves per CU.  Requests that join an HBM queue already holding the whole matrix wait microseconds
// (a 28 MB matrix asked for at once: the activations of late waves arrive after 2-3 us, and nothing can be
// computed before), so this form keeps little in flight: the workgroup stages the activations first, then every
// wave walks its rows with ONE fetch outstanding (16 waves x 2.3 KB per CU is what 8 TB/s x 1 us needs); the
// other waves of the SIMD compute meanwhile.  Row of (iteration i, wave wv, workgroup b) = (i*W + wv)*G + b, so all
// CUs walk the matrix front to back together.  Rows >= n0 belong to a second matrix of the same shape (the gate /
// up pair of a decode step in one launch).  Per-row arithmetic (order of the partial sums, per-16 activation sums)
// is that of gemv_kernel: the results are bit-identical.
struct SArgs {
    const void* x;
    const uint8_t* w0;
    const uint8_t* w1;
    float* y0;
    float* y1;
    uint32_t n0, n, k;
    uint32_t m4, m2, magic;
};

// LDS slot of 16-byte chunk ch (8 activations as 4 paired words): lanes that read together differ in the piece
// index (Q4_K / Q5_K: ch / 8) or in bits 1, 4, 5.. of ch (Q6_K: run half, block half, block), which the swizzle
// spreads over the sixteen 16-byte bank groups.
template <int TYPE>
__device__ __forceinline__ uint32_t stream_swz(uint32_t ch) {
    if constexpr (TYPE == HQ_Q6_K) return ch ^ (((ch >> 4) & 1u) | (((ch >> 5) & 3u) << 2));
    return ch ^ ((ch >> 4) & 7u);
}

template <int TYPE>
__device__ __forceinline__ void stream_load_x(const uint4* lds_x, const float* lds_s, uint32_t st, uint32_t lane, int c,
                                              uint32_t* xp, float* sx) {
    if constexpr (TYPE == HQ_Q6_K) {
        const uint32_t ch0 = st * 512u + (lane >> 2) * 32u + (uint32_t)(c >> 1) * 16u + (uint32_t)(c & 1) * 2u;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const uint4 v = lds_x[stream_swz<TYPE>(ch0 + 4 * r + u)];
                xp[8 * r + 4 * u] = v.x;
                xp[8 * r + 4 * u + 1] = v.y;
                xp[8 * r + 4 * u + 2] = v.z;
                xp[8 * r + 4 * u + 3] = v.w;
            }
            sx[r] = lds_s[(ch0 + 4 * r) / 2];
        }
    } else {
        const uint32_t ch0 = (st * 64u + lane) * 8u;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint4 v = lds_x[stream_swz<TYPE>(ch0 + j)];
            xp[4 * j] = v.x;
            xp[4 * j + 1] = v.y;
            xp[4 * j + 2] = v.z;
            xp[4 * j + 3] = v.w;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) sx[r] = lds_s[ch0 / 2 + r];
    }
}

// ROWS bf16 activation rows of k values into LDS as paired words (16 per thread and pass) with their per-16 sums.
template <int TYPE, int ROWS>
__device__ __forceinline__ void stream_stage_x(const void* x, uint32_t k, uint4* lds_x, float* lds_s, uint32_t tid, uint32_t nt) {
    for (uint32_t ii = tid; ii < ROWS * (k / 16u); ii += nt) {
        const uint32_t xr = ROWS == 1 ? 0u : ii / (k / 16u), i = ROWS == 1 ? ii : ii % (k / 16u);
        XRaw<true> raw;
        raw.fetch(static_cast<const uint8_t*>(x) + (size_t)xr * k * 2u, i);
        const uint4 p = raw.r[0], q = raw.r[1];
        const uint32_t w[8] = {p.x, p.y, p.z, p.w, q.x, q.y, q.z, q.w};
        uint4 o0, o1;
        o0.x = (w[0] & 0xffffu) | (w[1] << 16);
        o0.y = (w[0] >> 16) | (w[1] & 0xffff0000u);
        o0.z = (w[2] & 0xffffu) | (w[3] << 16);
        o0.w = (w[2] >> 16) | (w[3] & 0xffff0000u);
        o1.x = (w[4] & 0xffffu) | (w[5] << 16);
        o1.y = (w[4] >> 16) | (w[5] & 0xffff0000u);
        o1.z = (w[6] & 0xffffu) | (w[7] << 16);
        o1.w = (w[6] >> 16) | (w[7] & 0xffff0000u);
        lds_x[xr * (k / 8u) + stream_swz<TYPE>(2 * i)] = o0;
        lds_x[xr * (k / 8u) + stream_swz<TYPE>(2 * i + 1)] = o1;
        float sum = 0.f;  // the same order of additions as stage_store
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            sum += bf16_bits_to_f32(w[j] & 0xffffu);
            sum += bf16_bits_to_f32(w[j] >> 16);
        }
        lds_s[xr * (k / 16u) + i] = sum;
    }
}

// ROWS = 2 .. 4: that many activation rows (x[r] -> y[r] of one matrix) share every weight fetch and the
// nibble-to-bf16 work; the dot products and sums are per row, in the order of the one-row form.  Three and four rows
// read their activations from LDS per piece (in registers they would be 32 each per row).
// COPY (Q4_K / Q5_K, whose blocks are whole 16-byte pieces and whose steps of sixteen blocks are whole 128-byte lines:
// 2304 / 2816 bytes): a step is not fetched by the lanes that use it, three to five instructions touching each line,
// but copied -- consecutive lanes consecutive 16-byte pieces, non-temporal loads, every line asked for once -- into 3 KB
// of LDS the wave owns and read back from there as the same pieces; the next step's copy is in flight meanwhile.
// X_BF16 = false (one row, COPY): f32 activations, the dtype of the reference's call sites, staged and multiplied as in
// the flat walk (a lane's 64 activations as f32, exact products; the same bits as that walk gives for these rows).
template <int TYPE, int W, bool XREG, int ROWS = 1, bool COPY = false, bool X_BF16 = true>
__global__ __launch_bounds__(64 * W) void gemv_stream_kernel(SArgs a) {
    static_assert(!COPY || TYPE == HQ_Q4_K || TYPE == HQ_Q5_K, "blocks of whole 16-byte pieces");
    static_assert(X_BF16 || (ROWS == 1 && COPY), "f32 activations: the one-row copy form");
    constexpr uint32_t NT = 64 * W, BB = kBlockBytes<TYPE>;
    constexpr uint32_t PIECES = 16u * BB / 16u, NPV = (PIECES + 63u) / 64u;  // 16-byte pieces of a step; per lane
    using XF = FlatX1<TYPE, false>;
    extern __shared__ uint4 smem[];
    uint4* lds_x = smem;  // bf16: [ROWS][k / 8] paired words; f32: XF's layout
    float* lds_s = X_BF16 ? reinterpret_cast<float*>(lds_x + ROWS * (a.k / 8))  // [ROWS][k / 16]
                          : reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(smem) + XF::value_bytes(a.k));
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));  // the same in a wave: scalar loop control
    const int c = (int)(lane & 3u);
    const uint32_t S = a.k / 4096u, rowb = a.k / 256u * BB;
    const uint32_t stride = W * gridDim.x;
    const uint32_t row_first = wv * gridDim.x + blockIdx.x;
    const uint32_t rows_mine = row_first < a.n ? (a.n - row_first + stride - 1u) / stride : 0u;
    const uint32_t ntask = rows_mine * S;

    // the activations first, nothing else of this workgroup in front of them
    if constexpr (X_BF16) stream_stage_x<TYPE, ROWS>(a.x, a.k, lds_x, lds_s, tid, NT);
    else XF::stage(a.x, a.k, lds_x, lds_s, tid, NT);

    // One piece per lane in flight, refilled after every use (past the wave's last task: the last task again, not
    // used).  Results are not stored row by row from lane 0 but kept, lane i the wave's row i, and stored 64 rows at a
    // time: no store among the fetches, and the loop has one path.  (Two and three pieces in flight were measured,
    // with every wait of the loop allowing for the younger fetches: 103 against 94 us on the 151936 x 4096 Q6_K matrix.)
    Piece<TYPE> pc;
    [[maybe_unused]] uint4 pv[COPY ? NPV : 1];
    // (COPY: the wave's step buffer, 64 * NPV slots of 16 bytes, behind the activations and their sums)
    [[maybe_unused]] uint4* wbuf = reinterpret_cast<uint4*>(lds_s + ROWS * (a.k / 16)) + wv * (64u * NPV);
    uint32_t f_row = row_first, f_st = 0, f_left = ntask;  // the next task to fetch; tasks not yet fetched
    auto fetch_next = [&](Piece<TYPE>& p) {
        const uint8_t* base = f_row < a.n0 ? a.w0 + (size_t)f_row * rowb : a.w1 + (size_t)(f_row - a.n0) * rowb;
        if constexpr (COPY) {
#pragma unroll
            for (uint32_t i = 0; i < NPV; ++i) {
                const uint32_t pi = lane + 64u * i;
                pv[i] = ldnt16(base + (size_t)f_st * (16u * BB) + 16u * (pi < PIECES ? pi : PIECES - 1u));
            }
        } else {
            p.load(base + (f_st * 16u + (lane >> 2)) * BB, c);
        }
        if (f_left > 1u) {  // (scalar: no memory operation inside)
            --f_left;
            if (++f_st == S) {
                f_st = 0;
                f_row += stride;
            }
        }
    };
    if (ntask) fetch_next(pc);
    __syncthreads();

    [[maybe_unused]] uint32_t m4, m2, magic;
    if constexpr (X_BF16)
        asm volatile("v_mov_b32 %0, %3\n\tv_mov_b32 %1, %4\n\tv_mov_b32 %2, %5"
                     : "=v"(m4), "=v"(m2), "=v"(magic)
                     : "s"(a.m4), "s"(a.m2), "s"(a.magic));
    uint32_t xp[ROWS][X_BF16 ? 32 : 64];
    float sx[ROWS][4];
    auto load_x = [&](int r, uint32_t step) {
        if constexpr (X_BF16) stream_load_x<TYPE>(lds_x + r * (a.k / 8u), lds_s + r * (a.k / 16u), step, lane, c, xp[r], sx[r]);
        else XF::load(lds_x, lds_s, step * 16u + (lane >> 2), c, xp[r], sx[r]);
    };
    if constexpr (XREG) {  // k == 4096: one piece per lane for every row
#pragma unroll
        for (int r = 0; r < ROWS; ++r) load_x(r, 0);
    }

    uint32_t st = 0, done = 0;  // step inside the row; rows finished
    float acc[ROWS], keep[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] = 0.f, keep[r] = 0.f;
    auto flush = [&](uint32_t first, uint32_t count) {  // rows first .. first + count - 1 of this wave, from lanes 0 .. count - 1
        if (lane < count) {
            const uint32_t row = row_first + (first + lane) * stride;
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                if (row < a.n0) a.y0[(size_t)r * a.n + row] = keep[r];  // (ROWS == 2: one matrix, n0 == n)
                else a.y1[row - a.n0] = keep[r];
            }
        }
    };
    auto task = [&](Piece<TYPE>& p) {
        if constexpr (COPY) {
            // the copied step goes to LDS (behind the wave's reads of the previous one: a wave's LDS operations are served
            // in order), the next step's copy is issued, this step's pieces are read back
#pragma unroll
            for (uint32_t i = 0; i < NPV; ++i) wbuf[lane + 64u * i] = pv[i];
            asm volatile("" ::: "memory");
            fetch_next(p);
            const uint4* blk = wbuf + (lane >> 2) * (BB / 16u);
            p.hdr = blk[0];
            if constexpr (TYPE == HQ_Q5_K) {
                p.h0 = blk[1];
                p.h1 = blk[2];
                p.q0 = blk[3 + 2 * c];
                p.q1 = blk[4 + 2 * c];
            } else {
                p.q0 = blk[1 + 2 * c];
                p.q1 = blk[2 + 2 * c];
            }
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            if constexpr (!XREG) load_x(r, st);
            if constexpr (X_BF16) acc[r] += dot_pair(p, c, xp[r], sx[r], m4, m2, magic);
            else acc[r] += dot_f32(p, c, reinterpret_cast<const float*>(xp[r]), sx[r]);
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) asm volatile("" : "+v"(acc[r]));  // the refill follows the arithmetic that frees its registers
        if constexpr (!COPY) fetch_next(p);
        if (++st == S) {
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const float v = group_sum(acc[r], 6);
                keep[r] = lane == (done & 63u) ? v : keep[r];
                acc[r] = 0.f;
            }
            st = 0;
            if ((++done & 63u) == 0u) flush(done - 64u, 64u);
        }
    };
    for (uint32_t t = 0; t < ntask; ++t) task(pc);
    if (done & 63u) flush(done & ~63u, done & 63u);
}


// Q6_K rows of k = 4096 or 2048 elements (3360 / 1680 bytes, multiples of 16): the streaming kernel above with the weights
// fetched differently.  A lane fetching its own piece touches a row's 128-byte lines with five instructions; here a wave
// copies a chunk of sixteen blocks (one row of 4096, two of 2048) as 210 consecutive 16-byte pieces (four non-temporal
// loads per lane: each line is asked for once and not kept in the caches) into 4 KB of LDS it owns, and its lanes read
// their pieces back from there.  A wave takes groups of FOUR consecutive chunks, 13440 bytes = 105 whole lines, so that
// no line is shared with another wave (a non-temporal line fetched by two waves crosses the memory system twice).  Read
// alone this way the 510 MB matrix takes 75 us, with the lanes fetching their own pieces 82-84.  The blocks lie in LDS
// as in memory, 210 bytes apart, so a lane's fields start at even addresses: each is read as aligned words and shifted
// into place by v_alignbyte.  With bf16 activations the pieces, the dot products and the order of the sums are those of
// gemv_stream_kernel; with f32 activations (the dtype of the reference's call sites) those of the flat walk, a lane's 64
// activations in registers: the same bits as those kernels give for rows of 4096.
template <bool X_BF16>
constexpr int kQ6kCopyWaves = X_BF16 ? 16 : 12;  // (f32: 64 activation registers per lane)
template <bool X_BF16, int LOG_RPC>
__global__ __launch_bounds__(64 * kQ6kCopyWaves<X_BF16>) void gemv_q6k_rowcopy_kernel(SArgs a) {
    constexpr uint32_t W = kQ6kCopyWaves<X_BF16>, NT = 64 * W, CHUNKB = 16u * Q6K_BYTES, PIECES = CHUNKB / 16u;  // 3360 bytes, 210 pieces
    constexpr uint32_t RPC = 1u << LOG_RPC;  // rows per chunk: k = 4096 >> LOG_RPC
    using XF = FlatX1<HQ_Q6_K, false>;
    extern __shared__ uint4 smem[];
    __shared__ uint32_t lds_queue;
    uint4* lds_x = smem;
    float* lds_s = X_BF16 ? reinterpret_cast<float*>(lds_x + a.k / 8u) : reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(smem) + XF::value_bytes(a.k));
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    uint4* wbuf = reinterpret_cast<uint4*>(lds_s + a.k / 16u) + wv * 256u;  // this wave's chunk: 256 slots of 16 bytes
    const int c = (int)(lane & 3u);
    const uint32_t chunks = (a.n + RPC - 1u) >> LOG_RPC, groups = (chunks + 3u) / 4u;
    const uint32_t tail_pieces = (a.n - ((chunks - 1u) << LOG_RPC)) * (PIECES >> LOG_RPC);  // pieces of the last chunk that exist
    // The workgroup's groups are blockIdx.x + q gridDim.x, q < count; its waves take q from a counter in LDS (the first
    // claims are the wave indices), one ahead of the group they work on: the SIMD favours its oldest wave, and with
    // fixed shares the youngest would finish long after the others (head: 83.2 -> 82.1 us, f32 83.3 -> 81.6).
    const uint32_t count = blockIdx.x < groups ? (groups - blockIdx.x + gridDim.x - 1u) / gridDim.x : 0u;
    if (tid == 0) lds_queue = W;

    if constexpr (X_BF16) stream_stage_x<HQ_Q6_K, 1>(a.x, a.k, lds_x, lds_s, tid, NT);
    else XF::stage(a.x, a.k, lds_x, lds_s, tid, NT);

    // chunk r of group q, clamped to the matrix (a clamped chunk is not stored)
    uint4 pv[4];
    auto fetch = [&](uint32_t q, uint32_t r) {
        uint32_t ch = 4u * (blockIdx.x + q * gridDim.x) + r;
        ch = ch < chunks ? ch : chunks - 1u;
        const uint8_t* base = a.w0 + (size_t)ch * CHUNKB;
        const uint32_t last = (ch == chunks - 1u ? tail_pieces : PIECES) - 1u;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t pc = lane + 64u * (uint32_t)i;
            pv[i] = ldnt16(base + 16u * (pc < last ? pc : last));
        }
    };
    uint32_t q_cur = wv;
    if (q_cur < count) fetch(q_cur, 0);
    __syncthreads();

    [[maybe_unused]] uint32_t m4, m2, magic;
    if constexpr (X_BF16)
        asm volatile("v_mov_b32 %0, %3\n\tv_mov_b32 %1, %4\n\tv_mov_b32 %2, %5" : "=v"(m4), "=v"(m2), "=v"(magic) : "s"(a.m4), "s"(a.m2), "s"(a.magic));
    // the lane's activations: block (lane / 4) of its row, quarter c
    const uint32_t lane_in_row = lane & (63u >> LOG_RPC);
    uint32_t xp[X_BF16 ? 32 : 64];
    float sx[4];
    if constexpr (X_BF16) stream_load_x<HQ_Q6_K>(lds_x, lds_s, 0, lane_in_row, c, xp, sx);
    else XF::load(lds_x, lds_s, lane_in_row >> 2, c, xp, sx);

    // this lane's piece in the chunk buffer: block lane / 4 at byte 210 (lane / 4), fields at even offsets; sh = the bytes by
    // which a field's first aligned word starts early (0 or 2)
    const uint32_t blk = (lane >> 2) * Q6K_BYTES, h = (uint32_t)c >> 1, lr = (uint32_t)c & 1u;
    const uint32_t* wb32 = reinterpret_cast<const uint32_t*>(wbuf);
    const uint32_t o_qa = blk + 64u * h + 16u * lr, o_qb = o_qa + 32u, o_qh = blk + 128u + 32u * h + 16u * lr, o_sc = blk + 192u + 8u * h,
                   o_d = blk + 206u;
    auto field16 = [&](uint32_t o) -> uint4 {
        const uint32_t* p = wb32 + (o >> 2);
        const uint32_t sh = o & 3u, w0 = p[0], w1 = p[1], w2 = p[2], w3 = p[3], w4 = p[4];
        return make_uint4(__builtin_amdgcn_alignbyte(w1, w0, sh), __builtin_amdgcn_alignbyte(w2, w1, sh), __builtin_amdgcn_alignbyte(w3, w2, sh),
                          __builtin_amdgcn_alignbyte(w4, w3, sh));
    };

    // results: lane i keeps the wave's i-th finished row and its index, stored 64 at a time
    uint32_t done = 0, keep_row = 0;
    float keep = 0.f;
    auto flush = [&](uint32_t cnt) {
        if (lane < cnt && keep_row < a.n) a.y0[keep_row] = keep;
    };
    while (q_cur < count) {
        uint32_t claimed = 0, q_nxt = 0;
        if (lane == 0) claimed = __hip_atomic_fetch_add(&lds_queue, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma unroll
        for (uint32_t r = 0; r < 4u; ++r) {
            // the chunk fetched a task ago goes to LDS (the wave's earlier reads of the buffer precede these writes: one
            // wave's LDS operations are served in order), the next chunk's fetch is issued, then this chunk's pieces are read back
#pragma unroll
            for (int i = 0; i < 4; ++i) wbuf[lane + 64u * (uint32_t)i] = pv[i];
            asm volatile("" ::: "memory");  // (for the compiler: the reads below are of what was just written)
            if (r < 3u) {
                fetch(q_cur, r + 1u);
            } else {
                q_nxt = (uint32_t)__builtin_amdgcn_readfirstlane((int)claimed);
                if (q_nxt < count) fetch(q_nxt, 0);
            }
            Piece<HQ_Q6_K> pc;
            pc.qa = field16(o_qa);
            pc.qb = field16(o_qb);
            pc.qh = field16(o_qh);
            {
                const uint32_t* p = wb32 + (o_sc >> 2);
                const uint32_t sh = o_sc & 3u, w0 = p[0], w1 = p[1], w2 = p[2];
                pc.sc = make_uint2(__builtin_amdgcn_alignbyte(w1, w0, sh), __builtin_amdgcn_alignbyte(w2, w1, sh));
                const uint32_t* q = wb32 + (o_d >> 2);
                pc.d = __builtin_amdgcn_alignbyte(q[1], q[0], o_d & 3u);
            }
            float part;
            if constexpr (X_BF16) part = dot_pair(pc, c, xp, sx, m4, m2, magic);
            else part = dot_f32(pc, c, reinterpret_cast<const float*>(xp), sx);
            const float v = group_sum(part, 6 - LOG_RPC);
            const uint32_t row0 = (4u * (blockIdx.x + q_cur * gridDim.x) + r) << LOG_RPC;  // (past the matrix: not stored)
            if constexpr (RPC == 1) {
                const bool mine = lane == (done & 63u);
                keep = mine ? v : keep;
                keep_row = mine ? row0 : keep_row;
            } else {
                // (every lane of a half holds its row's sum: lanes 0 and 32 speak for the two rows)
                const float v0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
                const float v1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
                const bool m0 = lane == (done & 63u), m1 = lane == (done & 63u) + 1u;
                keep = m0 ? v0 : m1 ? v1 : keep;
                keep_row = m0 ? row0 : m1 ? row0 + 1u : keep_row;
            }
            done += RPC;
            if ((done & 63u) == 0u) flush(64u);
        }
        q_cur = q_nxt;
    }
    if (done & 63u) flush(done & 63u);
}
template <bool X_BF16>
int launch_q6k_rowcopy(hipStream_t s, const SArgs& sa, uint32_t cus) {
    constexpr int W = kQ6kCopyWaves<X_BF16>;
    const size_t lds_x = X_BF16 ? (size_t)sa.k * 2 + (size_t)(sa.k / 16) * 4 : FlatX1<HQ_Q6_K, false>::lds_bytes(sa.k);
    const size_t lds = lds_x + (size_t)W * 4096u;
    auto kern = sa.k == 4096 ? gemv_q6k_rowcopy_kernel<X_BF16, 0> : gemv_q6k_rowcopy_kernel<X_BF16, 1>;
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, "hipFuncSetAttribute(gemv row-copy LDS)")) return rc;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(64 * W), lds, s, sa);
    return check_launch("gemv row-copy kernel launch");
}
// One Q6_K matrix, 16-byte aligned, rows of 4096 or 2048 elements, two groups of four chunks per wave or more.
inline bool q6k_rowcopy_takes(const void* w, uint32_t n, uint32_t k, uint32_t cus) {
    return (k == 4096 || k == 2048) && (reinterpret_cast<uintptr_t>(w) & 15u) == 0 && (uint64_t)n * (k / 256u) >= (uint64_t)512u * cus;
}

// K-quant rows of nine super-blocks or more that are not whole windows of sixteen (k = 2560, 2816, 3072, 3584, 3840, 5120,
// 7168, 14336 ...), and rows of Q8_0 / Q4_0 block pairs (a lane each, 64 to a window) likewise.  The matrix is cut into the flat walk's windows of sixteen blocks; the pattern of row boundaries inside
// a window repeats every P = bu / gcd(bu, 16) windows = R = 16 / gcd(bu, 16) rows (k = 2816: 11 windows, 16 rows; k = 5120: 5
// windows, 4 rows).  Wave j of a sequence of P waves takes window j of every period the sequence owns: which super-block
// of a row a lane's quarter belongs to never changes, so its activations sit in registers (the flat walk reads them from
// LDS for every window), the rows a window touches are the same lane ranges every time, and the window is copied through
// LDS as in the kernels above (Q4_K / Q5_K: 18 / 22 whole lines; Q6_K: 26.25 lines, a line at a window's edge is asked for
// by two waves of the workgroup).  A window's per-row sums (one masked wave reduction per row it touches, three at most)
// go to slots in LDS, one per window a row lies in; after a barrier the workgroup adds a row's slots in the flat walk's
// order and stores the rows: the same bits as the flat walk gives with full windows.  Measured against the flat walk
// (bf16 / f32 activations): Q6_K 262144 x 2816 113 -> 100 / 118 -> 110 us, 152064 x 5120 112.6 -> 100.6 / 118.8 -> 108.9,
// 152064 x 3584 82.7 -> 75.3 / 85.7 -> 79.9, 32768 x 14336 71.4 -> 62.6 / 74.1 -> 67.4; Q4_K 262144 x 2816 85.5 -> 77.8 /
// 92.4 -> 82.2, 152064 x 5120 82.1 -> 74.0 / 89.0 -> 79.1; Q5_K 262144 x 2816 101.1 -> 90.8 / 107.5 -> 95.0, 262144 x 3840
// 129.2 -> 114.6 / 142.3 -> 121.9; Q4_0 262144 x 2816 81.2 -> 70.9 / 88.4 -> 78.6, Q8_0 120.2 -> 115.5 / 119.9 -> 115.6; with fewer
// than a dozen windows per wave the fixed shares leave waves idle at the end
// and the flat walk is as fast or faster.
struct PArgs {
    const void* x;
    const uint8_t* w;
    float* y;
    uint32_t n, k, bu;
    uint32_t period_windows, log_period_rows;  // P, log2 R
    uint32_t seqs;                             // the workgroup's waves are seqs * P: sequence s takes every seqs-th period of the workgroup
    uint32_t row_slots;                        // windows a row can lie in
    uint32_t periods_per_round;                // slots in LDS: periods_per_round * R * row_slots floats
    uint32_t m4, m2, magic;
};
// Waves per workgroup at most (with f32 activations, 64 registers of them per lane, the kernels take 110 .. 128 registers).
template <int TYPE, bool X_BF16>
constexpr uint32_t kPeriodMaxWaves = 16u;
template <int TYPE, bool X_BF16>
__global__ __launch_bounds__((64 * kPeriodMaxWaves<TYPE, X_BF16>)) void gemv_period_kernel(PArgs a) {
    static_assert(TYPE == HQ_Q4_K || TYPE == HQ_Q5_K || TYPE == HQ_Q6_K || TYPE == HQ_Q8_0_X2 || TYPE == kX2 + HQ_Q4_0,
                  "super-blocks of 256 weights, four lanes each, or pairs of 32-weight blocks, one lane each");
    // a window: 64 lanes = UW units of BB bytes; 2304 / 2816 / 3360 bytes (144 / 176 / 210 pieces), block pairs 4352 / 2304 (272 / 144)
    constexpr uint32_t LPU = kLanesPerUnit<TYPE>, UW = kUnitsPerWindow<TYPE>, BB = kBlockBytes<TYPE>, CHUNKB = UW * BB, PIECES = CHUNKB / 16u;
    constexpr int NPV = (int)((PIECES + 63u) / 64u);
    using X = FlatX<TYPE, X_BF16>;
    extern __shared__ uint4 smem[];
    uint4* lds_x = smem;
    float* lds_s = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(smem) + X::value_bytes(a.k));
    const uint32_t tid = threadIdx.x, lane = tid & 63u, nthreads = blockDim.x;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    uint4* wbuf = reinterpret_cast<uint4*>(lds_s + a.k / 16u) + wv * (64u * NPV);
    float* slots = reinterpret_cast<float*>(reinterpret_cast<uint4*>(lds_s + a.k / 16u) + (nthreads >> 6) * (64u * NPV));
    const int c = (int)(lane & 3u);
    const uint32_t P = a.period_windows, LR = a.log_period_rows, R = 1u << LR;
    const uint32_t j = wv % P, sq = wv / P;  // window of the period, sequence
    const uint32_t periods = a.n >> LR;
    const uint32_t cnt_wg = blockIdx.x < periods ? (periods - blockIdx.x + gridDim.x - 1u) / gridDim.x : 0u;

    X::stage(a.x, a.k, lds_x, lds_s, tid, nthreads);

    // period i of the workgroup's, window j (non-temporal loads throughout: fetching the pieces on the two lines a window
    // shares with its neighbours with ordinary loads measured the same, ordinary loads for all of it 4 % slower)
    uint4 pv[NPV];
    auto fetch = [&](uint32_t i) {
        const uint8_t* base = a.w + ((size_t)(blockIdx.x + i * gridDim.x) * P + j) * CHUNKB;
#pragma unroll
        for (int q = 0; q < NPV; ++q) {
            const uint32_t pc = lane + 64u * (uint32_t)q;
            pv[q] = ldnt16(base + 16u * (pc < PIECES - 1u ? pc : PIECES - 1u));
        }
    };
    uint32_t i_cur = sq;
    if (i_cur < cnt_wg) fetch(i_cur);
    __syncthreads();

    [[maybe_unused]] uint32_t m4, m2, magic;
    if constexpr (X::PAIR)
        asm volatile("v_mov_b32 %0, %3\n\tv_mov_b32 %1, %4\n\tv_mov_b32 %2, %5" : "=v"(m4), "=v"(m2), "=v"(magic) : "s"(a.m4), "s"(a.m2), "s"(a.magic));
    // the lane's unit of the period, its row there and its unit of that row
    const uint32_t bi = UW * j + lane / LPU, rl = bi / a.bu, ur = bi - rl * a.bu;
    const uint32_t r_lo = (UW * j) / a.bu, nseg = (UW * j + UW - 1u) / a.bu - r_lo + 1u;  // rows the window touches: r_lo .. r_lo + nseg - 1
    const uint32_t seg = rl - r_lo;
    uint32_t xr[X::XW];
    float sx[kIsX2<TYPE> ? 8 : 4] = {};
    X::load(lds_x, lds_s, ur, c, xr, sx);
    // lane s < nseg stores the sum of row r_lo + s: slot 0 if this is the row's first window, 1 if its second ...
    const uint32_t my_row = r_lo + (lane < nseg ? lane : 0u), MW = a.row_slots;
    const uint32_t my_slot = MW * my_row + (j - (my_row * a.bu) / UW);

    // Q6_K: block lane / 4 at byte 210 (lane / 4), fields at even offsets, read as aligned words and shifted into place
    [[maybe_unused]] const uint32_t blk = (lane >> 2) * BB, h = (uint32_t)c >> 1, lr = (uint32_t)c & 1u;
    [[maybe_unused]] const uint32_t* wb32 = reinterpret_cast<const uint32_t*>(wbuf);
    [[maybe_unused]] const uint32_t o_qa = blk + 64u * h + 16u * lr, o_qb = o_qa + 32u, o_qh = blk + 128u + 32u * h + 16u * lr,
                                    o_sc = blk + 192u + 8u * h, o_d = blk + 206u;
    [[maybe_unused]] auto field16 = [&](uint32_t o) -> uint4 {
        const uint32_t* p = wb32 + (o >> 2);
        const uint32_t sh = o & 3u, w0 = p[0], w1 = p[1], w2 = p[2], w3 = p[3], w4 = p[4];
        return make_uint4(__builtin_amdgcn_alignbyte(w1, w0, sh), __builtin_amdgcn_alignbyte(w2, w1, sh), __builtin_amdgcn_alignbyte(w3, w2, sh),
                          __builtin_amdgcn_alignbyte(w4, w3, sh));
    };

    for (uint32_t i0 = 0; i0 < cnt_wg; i0 += a.periods_per_round) {
        const uint32_t i1 = i0 + a.periods_per_round < cnt_wg ? i0 + a.periods_per_round : cnt_wg;
        while (i_cur < i1) {
#pragma unroll
            for (int q = 0; q < NPV; ++q) wbuf[lane + 64u * (uint32_t)q] = pv[q];
            asm volatile("" ::: "memory");
            if (i_cur + a.seqs < cnt_wg) fetch(i_cur + a.seqs);
            Piece<TYPE> pc;
            if constexpr (TYPE == kX2 + HQ_Q4_0) {  // [d0][16 bytes][d1][16 bytes] as nine words at a multiple of four bytes
                const uint32_t* q = wb32 + lane * (BB / 4u);
                const uint32_t w0 = q[0], w1 = q[1], w2 = q[2], w3 = q[3], w4 = q[4];
                pc.a.d = w0 & 0xffffu;
                pc.a.q = make_uint4(__builtin_amdgcn_alignbyte(w1, w0, 2), __builtin_amdgcn_alignbyte(w2, w1, 2), __builtin_amdgcn_alignbyte(w3, w2, 2),
                                    __builtin_amdgcn_alignbyte(w4, w3, 2));
                pc.b.d = w4 >> 16;
                pc.b.q = make_uint4(q[5], q[6], q[7], q[8]);
            } else if constexpr (TYPE == HQ_Q8_0_X2) {  // a block pair: seventeen words at a multiple of four bytes
                const uint32_t* q = wb32 + lane * (BB / 4u);
                pc.a = make_uint4(q[0], q[1], q[2], q[3]);
                pc.b = make_uint4(q[4], q[5], q[6], q[7]);
                pc.c = make_uint4(q[8], q[9], q[10], q[11]);
                pc.e = make_uint4(q[12], q[13], q[14], q[15]);
                pc.t = q[16];
            } else if constexpr (TYPE != HQ_Q6_K) {  // blocks of whole 16-byte pieces
                const uint4* b16 = wbuf + (lane >> 2) * (BB / 16u);
                pc.hdr = b16[0];
                if constexpr (TYPE == HQ_Q5_K) {
                    pc.h0 = b16[1];
                    pc.h1 = b16[2];
                    pc.q0 = b16[3 + 2 * c];
                    pc.q1 = b16[4 + 2 * c];
                } else {
                    pc.q0 = b16[1 + 2 * c];
                    pc.q1 = b16[2 + 2 * c];
                }
            } else {
                pc.qa = field16(o_qa);
                pc.qb = field16(o_qb);
                pc.qh = field16(o_qh);
                const uint32_t* p = wb32 + (o_sc >> 2);
                const uint32_t sh = o_sc & 3u, w0 = p[0], w1 = p[1], w2 = p[2];
                pc.sc = make_uint2(__builtin_amdgcn_alignbyte(w1, w0, sh), __builtin_amdgcn_alignbyte(w2, w1, sh));
                const uint32_t* q = wb32 + (o_d >> 2);
                pc.d = __builtin_amdgcn_alignbyte(q[1], q[0], o_d & 3u);
            }
            // (the sums of the activations are the same for every window: hidden from the compiler, so that no product of theirs
            // with a constant is moved out of the loop and rounded on its own where the flat walk, which reloads them per window,
            // fuses it into a multiply-add)
            if constexpr (kIsX2<TYPE>) {  // (the K-quants' sums only meet block scales, which change with the window)
#pragma unroll
                for (int q = 0; q < 8; ++q) asm volatile("" : "+v"(sx[q]));
            }
            float part;
            if constexpr (X::PAIR) part = dot_pair(pc, c, xr, sx, m4, m2, magic);
            else part = dot_f32(pc, c, reinterpret_cast<const float*>(xr), sx);
            float mine = group_sum(seg == 0u ? part : 0.f, 6);
            if (nseg > 1u) {
                const float v = group_sum(seg == 1u ? part : 0.f, 6);
                mine = lane == 1u ? v : mine;
            }
            if (nseg > 2u) {
                const float v = group_sum(seg == 2u ? part : 0.f, 6);
                mine = lane == 2u ? v : mine;
            }
            if (lane < nseg) slots[((i_cur - i0) << LR) * MW + my_slot] = mine;
            i_cur += a.seqs;
        }
        __syncthreads();
        // the windows of row r of a period, added in the flat walk's order: 0 + first + second ...
        const uint32_t rows = (i1 - i0) << LR;
        for (uint32_t idx = tid; idx < rows; idx += nthreads) {
            const uint32_t r = idx & (R - 1u), fb = r * a.bu, nwin = (fb + a.bu - 1u) / UW - fb / UW + 1u;
            float y = 0.f;
            for (uint32_t sl = 0; sl < nwin; ++sl) y += slots[MW * idx + sl];
            a.y[((size_t)(blockIdx.x + (i0 + (idx >> LR)) * gridDim.x) << LR) + r] = y;
        }
        if (i1 < cnt_wg) __syncthreads();
    }
}
template <int TYPE>
constexpr uint32_t kPeriodWaveBuf = (kUnitsPerWindow<TYPE> * kBlockBytes<TYPE> / 16u + 63u) / 64u * 1024u;  // bytes of a wave's window buffer
template <int TYPE, bool X_BF16>
inline size_t period_lds(uint32_t k, uint32_t waves, uint32_t slots) {
    return FlatX<TYPE, X_BF16>::lds_bytes(k) + (size_t)waves * kPeriodWaveBuf<TYPE> + (size_t)slots * 4u;
}
// P windows = R rows: the period of the row boundaries for rows of bu units in windows of uw
inline void period_of(uint32_t bu, uint32_t uw, uint32_t* P, uint32_t* R) {
    uint32_t a = bu, b = uw;
    while (b) {
        const uint32_t t = a % b;
        a = b;
        b = t;
    }
    *P = bu / a;
    *R = uw / a;
}
// One 16-byte aligned matrix, rows of more than half a window (nine super-blocks, 33 block pairs) and not whole windows, a period of sixteen windows at
// most, whole periods of rows, 176 windows per workgroup or more, ten waves or more with f32 activations (nine: Q6_K 65536 x
// 4608 48.3 -> 49.3 us), and a shape for which the flat walk would use full windows over whole periods (so that both give the
// same bits).
template <int TYPE, bool X_BF16>
inline bool period_takes(const void* w, uint32_t n, uint32_t k, uint32_t cus) {
    constexpr uint32_t MAXW = kPeriodMaxWaves<TYPE, X_BF16>, UE = kUnitElems<TYPE>, UW = kUnitsPerWindow<TYPE>;
    if (k % UE) return false;
    const uint32_t bu = k / UE;
    // (more than half a window per row: a window touches three rows at most)
    if (bu <= UW / 2u || bu % UW == 0u || (reinterpret_cast<uintptr_t>(w) & 15u)) return false;
    uint32_t P, R;
    period_of(bu, UW, &P, &R);
    if (P > MAXW || n % R || (uint64_t)(n / R) * P < (uint64_t)176u * cus || (uint64_t)n * bu >= 0x7fff0000ull) return false;
    if ((!X_BF16 && MAXW / P * P < 10u) || period_lds<TYPE, X_BF16>(k, MAXW / P * P, 4096u) > 160u * 1024u - 512u) return false;
    const FlatGeom fg = flat_geom(k, UE, UW, n, 1u, cus * (kBaseType<TYPE> == HQ_Q6_K || TYPE == HQ_Q8_0_X2 ? 12u : 16u));  // (as launch_flat asks)
    return fg.uwe == UW && (1u << fg.log_r) == R;
}
template <int TYPE, bool X_BF16>
int launch_period(hipStream_t s, const void* x, const uint8_t* w, float* y, uint32_t n, uint32_t k, uint32_t cus) {
    constexpr uint32_t UW = kUnitsPerWindow<TYPE>;
    const uint32_t bu = k / kUnitElems<TYPE>;
    uint32_t P, R;
    period_of(bu, UW, &P, &R);
    const uint32_t seqs = kPeriodMaxWaves<TYPE, X_BF16> / P, W = seqs * P;
    uint32_t log_r = 0;
    while ((1u << log_r) < R) ++log_r;
    const uint32_t periods = n / R, per_wg = (periods + cus - 1u) / cus;
    const uint32_t mw = (bu + UW - 2u) / UW + 1u, cap = 4096u / (R * mw);  // 16 KB of slots
    const uint32_t ppr = per_wg < cap ? per_wg : cap;
    const PArgs pa{x, w, y, n, k, bu, P, log_r, seqs, mw, ppr, kBaseType<TYPE> == HQ_Q6_K ? N4 : M4, kBaseType<TYPE> == HQ_Q5_K ? M1 : kBaseType<TYPE> == HQ_Q6_K ? N2 : M2, MAGIC};
    const size_t lds = period_lds<TYPE, X_BF16>(k, W, ppr * R * mw);
    auto kern = gemv_period_kernel<TYPE, X_BF16>;
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, "hipFuncSetAttribute(gemv period LDS)")) return rc;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(64 * W), lds, s, pa);
    return check_launch("gemv period kernel launch");
}

// Whether the streaming form takes (type, k, rows): K-quants, whole 4096-element steps, enough rows to occupy the waves.
template <int TYPE>
constexpr bool kStreamType = TYPE == HQ_Q4_K || TYPE == HQ_Q5_K || TYPE == HQ_Q6_K;
constexpr uint32_t STREAM_MIN_ROWS_PER_WAVE = 2;

template <int TYPE, int ROWS = 1>
int launch_stream(hipStream_t s, const SArgs& sa, uint32_t cus) {
    constexpr int W = TYPE == HQ_Q6_K ? 12 : 16;
    const size_t lds = ROWS * ((size_t)sa.k * 2 + (size_t)(sa.k / 16) * 4);
    // (three and four rows in registers would spill, so would the two-row Q5_K form: not instantiated)
    constexpr bool XREG_FITS = ROWS <= 2 && !(TYPE == HQ_Q5_K && ROWS == 2);
    bool launched = false;
    if constexpr (TYPE == HQ_Q6_K && ROWS == 1) {
        // (12288 rows of 4096: 9.4 against 10.7 us; 4096 rows: the same)
        if (sa.n0 == sa.n && q6k_rowcopy_takes(sa.w0, sa.n, sa.k, cus)) return launch_q6k_rowcopy<true>(s, sa, cus);
    }
    if constexpr ((TYPE == HQ_Q4_K || TYPE == HQ_Q5_K) && ROWS == 1) {
        // (Q4_K 12288 x 4096: 7.75 -> 7.4 us, 151936 x 4096: 63 -> 59 us; Q5_K 12288 x 4096: 9.07 -> 8.46 us; the same bits)
        if (((reinterpret_cast<uintptr_t>(sa.w0) | reinterpret_cast<uintptr_t>(sa.w1)) & 15u) == 0) {
            constexpr size_t wbytes = (size_t)W * 64u * ((kBlockBytes<TYPE> + 63u) / 64u) * 16u;
            auto kern = sa.k == 4096 ? gemv_stream_kernel<TYPE, W, true, 1, true> : gemv_stream_kernel<TYPE, W, false, 1, true>;
            if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds + wbytes, "hipFuncSetAttribute(gemv stream LDS)")) return rc;
            hipLaunchKernelGGL(kern, dim3(cus), dim3(64 * W), lds + wbytes, s, sa);
            return check_launch("gemv stream kernel launch");
        }
    }
    if constexpr (XREG_FITS) {
        if (sa.k == 4096) {
            auto kern = gemv_stream_kernel<TYPE, W, true, ROWS>;
            if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, "hipFuncSetAttribute(gemv stream LDS)")) return rc;
            hipLaunchKernelGGL(kern, dim3(cus), dim3(64 * W), lds, s, sa);
            launched = true;
        }
    }
    if (!launched) {
        auto kern = gemv_stream_kernel<TYPE, W, false, ROWS>;
        if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, "hipFuncSetAttribute(gemv stream LDS)")) return rc;
        hipLaunchKernelGGL(kern, dim3(cus), dim3(64 * W), lds, s, sa);
    }
    return check_launch("gemv stream kernel launch");
}

// One f32 activation row over a 16-byte aligned Q4_K / Q5_K matrix with rows of 4096: the copy form of the streaming
// kernel, a lane's 64 activations in registers, 12 waves (16 would spill).  Longer rows, whose activations a lane reads
// from LDS step by step, stay with the flat walk: measured there the copy form gains nothing (4096 x 12288 Q4_K: 9.0
// against 8.6 us, and 4 us more behind the gate / up launch of a decode FFN).
template <int TYPE>
int launch_stream_f32(hipStream_t s, const SArgs& sa, uint32_t cus) {
    constexpr uint32_t W = 12;
    constexpr size_t wbytes = (size_t)W * 64u * ((kBlockBytes<TYPE> + 63u) / 64u) * 16u;
    const size_t lds = FlatX1<TYPE, false>::lds_bytes(sa.k) + wbytes;
    auto kern = gemv_stream_kernel<TYPE, W, true, 1, true, false>;
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, "hipFuncSetAttribute(gemv stream LDS)")) return rc;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(64 * W), lds, s, sa);
    return check_launch("gemv stream kernel launch");
}

template <int TYPE>
bool stream_takes(uint32_t n_total, uint32_t k, uint32_t cus) {
    constexpr uint32_t W = TYPE == HQ_Q6_K ? 12 : 16;
    return k % 4096 == 0 && k <= 24576 && (uint64_t)n_total * (k / 4096) >= (uint64_t)cus * W * STREAM_MIN_ROWS_PER_WAVE;
}
// Activation rows one pass of the streaming kernel can stage: ROWS * (2k + k / 4) bytes of a CU's 160 KiB of LDS.
inline uint32_t stream_rows_that_fit(uint32_t k) {
    const size_t per_row = (size_t)k * 2 + (size_t)(k / 16) * 4;
    const size_t fit = (160 * 1024 - 512) / per_row;
    return fit >= 4 ? 4u : (uint32_t)fit;
}

// Dense single-row GEMV for everything the kernel above does not take: f32 activations (the dtype of the reference's
// call sites), any k that is whole blocks (k = 2816, 2048, 11264 ...), Q8_0 / Q4_0.  One workgroup of W waves per CU, the
// activations staged once, one window of 64 lanes per wave in flight, windows laid over the matrix as one contiguous
// run of blocks whatever the row length (gemv_walk.h).  With two matrices of one shape over the same activations (gate
// and up of a decode step) a wave walks the same rows of both.
struct FArgs {
    const void* x;
    const uint8_t* w0;
    const uint8_t* w1;
    float* y0;
    float* y1;
    uint32_t n, k, nm;
    uint32_t swiglu;  // nm == 2: y0 = silu(W0 . x) * (W1 . x) instead of the two products
    FlatGeom g;
    uint32_t m4, m2, magic;
};

// DYN: the waves of a workgroup take its super-tasks from a counter (see gemv_walk.h): worth it where a wave has many
// (the 151936-row head in f32: 101 against 108 us); with a handful per wave the three claimed ahead are all there is.
template <int TYPE, bool X_BF16, int W, int D, bool DYN, bool COPY = false>
__global__ __launch_bounds__(64 * W) void gemv_flat_kernel(FArgs a) {
    using X = FlatX<TYPE, X_BF16>;
    extern __shared__ uint4 smem[];
    __shared__ uint32_t lds_queue;
    uint4* lds_x = smem;
    float* lds_s = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(smem) + X::value_bytes(a.k));
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    if (tid == 0) lds_queue = W;
    // the activations first, nothing else of this workgroup in front of them
    X::stage(a.x, a.k, lds_x, lds_s, tid, 64u * W);
    FlatWalk<TYPE, X_BF16, D, false, DYN, COPY> wk;
    // (COPY: a window buffer of 64 kCopyNPV slots of 16 bytes per wave behind the activations' sums)
    uint4* wbuf = COPY ? reinterpret_cast<uint4*>(lds_s + a.k / 16u) + wv * (64u * kCopyNPV<TYPE>) : nullptr;
    if constexpr (DYN)
        wk.init(a.w0, a.w1, a.n, a.nm, a.g, blockIdx.x, gridDim.x, &lds_queue, wv, wbuf);
    else
        wk.init(a.w0, a.w1, a.n, a.nm, a.g, wv * gridDim.x + blockIdx.x, W * gridDim.x, nullptr, 0, wbuf);
    if constexpr (!DYN) wk.prime();
    __syncthreads();
    if constexpr (DYN) wk.prime();
    wk.load_masks(a.m4, a.m2, a.magic);
    wk.run(lds_x, lds_s, [&](uint32_t cnt, float k0, float k1, uint32_t row) {
        if (lane < cnt && row < a.n) {
            if (a.swiglu) {
                a.y0[row] = silu_mul_f32(k0, k1);
            } else {
                a.y0[row] = k0;
                if (a.nm == 2u) a.y1[row] = k1;
            }
        }
    });
}

#ifndef HQ_FLAT_MIN_WINDOWS_PER_CU
#define HQ_FLAT_MIN_WINDOWS_PER_CU 8
#endif
#ifndef HQ_FLAT_D_Q80
#define HQ_FLAT_D_Q80 1
#endif
#ifndef HQ_FLAT_D_Q40
#define HQ_FLAT_D_Q40 1
#endif
// Whether the flat form takes (type, rows, k): about a window per wave of the device or more, block counts that fit 32 bits.
template <int TYPE>
bool flat_takes(uint64_t n_total, uint32_t k, uint32_t cus, size_t lds) {
    constexpr uint32_t UE = kUnitElems<TYPE>, UW = kUnitsPerWindow<TYPE>;
    if (k % UE || k / UE < 2 || lds > 160 * 1024 - 512) return false;
    const uint64_t units = n_total * (k / UE);
    return units < 0x7fff0000ull && units / UW >= (uint64_t)cus * HQ_FLAT_MIN_WINDOWS_PER_CU;
}
// One small matrix (the projections of a decode step: 512 .. 4096 rows): the flat form from half a window per CU on, where
// the kernel of 4-wave workgroups below is the slower one -- f32 activations (Q4_K 2048 x 1024: 4.35 -> 3.25 us, 128 x 4096: 4.2 ->
// 3.1), 32-weight blocks with rows of 2048 weights or more (Q8_0 512 x 4096: 3.8 -> 3.55) -- and from sixteen windows on for
// rows whose unit count is not a power of two, which that kernel's lane groups fit badly (k = 2816, 1024 rows: Q5_K 9.8 / 12.7 ->
// 3.2 / 3.4 us, Q6_K 10.2 / 11.4 -> 3.2 / 3.4, Q8_0 8.0 -> 3.5; k = 5120, 1024 rows: Q4_K 5.7 / 11.8 -> 3.7 / 4.1).  K-quant rows
// of a power-of-two length under bf16 activations stay with it (Q4_K 2048 x 512: 2.5 against 3.4 us).
template <int TYPE, bool X_BF16>
bool flat_takes_small(uint64_t n_total, uint32_t k, uint32_t cus, size_t lds) {
    constexpr uint32_t UE = kUnitElems<TYPE>, UW = kUnitsPerWindow<TYPE>;
    if (k % UE || k / UE < 2 || lds > 160 * 1024 - 512) return false;
    const uint32_t bu = k / UE;
    const uint64_t windows = n_total * bu / UW;
    if (n_total * bu >= 0x7fff0000ull) return false;
    if (bu & (bu - 1u)) return windows * 16u >= cus;
    return ((!X_BF16 && bu >= 4u) || (kBlock32<TYPE> && k >= 2048u)) && windows * 2u >= cus;  // (rows of two super-blocks: 2048 x 512 f32 3.2 against 3.4 us)
}
// Fetches a wave keeps in flight: one (a ring of two or four windows of 32-weight blocks, which are only 1.1 / 2.2 KB,
// measured slower: Q4_0 12288 x 4096 13.8 against 9.7 us).
template <int TYPE>
constexpr int kFlatDepth = kIsX2<TYPE> ? 1 : TYPE == HQ_Q8_0 ? HQ_FLAT_D_Q80 : TYPE == HQ_Q4_0 ? HQ_FLAT_D_Q40 : 1;

template <int TYPE, bool X_BF16>
int launch_flat(hipStream_t s, const void* x, const uint8_t* w0, const uint8_t* w1, float* y0, float* y1, uint32_t n, uint32_t k,
                uint32_t nm, uint32_t cus, bool swiglu = false) {
    if constexpr (kBlock32<TYPE>)
        if (walk_doubled<TYPE, X_BF16>((uint64_t)n * nm, k)) return launch_flat<kX2 + TYPE, X_BF16>(s, x, w0, w1, y0, y1, n, k, nm, cus, swiglu);
    // waves per CU: 16; 12 for Q6_K (measured with both activation types: f32 262144 x 2816 123 -> 117 us, 8192 x 28672
    // 43.8 -> 38.9, 4096 x 14336 14.9 -> 13.0; bf16 112 against 121 with 16) and for Q8_0 block pairs, whose windows are
    // copied through LDS (12288 x 4096 12.0 -> 11.1 us, 4096 x 14336 14.2 -> 13.1, 262144 x 2816 127.3 -> 123.1; 5120 x 17408
    // 19.6 -> 20.3); Q4_K, Q5_K and Q4_0 are faster or equal with 16
    constexpr int W = kBaseType<TYPE> == HQ_Q6_K || TYPE == HQ_Q8_0_X2 ? 12 : 16;
    using X = FlatX<TYPE, X_BF16>;
    const FArgs fa{x, w0, w1, y0, y1, n, k, nm, swiglu ? 1u : 0u, flat_geom(k, kUnitElems<TYPE>, kUnitsPerWindow<TYPE>, n, nm, cus * W),
                   kBaseType<TYPE> == HQ_Q6_K ? N4 : M4, kBaseType<TYPE> == HQ_Q5_K ? M1 : kBaseType<TYPE> == HQ_Q6_K ? N2 : M2, MAGIC};
    const uint64_t supers = ((uint64_t)n + (1u << fa.g.log_r) - 1) >> fa.g.log_r;
    const bool dyn = kFlatDepth<TYPE> == 1 && supers >= (uint64_t)cus * W * 8u;
    auto kern = dyn ? gemv_flat_kernel<TYPE, X_BF16, W, 1, true> : gemv_flat_kernel<TYPE, X_BF16, W, kFlatDepth<TYPE>, false>;
    size_t lds = X::lds_bytes(k);
    if constexpr (TYPE == HQ_Q6_K && X_BF16) {
        // Windows copied through LDS (see FlatWalk) where every window starts on a 16-byte boundary, no copy reads past the
        // matrix and a row is a window or more: 8192 x 28672 37.0 -> 33.5 us, 17408 x 5120 17.5 -> 16.7, 4096 x 14336 11.75 ->
        // 11.4; rows shorter than a window gain nothing (262144 x 2816: 108.5 against 110), and with f32 activations, whose
        // products keep the VALU busier, the form is slower (262144 x 2816: 124 against 112 us)
        if (fa.g.bu >= kUnitsPerWindow<TYPE> && flat_copy_fits(fa.g, kUnitsPerWindow<TYPE>, n, kCopyAlignUnits<TYPE>, reinterpret_cast<uintptr_t>(w0), reinterpret_cast<uintptr_t>(w1)) &&
            lds + (size_t)W * 4096u <= 160 * 1024 - 512) {
            kern = dyn ? gemv_flat_kernel<TYPE, X_BF16, W, 1, true, true> : gemv_flat_kernel<TYPE, X_BF16, W, 1, false, true>;
            lds += (size_t)W * 4096u;
        }
    }
    if constexpr (TYPE == kX2 + HQ_Q4_0) {
        // Q4_0 block pairs (windows of 2304 bytes, nine words per lane): 12288 x 4096 8.3 -> 7.4 us, 17408 x 5120 14.5 -> 12.7,
        // 8192 x 28672 28.6 -> 26.0, f32 activations 8.5 -> 7.5 / 15.3 -> 14.0 / the same; with f32 activations and rows shorter
        // than a window (262144 x 2816) 89.8 -> 93.9, so not there
        constexpr size_t wb = (size_t)W * 64u * kCopyNPV<TYPE> * 16u;
        if ((X_BF16 || fa.g.bu >= kUnitsPerWindow<TYPE>) && flat_copy_fits(fa.g, kUnitsPerWindow<TYPE>, n, kCopyAlignUnits<TYPE>, reinterpret_cast<uintptr_t>(w0), reinterpret_cast<uintptr_t>(w1)) &&
            lds + wb <= 160 * 1024 - 512) {
            kern = dyn ? gemv_flat_kernel<TYPE, X_BF16, W, 1, true, true> : gemv_flat_kernel<TYPE, X_BF16, W, 1, false, true>;
            lds += wb;
        }
    }
    if constexpr (TYPE == HQ_Q8_0_X2) {
        // Q8_0 block pairs (windows of 4352 bytes, read back as seventeen aligned words per lane), either activation type:
        // lm_head 262144 x 2816 140.7 -> 127.2 us (f32 135.0 -> 122.8), 5120 x 17408 21.3 -> 20.2, 12288 x 4096 12.3 -> 12.0
        constexpr size_t wb = (size_t)W * 64u * kCopyNPV<TYPE> * 16u;
        if (flat_copy_fits(fa.g, kUnitsPerWindow<TYPE>, n, kCopyAlignUnits<TYPE>, reinterpret_cast<uintptr_t>(w0), reinterpret_cast<uintptr_t>(w1)) &&
            lds + wb <= 160 * 1024 - 512) {
            kern = dyn ? gemv_flat_kernel<TYPE, X_BF16, W, 1, true, true> : gemv_flat_kernel<TYPE, X_BF16, W, 1, false, true>;
            lds += wb;
        }
    }
    if (lds < 81 * 1024) lds = 81 * 1024;  // more than half a CU's LDS: one workgroup per CU
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds, "hipFuncSetAttribute(gemv flat LDS)")) return rc;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(64 * W), lds, s, fa);
    return check_launch("gemv flat kernel launch");
}

template <typename K>
int set_lds_limit(K kern, size_t lds, const char* what) {
    return ensure_lds_limit(reinterpret_cast<const void*>(kern), (size_t)lds, what);
}

template <int TYPE, bool X_BF16, bool PAIR, int NR, int D>
int launch_r(hipStream_t s, const KArgs& ka, uint32_t pairs, uint32_t rpw, size_t lds) {
    auto kern = gemv_kernel<TYPE, X_BF16, PAIR, NR, D>;
    if (int rc = set_lds_limit(kern, lds, "hipFuncSetAttribute(gemv LDS)")) return rc;
    const uint32_t rows_per_wg = 4 * rpw * NR;
    hipLaunchKernelGGL(kern, dim3((ka.n + rows_per_wg - 1) / rows_per_wg, pairs), dim3(256), lds, s, ka);
    return check_launch("gemv kernel launch");
}

template <int TYPE, bool X_BF16, bool PAIR, int NR, int D, int WAVES>
int launch_q(hipStream_t s, KArgs ka, uint32_t cus, uint32_t rpw, size_t lds) {
    auto kern = gemv_queue_kernel<TYPE, X_BF16, PAIR, NR, D, WAVES>;
    if (lds < 81 * 1024) lds = 81 * 1024;  // more than half a CU's LDS: one workgroup per CU
    if (int rc = set_lds_limit(kern, lds, "hipFuncSetAttribute(gemv queue LDS)")) return rc;
    const uint32_t rows_per_group = rpw * NR;
    ka.groups = (ka.n + rows_per_group - 1) / rows_per_group;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(64 * WAVES), lds, s, ka);
    return check_launch("gemv queue kernel launch");
}

// Lanes per row, LDS bytes and slot count of one job.
template <int TYPE, bool X_BF16>
int plan_job(const GemvArgs& a, KArgs* ka, size_t* lds, uint64_t* slots) {
    constexpr bool PAIR = X_BF16 && !kBlock32<TYPE>;
    constexpr int EPL = Lane<TYPE>::kElems;
    if (a.x2 && X_BF16) return fail(HQ_ERR_UNSUPPORTED, "gemv: the fused SwiGLU form takes f32 activations");
    *ka = KArgs{a.x, a.x2, a.w, a.ids, a.route_logits, a.route_ids, a.route_w, a.y, a.top_k, a.n, a.k, a.n_experts, a.expert_stride, 0, 0, a.pairs, 0, TYPE == HQ_Q6_K ? N4 : M4, TYPE == HQ_Q5_K ? M1 : TYPE == HQ_Q6_K ? N2 : M2, MAGIC};
    const uint32_t pieces = a.k / EPL;
    // L = largest power of two <= 64 that divides the pieces of a row ...
    uint32_t log_l = 0;
    while (log_l < 6 && pieces % (2u << log_l) == 0) ++log_l;
    // ... unless that leaves fewer than sixteen lanes per row (k = 2816: 44 quarters of a super-block, four lanes walking eleven
    // steps each; 1024 x 2816 Q5_K: 9.8 us): then the L of 16, 32, 64 that wastes the fewest lane steps, the last step of a row
    // ragged, its idle lanes multiplying zeros staged behind the activations (q / k / v of 4096 + 1024 + 1024 rows x 2816 as one
    // launch, Q5_K: 12.9 -> 8.8 us).  bf16 activations only: with f32 ones the four times as many workgroups, each staging 11 KB
    // of them, cost more than the shorter walk saves (15.8 -> 20.3 us)
    if (X_BF16 && log_l < 4 && pieces >= 12) {
        uint32_t best = 0;
        for (uint32_t l = 4; l <= 6; ++l) {
            const uint32_t padded = (pieces + (1u << l) - 1u) >> l << l;
            if (!best || padded <= best) best = padded, log_l = l;
        }
        ka->xpad = kBlock32<TYPE> ? 32u : 256u;
    }
    ka->log_l = log_l;
    const uint32_t rpw = 64u >> log_l;
    // activations (and the zeros behind them), their per-16 sums, the queue counter
    const uint32_t kx = a.k + ka->xpad;
    *lds = (size_t)(PAIR ? kx * 2 : kx * 4) + (size_t)(kx / 16) * 4 + 16;
    if (*lds > 160 * 1024 - 512)
        return fail(HQ_ERR_UNSUPPORTED, "gemv: k = %u needs %zu bytes of LDS (limit 160 KiB)", a.k, *lds);
    *slots = (uint64_t)((a.n + rpw - 1) / rpw) * a.pairs;
    return HQ_OK;
}

template <int TYPE, bool X_BF16>
int launch_t(hipStream_t s, const GemvArgs& a) {
    constexpr bool PAIR = X_BF16 && !kBlock32<TYPE>;
    constexpr int EPL = Lane<TYPE>::kElems;
    KArgs ka;
    size_t lds;
    uint64_t slots;
    if (int rc = plan_job<TYPE, X_BF16>(a, &ka, &lds, &slots)) return rc;
    const uint32_t log_l = ka.log_l, rpw = 64u >> log_l;
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    if constexpr (X_BF16 && kStreamType<TYPE>) {
        // (one row over Q6_K rows longer than 4096: the flat walk with its windows copied through LDS is the faster where
        // that form fits -- 4096 x 12288 11.2 -> 9.9 us, 128256 x 8192 145.5 -> 135.7, 8192 x 24576 32.2 -> 29.4; the same bits)
        bool flat_copy_instead = false;
        if constexpr (TYPE == HQ_Q6_K) {
            if (a.pairs == 1 && a.k > 4096 && flat_takes<TYPE>(a.n, a.k, cus, FlatX<TYPE, true>::lds_bytes(a.k) + 12u * 4096u)) {
                const FlatGeom g = flat_geom(a.k, kUnitElems<TYPE>, kUnitsPerWindow<TYPE>, a.n, 1, cus * 12u);
                flat_copy_instead = flat_copy_fits(g, kUnitsPerWindow<TYPE>, a.n, kCopyAlignUnits<TYPE>, reinterpret_cast<uintptr_t>(a.w), reinterpret_cast<uintptr_t>(a.w));
            }
        }
        if (a.top_k == 1 && !a.x2 && !a.ids && !a.route_logits && stream_takes<TYPE>(a.n, a.k, cus) && !flat_copy_instead) {
            // activation rows of a dense product up to four at a time (one pass over the weights for them)
            for (uint32_t r = 0; r < a.pairs;) {
                const SArgs sa{static_cast<const uint8_t*>(a.x) + (size_t)r * a.k * 2, a.w, a.w, a.y + (size_t)r * a.n, a.y + (size_t)r * a.n,
                               a.n, a.n, a.k, TYPE == HQ_Q6_K ? N4 : M4, TYPE == HQ_Q5_K ? M1 : TYPE == HQ_Q6_K ? N2 : M2, MAGIC};
                const uint32_t fit = stream_rows_that_fit(a.k), left = a.pairs - r, take = left >= fit ? fit : left;
                if (int rc = take == 4   ? launch_stream<TYPE, 4>(s, sa, cus)
                             : take == 3 ? launch_stream<TYPE, 3>(s, sa, cus)
                             : take == 2 ? launch_stream<TYPE, 2>(s, sa, cus)
                                         : launch_stream<TYPE, 1>(s, sa, cus))
                    return rc;
                r += take;
            }
            return HQ_OK;
        }
    }
    // f32 activations over Q4_K / Q5_K rows of 4096: the copy form of the streaming kernel, a pass per row
    // (12288 x 4096: Q4_K 8.2 -> 7.7 us, Q5_K 9.1 -> 8.2 on one device, no difference on another)
    if constexpr (!X_BF16 && (TYPE == HQ_Q4_K || TYPE == HQ_Q5_K)) {
        if (a.top_k == 1 && !a.x2 && !a.ids && !a.route_logits && a.k == 4096 && stream_takes<TYPE>(a.n, a.k, cus) &&
            (reinterpret_cast<uintptr_t>(a.w) & 15u) == 0) {
            for (uint32_t r = 0; r < a.pairs; ++r) {
                const SArgs sa{static_cast<const uint8_t*>(a.x) + (size_t)r * a.k * 4, a.w, a.w, a.y + (size_t)r * a.n, a.y + (size_t)r * a.n,
                               a.n, a.n, a.k, 0, 0, 0};
                if (int rc = launch_stream_f32<TYPE>(s, sa, cus)) return rc;
            }
            return HQ_OK;
        }
    }
    // Q6_K rows of 4096 / 2048 elements not taken above (f32 activations, k = 2048): chunks copied through LDS, a pass per row.
    if constexpr (TYPE == HQ_Q6_K) {
        if (a.top_k == 1 && !a.x2 && !a.ids && !a.route_logits && q6k_rowcopy_takes(a.w, a.n, a.k, cus)) {
            for (uint32_t r = 0; r < a.pairs; ++r) {
                const SArgs sa{static_cast<const uint8_t*>(a.x) + (size_t)r * a.k * (X_BF16 ? 2 : 4), a.w, a.w, a.y + (size_t)r * a.n,
                               a.y + (size_t)r * a.n, a.n, a.n, a.k, N4, N2, MAGIC};
                if (int rc = launch_q6k_rowcopy<X_BF16>(s, sa, cus)) return rc;
            }
            return HQ_OK;
        }
    }
    // K-quant rows that are not whole windows (lm_heads of hidden size 2560 .. 3840, 5120, 7168; k = 14336): a fixed window of
    // the row period per wave, a pass per row.
    if constexpr (kBlock32<TYPE>) {  // (as block pairs, where the flat walk would pair them)
        if (a.top_k == 1 && !a.x2 && !a.ids && !a.route_logits && walk_doubled<TYPE, X_BF16>(a.n, a.k) &&
            period_takes<kX2 + TYPE, X_BF16>(a.w, a.n, a.k, cus)) {
            for (uint32_t r = 0; r < a.pairs; ++r)
                if (int rc = launch_period<kX2 + TYPE, X_BF16>(s, static_cast<const uint8_t*>(a.x) + (size_t)r * a.k * (X_BF16 ? 2 : 4), a.w,
                                                               a.y + (size_t)r * a.n, a.n, a.k, cus))
                    return rc;
            return HQ_OK;
        }
    }
    if constexpr (TYPE == HQ_Q4_K || TYPE == HQ_Q5_K || TYPE == HQ_Q6_K) {
        if (a.top_k == 1 && !a.x2 && !a.ids && !a.route_logits && period_takes<TYPE, X_BF16>(a.w, a.n, a.k, cus)) {
            for (uint32_t r = 0; r < a.pairs; ++r)
                if (int rc = launch_period<TYPE, X_BF16>(s, static_cast<const uint8_t*>(a.x) + (size_t)r * a.k * (X_BF16 ? 2 : 4), a.w,
                                                       a.y + (size_t)r * a.n, a.n, a.k, cus))
                    return rc;
            return HQ_OK;
        }
    }
    // Other dense matrices with enough rows (any k of whole blocks, f32 activations, Q8_0 / Q4_0): the flat streaming form,
    // one pass per activation row.
    if (a.top_k == 1 && !a.x2 && !a.ids && !a.route_logits &&
        (flat_takes<TYPE>(a.n, a.k, cus, FlatX<TYPE, X_BF16>::lds_bytes(a.k)) || flat_takes_small<TYPE, X_BF16>(a.n, a.k, cus, FlatX<TYPE, X_BF16>::lds_bytes(a.k)))) {
        for (uint32_t r = 0; r < a.pairs; ++r)
            if (int rc = launch_flat<TYPE, X_BF16>(s, static_cast<const uint8_t*>(a.x) + (size_t)r * a.k * (X_BF16 ? 2 : 4), a.w, a.w,
                                                   a.y + (size_t)r * a.n, a.y + (size_t)r * a.n, a.n, a.k, 1, cus))
                return rc;
        return HQ_OK;
    }
    // Dense matrices with many tasks per wave: the queue kernel.
    if (a.pairs == 1 && !a.x2 && !a.ids && !a.route_logits &&
        slots * ((a.k / EPL) >> log_l) >= (uint64_t)cus * QUEUE_MIN_TASKS_PER_CU)
        return launch_q<TYPE, X_BF16, PAIR, 2, 2, 12>(s, ka, cus, rpw, lds);
    // Slots one SIMD would get if the work were spread evenly; more slots per wave
    // amortise the per-wave set-up, fewer keep every SIMD busy on small problems.
    const uint64_t per_simd = slots / (4ull * cus);
    if (per_simd >= 8) return launch_r<TYPE, X_BF16, PAIR, 4, 4>(s, ka, a.pairs, rpw, lds);
    if (per_simd >= 2) return launch_r<TYPE, X_BF16, PAIR, 2, 2>(s, ka, a.pairs, rpw, lds);
    return launch_r<TYPE, X_BF16, PAIR, 1, 1>(s, ka, a.pairs, rpw, lds);
}

template <int TYPE, bool X_BF16, bool PAIR, int NR, int D>
int launch_j(hipStream_t s, const KJobs& js, uint32_t n_jobs, size_t lds) {
    auto kern = gemv_jobs_kernel<TYPE, X_BF16, PAIR, NR, D>;
    if (int rc = set_lds_limit(kern, lds, "hipFuncSetAttribute(gemv jobs LDS)")) return rc;
    uint32_t gx = 0, gy = 0;
    for (uint32_t i = 0; i < n_jobs; ++i) {
        const uint32_t rows_per_wg = 4u * (64u >> js.j[i].log_l) * NR;
        const uint32_t bx = (js.j[i].n + rows_per_wg - 1) / rows_per_wg;
        gx = bx > gx ? bx : gx;
        gy = js.j[i].pairs > gy ? js.j[i].pairs : gy;
    }
    hipLaunchKernelGGL(kern, dim3(gx, gy, n_jobs), dim3(256), lds, s, js);
    return check_launch("gemv jobs kernel launch");
}

template <int TYPE, bool X_BF16>
int launch_jobs_t(hipStream_t s, const GemvArgs* jobs, uint32_t n_jobs) {
    constexpr bool PAIR = X_BF16 && !kBlock32<TYPE>;
    KJobs js{};
    size_t lds = 0;
    uint64_t slots = 0;
    for (uint32_t i = 0; i < n_jobs; ++i) {
        size_t l;
        uint64_t sl;
        if (int rc = plan_job<TYPE, X_BF16>(jobs[i], &js.j[i], &l, &sl)) return rc;
        lds = l > lds ? l : lds;
        slots += sl;
    }
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    if constexpr (X_BF16 && kStreamType<TYPE>) {
        const GemvArgs &j0 = jobs[0], &j1 = jobs[1];
        auto plain = [](const GemvArgs& j) { return j.pairs == 1 && !j.x2 && !j.ids && !j.route_logits; };
        if (n_jobs == 2 && plain(j0) && plain(j1) && j0.x == j1.x && j0.k == j1.k && stream_takes<TYPE>(j0.n + j1.n, j0.k, cus))
            return launch_stream<TYPE>(s, SArgs{j0.x, j0.w, j1.w, j0.y, j1.y, j0.n, j0.n + j1.n, j0.k, TYPE == HQ_Q6_K ? N4 : M4, TYPE == HQ_Q5_K ? M1 : TYPE == HQ_Q6_K ? N2 : M2, MAGIC}, cus);
    }
    {
        const GemvArgs &j0 = jobs[0], &j1 = jobs[1];
        auto plain = [](const GemvArgs& j) { return j.pairs == 1 && !j.x2 && !j.ids && !j.route_logits; };
        if (n_jobs == 2 && plain(j0) && plain(j1) && j0.x == j1.x && j0.k == j1.k && j0.n == j1.n &&
            flat_takes<TYPE>((uint64_t)j0.n * 2, j0.k, cus, FlatX<TYPE, X_BF16>::lds_bytes(j0.k)))
            return launch_flat<TYPE, X_BF16>(s, j0.x, j0.w, j1.w, j0.y, j1.y, j0.n, j0.k, 2, cus);
    }
    const uint64_t per_simd = slots / (4ull * cus);
    if (per_simd >= 8) return launch_j<TYPE, X_BF16, PAIR, 4, 4>(s, js, n_jobs, lds);
    if (per_simd >= 2) return launch_j<TYPE, X_BF16, PAIR, 2, 2>(s, js, n_jobs, lds);
    return launch_j<TYPE, X_BF16, PAIR, 1, 1>(s, js, n_jobs, lds);
}

}  // namespace

// A K-quant with bf16 activations on a matrix the streaming kernel takes: passes of up to four rows (one pass over the
// weights each, every row's sum in the order of the one-row form) against the small-batch MFMA kernels, which cost the
// same for any 3 / 4 .. 8 rows.  Q6_K, 151936 x 4096: 163 / 173 us for three / four rows and 252 .. 281 for five .. seven
// against 307; 12288 x 4096: 13 .. 28 against 29.  Q4_K / Q5_K: three and four rows, 10.8 / 12.9 against 14.2 us at
// 12288 x 4096 (102 / 132 against 134 at 151936 x 4096); from five rows on their small-batch kernel is ahead.
// Where the small-batch kernel has its stage-once form (gemv_rows_stream_fast: Q6_K 151936 x 4096 134 us, Q4_K 65536 x 4096
// 41 us, Q4_K / Q6_K 12288 x 4096 13 / 21 us for any 3 .. 8 rows) it is ahead from five rows on, and from three on
// matrices of 32768 rows or more (three and four rows in passes: 55 / 62 us on the 65536-row Q4_K matrix).
// The flat walk's plan for an n x k matrix of type t on `waves` waves (host arithmetic).
void gemv_flat_plan(hq_ggml_type t, uint32_t n, uint32_t k, uint32_t waves, uint32_t* units_per_row, uint32_t* rows_per_task,
                    uint32_t* windows_per_task, uint32_t* units_per_window, uint32_t* window_capacity) {
    const bool b32 = t == HQ_Q8_0 || t == HQ_Q4_0;
    const uint32_t ue = b32 ? 32u : 256u, uw = b32 ? 64u : 16u;
    const FlatGeom g = flat_geom(k, ue, uw, n, 1, waves);
    *units_per_row = g.bu;
    *rows_per_task = 1u << g.log_r;
    *windows_per_task = g.st;
    *units_per_window = g.uwe;
    *window_capacity = uw;
}

bool gemv_stream_passes_preferred(hq_ggml_type t, hq_act_dtype xdt, uint32_t m, uint32_t n, uint32_t k) {
    if (xdt != HQ_BF16 || m < 3) return false;
    uint32_t cus = 0;
    if (cu_count(&cus)) return false;
    if (gemv_rows_stream_fast(t, xdt, m, n, k) && (m >= 5 || n >= 32768)) return false;
    if (t == HQ_Q6_K) return m <= 7 && stream_takes<HQ_Q6_K>(n, k, cus);
    if (t == HQ_Q4_K) return m <= 4 && stream_takes<HQ_Q4_K>(n, k, cus);
    if (t == HQ_Q5_K) return m <= 4 && stream_takes<HQ_Q5_K>(n, k, cus);
    return false;
}

namespace {
template <int TYPE, bool X_BF16>
int swiglu_t(hipStream_t s, const void* x, const void* wg, const void* wu, float* y, uint32_t m, uint32_t n, uint32_t k, bool dry) {
    uint32_t cus = 256;
    if (!dry)
        if (int rc = cu_count(&cus)) return rc;
    if (!flat_takes<TYPE>((uint64_t)n * 2, k, cus, FlatX<TYPE, X_BF16>::lds_bytes(k)))
        return fail(HQ_ERR_UNSUPPORTED, "gate + up + SwiGLU GEMV: %u x %u is too small for the streaming form (or k = %u does not fit a CU's LDS)", n, k, k);
    if (dry) return HQ_OK;
    for (uint32_t r = 0; r < m; ++r)
        if (int rc = launch_flat<TYPE, X_BF16>(s, static_cast<const uint8_t*>(x) + (size_t)r * k * (X_BF16 ? 2 : 4), static_cast<const uint8_t*>(wg),
                                               static_cast<const uint8_t*>(wu), y + (size_t)r * n, y + (size_t)r * n, n, k, 2, cus, true))
            return rc;
    return HQ_OK;
}
}  // namespace

// y[r] = silu(W_gate . x[r]) * (W_up . x[r]) for m activation rows, one pass over both matrices per row; dry: only whether
// the shape is taken.
int launch_gemv_swiglu(hipStream_t s, const void* x, hq_act_dtype xdt, const void* wg, const void* wu, float* y, uint32_t m, uint32_t n,
                       uint32_t k, hq_ggml_type t, bool dry) {
    const bool bf = xdt == HQ_BF16;
    switch (t) {
        case HQ_Q4_K: return bf ? swiglu_t<HQ_Q4_K, true>(s, x, wg, wu, y, m, n, k, dry) : swiglu_t<HQ_Q4_K, false>(s, x, wg, wu, y, m, n, k, dry);
        case HQ_Q6_K: return bf ? swiglu_t<HQ_Q6_K, true>(s, x, wg, wu, y, m, n, k, dry) : swiglu_t<HQ_Q6_K, false>(s, x, wg, wu, y, m, n, k, dry);
        case HQ_Q8_0: return bf ? swiglu_t<HQ_Q8_0, true>(s, x, wg, wu, y, m, n, k, dry) : swiglu_t<HQ_Q8_0, false>(s, x, wg, wu, y, m, n, k, dry);
        case HQ_Q5_K: return bf ? swiglu_t<HQ_Q5_K, true>(s, x, wg, wu, y, m, n, k, dry) : swiglu_t<HQ_Q5_K, false>(s, x, wg, wu, y, m, n, k, dry);
        case HQ_Q4_0: return bf ? swiglu_t<HQ_Q4_0, true>(s, x, wg, wu, y, m, n, k, dry) : swiglu_t<HQ_Q4_0, false>(s, x, wg, wu, y, m, n, k, dry);
    }
    return fail(HQ_ERR_UNSUPPORTED, "gemv: ggml type %d", (int)t);
}

int launch_gemv(hipStream_t s, const GemvArgs& a, hq_act_dtype xdt, hq_ggml_type t) {
    const bool bf = xdt == HQ_BF16;
    switch (t) {
        case HQ_Q4_K: return bf ? launch_t<HQ_Q4_K, true>(s, a) : launch_t<HQ_Q4_K, false>(s, a);
        case HQ_Q6_K: return bf ? launch_t<HQ_Q6_K, true>(s, a) : launch_t<HQ_Q6_K, false>(s, a);
        case HQ_Q8_0: return bf ? launch_t<HQ_Q8_0, true>(s, a) : launch_t<HQ_Q8_0, false>(s, a);
        case HQ_Q5_K: return bf ? launch_t<HQ_Q5_K, true>(s, a) : launch_t<HQ_Q5_K, false>(s, a);
        case HQ_Q4_0: return bf ? launch_t<HQ_Q4_0, true>(s, a) : launch_t<HQ_Q4_0, false>(s, a);
    }
    return fail(HQ_ERR_UNSUPPORTED, "gemv: ggml type %d", (int)t);
}

int launch_gemv_jobs(hipStream_t s, const GemvArgs* jobs, uint32_t n_jobs, hq_act_dtype xdt, hq_ggml_type t) {
    if (n_jobs == 0) return HQ_OK;
    if (n_jobs == 1) return launch_gemv(s, jobs[0], xdt, t);
    if (n_jobs > MAX_JOBS) return fail(HQ_ERR_INVALID_ARGUMENT, "gemv: %u jobs in one launch (limit %u)", n_jobs, MAX_JOBS);
    const bool bf = xdt == HQ_BF16;
    switch (t) {
        case HQ_Q4_K: return bf ? launch_jobs_t<HQ_Q4_K, true>(s, jobs, n_jobs) : launch_jobs_t<HQ_Q4_K, false>(s, jobs, n_jobs);
        case HQ_Q6_K: return bf ? launch_jobs_t<HQ_Q6_K, true>(s, jobs, n_jobs) : launch_jobs_t<HQ_Q6_K, false>(s, jobs, n_jobs);
        case HQ_Q8_0: return bf ? launch_jobs_t<HQ_Q8_0, true>(s, jobs, n_jobs) : launch_jobs_t<HQ_Q8_0, false>(s, jobs, n_jobs);
        case HQ_Q5_K: return bf ? launch_jobs_t<HQ_Q5_K, true>(s, jobs, n_jobs) : launch_jobs_t<HQ_Q5_K, false>(s, jobs, n_jobs);
        case HQ_Q4_0: return bf ? launch_jobs_t<HQ_Q4_0, true>(s, jobs, n_jobs) : launch_jobs_t<HQ_Q4_0, false>(s, jobs, n_jobs);
    }
    return fail(HQ_ERR_UNSUPPORTED, "gemv: ggml type %d", (int)t);
}

}  // namespace hq

// The streaming row walk shared by the dense GEMV of any k (gemv.hip) and the one-launch dense FFN block
// (dense_ffn.hip).
//
// A weight matrix [n][k] of GGML blocks is one contiguous run of units (a unit = one 256-weight super-block of a
// K-quant, four lanes, or one 32-weight block of Q8_0 / Q4_0, one lane).  A wave reads it in WINDOWS of 64 lanes =
// 16 super-blocks (2304 .. 3360 contiguous bytes) or 64 blocks (1152 / 2176 bytes), whatever the row length is:
// a window may start and end in the middle of a row.  Windows are grouped into SUPER-TASKS of R whole rows = ST windows
// (R a power of two; the host picks R and the units per window, flat_geom below); a wave owns super-tasks first,
// first + stride, ...  After the dot products of a window the
// lanes' partial sums are added per row (one masked wave reduction for every row the window touches) into the
// lane that keeps that row's result; 64 finished rows leave through one call of the caller's output functor.
//
// One fetch per wave is in flight (D = 1), or a ring of D; every fetch is unconditional (past the wave's last task it
// repeats the last one) and its address is clamped to the matrix, so the loop has one path and no branch around a load.
#pragma once

#include "gemv_pieces.h"

namespace hq {
namespace {

template <int TYPE>
constexpr bool kLaneUnit = kBlock32<kBaseType<TYPE>>;  // a unit is one lane's piece
template <int TYPE>
constexpr uint32_t kLanesPerUnit = kLaneUnit<TYPE> ? 1u : 4u;
template <int TYPE>
constexpr uint32_t kUnitsPerWindow = 64u / kLanesPerUnit<TYPE>;
template <int TYPE>
constexpr uint32_t kUnitElems = (kLaneUnit<TYPE> ? 32u : 256u) * (kIsX2<TYPE> ? 2u : 1u);

// Whether rows of type t are walked with doubled pieces (kX2 + t): the 32-weight block types (Q8_0 12288 x 4096: 15.9 ->
// 12.4 us; the K-quants, whose pieces are larger and whose arithmetic is heavier, lose 7 .. 50 % to the registers a
// doubled piece takes), rows of whole doubled units, about a window per wave of the device or more.  The same rule
// wherever the walk is used, so that every caller gets the same sums.
template <int TYPE, bool X_BF16>
inline bool walk_doubled(uint64_t n_total, uint32_t k) {
    static_assert(!kIsX2<TYPE>, "asked of the base type");
    if (!kBlock32<TYPE>) return false;
    constexpr uint32_t UE2 = 2u * kUnitElems<TYPE>;
    return k % UE2 == 0 && n_total * (k / UE2) >= (uint64_t)kUnitsPerWindow<TYPE> * 4096ull;
}

struct FlatGeom {
    uint32_t bu;     // units per row
    uint32_t magic;  // ceil(2^32 / bu): v / bu == umulhi(v, magic) while v * bu < 2^32
    uint32_t log_r;  // a super-task is 1 << log_r rows ...
    uint32_t st;     // ... = st windows ...
    uint32_t uwe;    // ... of uwe <= UW units each (the lanes past uwe * lanes-per-unit idle); the last window of a
                     // super-task may be ragged (st * uwe > the super-task's units): its lanes past the end idle too
};

// The window width and the rows per super-task for a matrix of n rows (nm matrices walked side by side) on `waves` waves.
// Full windows (uwe = uw) waste no lane but tie R = uw / gcd(bu, uw) rows together, which leaves waves without work when
// n / R is small (k = 2816: 11 super-blocks per row, R = 16); narrower windows that divide R * bu for a smaller R (11 of 16
// units: one row per window) spread the rows over more waves at the price of idle lanes.  Chosen: the pair with the smallest
// sum of the windows on the busiest wave and the windows per wave on average.
inline FlatGeom flat_geom(uint32_t k, uint32_t unit_elems, uint32_t uw, uint32_t n, uint32_t nm, uint32_t waves) {
    FlatGeom g{};
    g.bu = k / unit_elems;
    g.magic = (uint32_t)((0x100000000ull + g.bu - 1) / g.bu);  // bu >= 2
    uint64_t best = ~0ull;
    for (uint32_t log_r = 0; (1u << log_r) <= uw; ++log_r) {
        const uint32_t r = 1u << log_r;
        uint32_t uwe = uw;
        while ((r * g.bu) % uwe) --uwe;
        // the widest window that divides the super-task, and full windows with a ragged last one (68 super-blocks per row:
        // windows of 16, 16, 16, 16 and 4 where the divisors offer 4 per row or 17 windows of 16 for four rows)
        for (int ragged = 0; ragged < 2; ++ragged) {
            if (ragged && uwe == uw) break;
            const uint32_t w = ragged ? uw : uwe;
            const uint32_t st = (r * g.bu + w - 1) / w;
            const uint64_t n_super = (n + r - 1) / r;
            const uint64_t crit = ((n_super + waves - 1) / waves) * nm * st, total = n_super * nm * st;
            // windows of the busiest wave + windows per wave on average: the first bounds the time when waves run short
            // of work, the second when the device is busy throughout (a ragged window's idle lanes cost their arithmetic)
            const uint64_t score = crit * waves + total;
            if (score < best) {
                best = score;
                g.log_r = log_r;
                g.st = st;
                g.uwe = w;
            }
        }
    }
    return g;
}

// ---- activations of one row in LDS: the values in the order the dot products read them + per-16 sums ----
// PAIR (bf16 activations; K-quants and Q4_0): pre-paired bf16 words, 16-byte chunks of 8 activations, for
// v_dot2c_f32_bf16.  Otherwise f32 values (f32 activations; bf16 ones widened for Q8_0), 16-byte chunks of 4.  A lane reads
// the chunks of its piece one after the other, sixteen lanes of a ds_read_b128 at a time: the pieces are padded apart
// (one chunk per piece; Q6_K, whose lane reads four runs of a super-block: 36 / 81 chunks per super-block with the
// halves 17 / 40 apart) so that those sixteen lanes hit sixteen different 16-byte bank groups and every chunk of a
// piece is an immediate offset from the lane's one base address.
template <int TYPE, bool X_BF16>
struct FlatX1 {
    static constexpr bool PAIR = X_BF16 && TYPE != HQ_Q8_0 && TYPE != HQ_Q8_0_X2;
    static constexpr int XW = PAIR ? (kBlock32<TYPE> ? 16 : 32) : (kBlock32<TYPE> ? 32 : 64);  // registers of one lane's activations
    static constexpr uint32_t CA = PAIR ? 8u : 4u;                                              // activations per chunk
    static constexpr uint32_t G = (kBlock32<TYPE> ? 32u : 64u) / CA;                             // chunks per piece

    // LDS slot of chunk ch
    static __host__ __device__ __forceinline__ uint32_t slot(uint32_t ch) {
        if constexpr (TYPE == HQ_Q6_K) {
            if constexpr (PAIR) return (ch >> 5) * 36u + ((ch >> 4) & 1u) * 17u + (ch & 15u);
            return (ch >> 6) * 81u + ((ch >> 5) & 1u) * 40u + (ch & 31u);
        } else {
            return ch + ch / G;
        }
    }
    static __host__ __device__ __forceinline__ size_t value_bytes(uint32_t k) { return (size_t)slot(k / CA) * 16; }
    static __host__ __device__ __forceinline__ size_t lds_bytes(uint32_t k) { return value_bytes(k) + (size_t)(k / 16) * 4; }

    // 16 activations per thread and pass; the sum of a run of sixteen adds them in index order.
    static __device__ __forceinline__ void stage(const void* x, uint32_t k, uint4* lds_x, float* lds_s, uint32_t tid,
                                                 uint32_t nthreads) {
        for (uint32_t i = tid; i < k / 16u; i += nthreads) {
            XRaw<X_BF16> raw;
            raw.fetch(x, i);
            float v[16];
            if constexpr (X_BF16) {
                const uint4 p = raw.r[0], q = raw.r[1];
                const uint32_t w[8] = {p.x, p.y, p.z, p.w, q.x, q.y, q.z, q.w};
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
                    lds_x[slot(2 * i)] = o0;
                    lds_x[slot(2 * i + 1)] = o1;
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
                    reinterpret_cast<float4*>(lds_x)[slot(4 * i + j)] = make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
            }
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < 16; ++j) s += v[j];
            lds_s[i] = s;
        }
    }

    // The activations of the lane's piece: unit `ur` of the row, sub-piece c (K-quants: the lane's quarter).
    static __device__ __forceinline__ void load(const uint4* lds_x, const float* lds_s, uint32_t ur, int c, uint32_t* xr,
                                                float* sx) {
        auto put = [&](int at, const uint4 v) {
            xr[at] = v.x;
            xr[at + 1] = v.y;
            xr[at + 2] = v.z;
            xr[at + 3] = v.w;
        };
        if constexpr (TYPE == HQ_Q6_K) {
            // four runs of 16 activations, 32 apart, in the half (c >> 1) of the super-block, starting at 16 * (c & 1)
            constexpr int CR = 16 / (int)CA;  // chunks per run
            const uint4* base = lds_x + (PAIR ? ur * 36u + (uint32_t)(c >> 1) * 17u : ur * 81u + (uint32_t)(c >> 1) * 40u) +
                                (uint32_t)(c & 1) * CR;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
#pragma unroll
                for (int u = 0; u < CR; ++u) put((CR * r + u) * 4, base[2 * CR * r + u]);
                sx[r] = lds_s[ur * 16u + (uint32_t)(c >> 1) * 8u + (uint32_t)(c & 1) + 2u * r];
            }
        } else {
            const uint32_t piece = kLaneUnit<TYPE> ? ur : ur * 4u + (uint32_t)c;
            const uint4* base = lds_x + piece * (G + 1u);
#pragma unroll
            for (int j = 0; j < (int)G; ++j) put(4 * j, base[j]);
            constexpr int RUNS = kBlock32<TYPE> ? 2 : 4;
#pragma unroll
            for (int r = 0; r < RUNS; ++r) sx[r] = lds_s[piece * RUNS + r];
        }
    }

    // f32 K-quant pieces in two halves of 32 activations (see dot_f32_half); h = 0 also loads the four run sums.
    static __device__ __forceinline__ void load_half(const uint4* lds_x, const float* lds_s, uint32_t ur, int c, int h, uint32_t* xh,
                                                     float* sx) {
        static_assert(!PAIR && !kBlock32<TYPE>, "f32 activations of a K-quant");
        auto put = [&](int at, const uint4 v) {
            xh[at] = v.x;
            xh[at + 1] = v.y;
            xh[at + 2] = v.z;
            xh[at + 3] = v.w;
        };
        if constexpr (TYPE == HQ_Q6_K) {
            const uint4* base = lds_x + ur * 81u + (uint32_t)(c >> 1) * 40u + (uint32_t)(c & 1) * 4u + 16u * (uint32_t)h;
#pragma unroll
            for (int r = 0; r < 2; ++r) {
#pragma unroll
                for (int u = 0; u < 4; ++u) put((4 * r + u) * 4, base[8 * r + u]);
            }
            if (h == 0) {
#pragma unroll
                for (int r = 0; r < 4; ++r) sx[r] = lds_s[ur * 16u + (uint32_t)(c >> 1) * 8u + (uint32_t)(c & 1) + 2u * r];
            }
        } else {
            const uint32_t piece = ur * 4u + (uint32_t)c;
            const uint4* base = lds_x + piece * (G + 1u) + 8u * (uint32_t)h;
#pragma unroll
            for (int j = 0; j < 8; ++j) put(4 * j, base[j]);
            if (h == 0) {
#pragma unroll
                for (int r = 0; r < 4; ++r) sx[r] = lds_s[piece * 4u + r];
            }
        }
    }
};

// Base types (and the Q8_0 block pair, which has a piece and a layout of its own): as above.  The other doubled types:
// the base type's layout, a lane's activations are those of unit 2 ur and of unit 2 ur + 1.
template <int TYPE, bool X_BF16, bool = (kIsX2<TYPE> && TYPE != HQ_Q8_0_X2)>
struct FlatX : FlatX1<TYPE, X_BF16> {};
template <int TYPE, bool X_BF16>
struct FlatX<TYPE, X_BF16, true> {
    using B = FlatX1<kBaseType<TYPE>, X_BF16>;
    static constexpr bool PAIR = B::PAIR;
    static constexpr int XW = 2 * B::XW;
    static constexpr int RUNS1 = kBlock32<kBaseType<TYPE>> ? 2 : 4;
    static constexpr uint32_t CA = B::CA, G = B::G;
    static __host__ __device__ __forceinline__ uint32_t slot(uint32_t ch) { return B::slot(ch); }
    static __host__ __device__ __forceinline__ size_t value_bytes(uint32_t k) { return B::value_bytes(k); }
    static __host__ __device__ __forceinline__ size_t lds_bytes(uint32_t k) { return B::lds_bytes(k); }
    static __device__ __forceinline__ void stage(const void* x, uint32_t k, uint4* lds_x, float* lds_s, uint32_t tid, uint32_t nthreads) {
        B::stage(x, k, lds_x, lds_s, tid, nthreads);
    }
    static __device__ __forceinline__ void load(const uint4* lds_x, const float* lds_s, uint32_t ur, int c, uint32_t* xr, float* sx) {
        B::load(lds_x, lds_s, 2u * ur, c, xr, sx);
        B::load(lds_x, lds_s, 2u * ur + 1u, c, xr + B::XW, sx + RUNS1);
    }
};

// XHALF: f32 activations of a K-quant are read from LDS 32 at a time (half the registers; the same sums).
// DYN (D == 1): the waves of a workgroup take the workgroup's super-tasks from a counter in LDS instead of a fixed split.
// The SIMD's issue arbitration favours its oldest wave, so with equal shares the youngest wave of every SIMD finishes long
// after the others; with the counter all waves of a CU end together.  A wave claims its next super-task one ahead, so its
// fetch runs on across the boundary.
// COPY (Q6_K, Q8_0 and Q4_0 block pairs, D == 1): a window is not fetched by the lanes that use it, five instructions touching
// each 128-byte line, but copied -- consecutive lanes consecutive 16-byte pieces, non-temporal loads, every line asked
// for once -- into 4-5 KB of LDS the wave owns, and the lanes read their pieces back from there (Q6_K blocks lie 210
// bytes apart: aligned words shifted into place by v_alignbyte; a Q8_0 block pair is seventeen aligned words, a Q4_0
// pair nine); the next
// window's copy is in flight meanwhile.  The same pieces, the same sums.  The host checks flat_copy_fits: every window
// starts at a multiple of 16 bytes and no copy reads past the matrix.
// (au: the units after which a window start is a multiple of 16 bytes again: 8 for Q6_K's 210 bytes, 4 for a Q8_0 block pair's 68)
inline bool flat_copy_fits(const FlatGeom& g, uint32_t uw, uint32_t n, uint32_t au, uintptr_t base0, uintptr_t base1) {
    return g.uwe == uw && ((g.bu << g.log_r) % au) == 0 && ((uint64_t)n * g.bu) % au == 0 && ((base0 | base1) & 15u) == 0;
}
template <int TYPE>
constexpr uint32_t kCopyAlignUnits = TYPE == HQ_Q6_K ? 8u : 4u;
template <int TYPE>
constexpr uint32_t kCopyNPV = (kUnitsPerWindow<TYPE> * kBlockBytes<TYPE> / 16u + 63u) / 64u;  // 16-byte pieces of a window per lane
template <int TYPE, bool X_BF16, int D = 1, bool XHALF = false, bool DYN = false, bool COPY = false>
struct FlatWalk {
    static_assert(!DYN || D == 1, "the dynamic split keeps one fetch in flight");
    static_assert(!COPY || ((TYPE == HQ_Q6_K || TYPE == HQ_Q8_0_X2 || TYPE == kX2 + HQ_Q4_0) && D == 1 && !XHALF), "Q6_K super-blocks or block pairs, one window in flight");
    static constexpr uint32_t NPV = COPY ? kCopyNPV<TYPE> : 1u, CAU = kCopyAlignUnits<TYPE>;
    using X = FlatX<TYPE, X_BF16>;
    static constexpr uint32_t LPU = kLanesPerUnit<TYPE>, UW = kUnitsPerWindow<TYPE>, BB = kBlockBytes<TYPE>;

    const uint8_t* w0;
    const uint8_t* w1;       // second matrix of the same shape (nm == 2), walked super-task by super-task beside the first
    uint32_t nrows, nm;
    FlatGeom g;
    // Super-task q of the sequence is seq_first + q * seq_stride, q < count.  Fixed split: the sequence is the wave's own and
    // it takes q = 0, 1, ...; dynamic: the sequence is the workgroup's and q comes from *queue (the first claims are the
    // wave indices: the kernel sets the counter to the number of waves before its first barrier).
    uint32_t seq_first, seq_stride, count;
    uint32_t* queue;
    uint32_t q_cur, q_nxt, q_nn;  // the super-task being summed, its successor and the one after (dynamic: claimed ahead)
    uint32_t lane, lv;  // lv: the lane's unit inside a window (idle lanes: the last active one's)
    bool active;
    int c;
    uint32_t m4, m2, magic;
    uint32_t f_q, f_m, f_w;  // the next task to fetch
    Piece<TYPE> buf[D];
    [[maybe_unused]] uint4 pv[NPV];  // COPY: the window in flight, 16-byte piece lane + 64 i of it
    [[maybe_unused]] uint4* wbuf;    // COPY: the wave's window buffer in LDS, 64 NPV slots of 16 bytes

    __device__ __forceinline__ void init(const uint8_t* wa, const uint8_t* wb, uint32_t n, uint32_t n_matrices, const FlatGeom& geom,
                                         uint32_t first_super, uint32_t super_stride, uint32_t* lds_queue = nullptr,
                                         uint32_t first_claim = 0, uint4* copy_buf = nullptr) {
        wbuf = copy_buf;
        w0 = wa;
        w1 = wb;
        nrows = n;
        nm = n_matrices;
        g = geom;
        lane = threadIdx.x & 63u;
        c = (int)(lane & 3u);
        active = lane / LPU < g.uwe;
        lv = active ? lane / LPU : g.uwe - 1u;
        const uint32_t n_super = (n + (1u << g.log_r) - 1u) >> g.log_r;
        seq_first = first_super;
        seq_stride = super_stride;
        count = first_super < n_super ? (n_super - first_super + super_stride - 1u) / super_stride : 0u;
        queue = lds_queue;
        q_cur = DYN ? first_claim : 0u;
        q_nxt = q_nn = q_cur + 1u;  // (dynamic: replaced by the first claims in prime())
        f_q = q_cur;
        f_m = f_w = 0;
    }

    // The conversion masks of the paired-bf16 dot products must sit in VGPRs (v_and_or_b32 takes one scalar operand at
    // most); the copy is opaque so they stay there.
    __device__ __forceinline__ void load_masks(uint32_t a_m4, uint32_t a_m2, uint32_t a_magic) {
        asm volatile("v_mov_b32 %0, %3\n\tv_mov_b32 %1, %4\n\tv_mov_b32 %2, %5"
                     : "=v"(m4), "=v"(m2), "=v"(magic)
                     : "s"(a_m4), "s"(a_m2), "s"(a_magic));
    }

    __device__ __forceinline__ void fetch_next(Piece<TYPE>& p) {
        const uint32_t sid = seq_first + f_q * seq_stride;
        // (a ragged last window: the lanes past the super-task's end fetch its last unit again)
        const uint32_t wu = g.uwe * f_w + lv, su = g.bu << g.log_r;
        uint32_t u = (sid << g.log_r) * g.bu + (wu < su ? wu : su - 1u);
        const uint32_t last = nrows * g.bu - 1u;
        u = u < last ? u : last;
        const uint8_t* base = f_m ? w1 : w0;
        if constexpr (COPY) {
            // the window's units [ub, ub + cnt): a multiple of CAU units from the matrix's start (whole 16-byte pieces),
            // clamped to the matrix (n * bu is a multiple of CAU); past a window that ends inside the matrix the last
            // piece reads up to 14 bytes of the next unit
            const uint32_t total = last + 1u;
            uint32_t ub = (sid << g.log_r) * g.bu + g.uwe * f_w;
            ub = ub < total ? ub : total - CAU;
            uint32_t cnt = su - g.uwe * f_w;
            cnt = cnt < g.uwe ? cnt : g.uwe;
            cnt = cnt < total - ub ? cnt : total - ub;
            const uint32_t last_piece = (cnt * BB + 15u) / 16u - 1u;
            const uint8_t* wb = base + (size_t)ub * BB;
#pragma unroll
            for (uint32_t i = 0; i < NPV; ++i) {
                const uint32_t pi = lane + 64u * i;
                pv[i] = ldnt16(wb + 16u * (pi < last_piece ? pi : last_piece));
            }
        } else {
            p.load(base + (size_t)u * BB, c);
        }
        // (scalar: no memory operation inside)  Past the sequence's end the last task is fetched again, not used.
        if (f_w + 1u < g.st) {
            ++f_w;
        } else if (f_m + 1u < nm) {
            f_w = 0;
            ++f_m;
        } else {
            // the fetch is one task ahead of the sums: it is in their super-task or in its successor
            const uint32_t nq = DYN ? (f_q == q_cur ? q_nxt : q_nn) : f_q + 1u;
            if (nq < count) {
                f_w = 0;
                f_m = 0;
                f_q = nq;
            }
        }
    }

    // (dynamic: call after the barrier behind which the counter is initialised)
    __device__ __forceinline__ void prime() {
        if constexpr (DYN) {
            q_nxt = claim_wait(claim());
            q_nn = claim_wait(claim());
        }
        if (q_cur < count) {
#pragma unroll
            for (int d = 0; d < D; ++d) fetch_next(buf[d]);
        }
    }

    __device__ __forceinline__ uint32_t claim() {
        uint32_t v = 0;
        if (lane == 0) v = __hip_atomic_fetch_add(queue, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return v;
    }
    __device__ __forceinline__ uint32_t claim_wait(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

    // out(count, keep0, keep1, row): lane l < count holds the sums of row `row` (its own value of the argument) over the first
    // (keep0) and the second matrix (keep1).
    template <typename OUT>
    __device__ __forceinline__ void run(const uint4* lds_x, const float* lds_s, OUT&& out) {
        uint32_t c_m = 0, c_w = 0, done = 0;
        float keep0 = 0.f, keep1 = 0.f;
        uint32_t keep_row = 0;
        constexpr bool HALVES = XHALF && !X::PAIR && !kLaneUnit<TYPE> && !kIsX2<TYPE>;
        uint32_t xr[HALVES ? 32 : X::XW];
        float sx[kIsX2<TYPE> ? 8 : 4] = {};
        // every window is one whole row (and not a ragged one): the lane's activations never change
        const bool xinv = !HALVES && g.st == 1u && g.log_r == 0u && g.uwe == g.bu;
        if constexpr (!HALVES)
            if (xinv) X::load(lds_x, lds_s, lv, c, xr, sx);
        const int last_lane = (int)(g.uwe * LPU - 1u);
        const bool one_row = g.log_r == 0u;
        float acc = 0.f;
        [[maybe_unused]] uint32_t pending = 0;
        if constexpr (DYN)
            if (q_cur < count) pending = claim();  // the third super-task from here
        // COPY: the lane's fields in the window buffer, block lv at byte 210 lv, at even offsets
        [[maybe_unused]] const uint32_t* wb32 = reinterpret_cast<const uint32_t*>(wbuf);
        [[maybe_unused]] const uint32_t cblk = lv * BB, ch = (uint32_t)c >> 1, clr = (uint32_t)c & 1u;
        [[maybe_unused]] const uint32_t o_qa = cblk + 64u * ch + 16u * clr, o_qh = cblk + 128u + 32u * ch + 16u * clr,
                                        o_sc = cblk + 192u + 8u * ch, o_d = cblk + 206u;
        [[maybe_unused]] auto field16 = [&](uint32_t o) -> uint4 {
            const uint32_t* q = wb32 + (o >> 2);
            const uint32_t sh = o & 3u, a0 = q[0], a1 = q[1], a2 = q[2], a3 = q[3], a4 = q[4];
            return make_uint4(__builtin_amdgcn_alignbyte(a1, a0, sh), __builtin_amdgcn_alignbyte(a2, a1, sh),
                              __builtin_amdgcn_alignbyte(a3, a2, sh), __builtin_amdgcn_alignbyte(a4, a3, sh));
        };
        while (q_cur < count) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                Piece<TYPE>& p = buf[d];
                if constexpr (COPY) {
                    // the window copied a task ago goes to LDS (behind the wave's reads of the previous one: a wave's LDS
                    // operations are served in order), the next window's copy is issued, this window's fields are read back
#pragma unroll
                    for (uint32_t i = 0; i < NPV; ++i) wbuf[lane + 64u * i] = pv[i];
                    asm volatile("" ::: "memory");
                    fetch_next(p);
                    if constexpr (TYPE == HQ_Q6_K) {
                        p.qa = field16(o_qa);
                        p.qb = field16(o_qa + 32u);
                        p.qh = field16(o_qh);
                        const uint32_t* q = wb32 + (o_sc >> 2);
                        const uint32_t sh = o_sc & 3u, a0 = q[0], a1 = q[1], a2 = q[2];
                        p.sc = make_uint2(__builtin_amdgcn_alignbyte(a1, a0, sh), __builtin_amdgcn_alignbyte(a2, a1, sh));
                        const uint32_t* qd = wb32 + (o_d >> 2);
                        p.d = __builtin_amdgcn_alignbyte(qd[1], qd[0], o_d & 3u);
                    } else if constexpr (TYPE == kX2 + HQ_Q4_0) {  // [d0][16 bytes][d1][16 bytes] as nine words at a multiple of four bytes
                        const uint32_t* q = wb32 + lv * (BB / 4u);
                        const uint32_t w0 = q[0], w1 = q[1], w2 = q[2], w3 = q[3], w4 = q[4];
                        p.a.d = w0 & 0xffffu;
                        p.a.q = make_uint4(__builtin_amdgcn_alignbyte(w1, w0, 2), __builtin_amdgcn_alignbyte(w2, w1, 2),
                                           __builtin_amdgcn_alignbyte(w3, w2, 2), __builtin_amdgcn_alignbyte(w4, w3, 2));
                        p.b.d = w4 >> 16;
                        p.b.q = make_uint4(q[5], q[6], q[7], q[8]);
                    } else {  // a block pair: seventeen words at a multiple of four bytes
                        const uint32_t* q = wb32 + lv * (BB / 4u);
                        p.a = make_uint4(q[0], q[1], q[2], q[3]);
                        p.b = make_uint4(q[4], q[5], q[6], q[7]);
                        p.c = make_uint4(q[8], q[9], q[10], q[11]);
                        p.e = make_uint4(q[12], q[13], q[14], q[15]);
                        p.t = q[16];
                    }
                }
                const uint32_t lu_raw = g.uwe * c_w + lv, su = g.bu << g.log_r;
                const bool in_task = lu_raw < su;  // false only in the idle part of a ragged last window
                const uint32_t lu = in_task ? lu_raw : su - 1u;
                uint32_t lrow = __umulhi(lu, g.magic);
                const uint32_t ur = lu - lrow * g.bu;
                float part;
                if constexpr (HALVES) {
                    float lo[2], hi[2];
                    X::load_half(lds_x, lds_s, ur, c, 0, xr, sx);
                    dot_f32_half(p, c, 0, reinterpret_cast<const float*>(xr), lo);
                    asm volatile("" : "+v"(lo[0]));  // the second half's activations take the first half's registers
                    X::load_half(lds_x, lds_s, ur, c, 1, xr, sx);
                    dot_f32_half(p, c, 1, reinterpret_cast<const float*>(xr), hi);
                    part = dot_f32_finish(p, c, lo, hi, sx);
                } else {
                    if (!xinv) X::load(lds_x, lds_s, ur, c, xr, sx);
                    if constexpr (X::PAIR)
                        part = dot_pair(p, c, xr, sx, m4, m2, magic);
                    else
                        part = dot_f32(p, c, reinterpret_cast<const float*>(xr), sx);
                }
                asm volatile("" : "+v"(part));  // the refill follows the arithmetic that frees its registers
                if constexpr (!COPY) fetch_next(p);
                const bool live = D == 1 || q_cur < count;  // (a ring's last round may run past the end)
                const uint32_t row0 = (seq_first + q_cur * seq_stride) << g.log_r;
                if (one_row) {
                    // every window of the super-task belongs to its one row: the lanes add their windows up and meet once
                    // (the order of sums of the aligned streaming kernel: the same bits)
                    acc += active && in_task && live ? part : 0.f;
                    if (live && c_w + 1u == g.st) {
                        const float v = group_sum(acc, 6);
                        acc = 0.f;
                        const bool mine = lane == (done & 63u);
                        keep0 = mine && c_m == 0u ? v : keep0;
                        keep1 = mine && c_m != 0u ? v : keep1;
                        keep_row = mine ? row0 : keep_row;
                    }
                } else {
                    const uint32_t r_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)lrow);
                    const uint32_t r_hi = (uint32_t)__builtin_amdgcn_readlane((int)lrow, last_lane);
                    lrow = active && in_task ? lrow : 0xffffffffu;  // an idle lane's duplicate belongs to no row
                    for (uint32_t r = r_lo; r <= r_hi; ++r) {
                        float v = lrow == r ? part : 0.f;
                        v = group_sum(v, 6);
                        const bool mine = live && lane == ((done + r) & 63u);
                        keep0 = mine && c_m == 0u ? keep0 + v : keep0;
                        keep1 = mine && c_m != 0u ? keep1 + v : keep1;
                        keep_row = mine ? row0 + r : keep_row;
                    }
                }
                if (live && ++c_w == g.st) {
                    c_w = 0;
                    if (++c_m == nm) {
                        c_m = 0;
                        done += 1u << g.log_r;
                        if ((done & 63u) == 0u) {
                            out(64u, keep0, keep1, keep_row);
                            keep0 = keep1 = 0.f;
                        }
                        if constexpr (DYN) {
                            q_cur = q_nxt;
                            q_nxt = q_nn;
                            q_nn = claim_wait(pending);
                            if (q_cur < count) pending = claim();
                        } else {
                            ++q_cur;
                        }
                    }
                }
            }
        }
        if (done & 63u) out(done & 63u, keep0, keep1, keep_row);
    }
};

}  // namespace
}  // namespace hq

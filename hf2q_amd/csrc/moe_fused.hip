// The MoE FFN block of a decode step (1..8 tokens) as ONE launch: router and shared-gate logits, softmax / top-k,
// gate and up projections of the routed and the shared expert with their SwiGLU, the down projections, and the
// weighted reduction (+ sigmoid-gated shared expert, + residual).  build_moe_ffn_layer_gpu_q_into
// (src/inference/models/qwen35/gpu_ffn.rs:2313-2802) encodes these as phases A-F of one command buffer;
// moe_ffn_cpu_ref (src/inference/models/qwen35/ffn.rs:179-336) is the specification.
//
// As separate launches the block costs four to five launch latencies in series (each small kernel spends 3-4 us
// before its first result whatever it computes).  Here one workgroup per CU walks the phases and hands results
// to the other workgroups through memory:
//   * every hand-over is a relaxed device-scope atomic store / load (write-through, cache-bypassing accesses) and no
//     fence is ever executed: a device-scope release fence writes a whole L2 back on this multi-XCD part;
//   * a consumer recognises fresh data by a TAG = (calls so far on this scratch) + 1: router logits and SwiGLU
//     activations travel as 64-bit (tag, value) words, so a value and its freshness arrive in one store, no store has
//     to be ordered behind another, and nothing has to be cleared between calls; workgroup 0 stores the new call count
//     when it leaves (every workgroup has read the old one by then: every workgroup delivers logits of every token,
//     so workgroup 0 cannot get past its token's routing before all of them have started);
//   * after the logits a workgroup works for one token (token b % T): it polls that token's logits only, routes it,
//     takes gate / up rows and down columns of that token;
//   * the down projections are cut by output columns, not by expert: a workgroup computes its 8 .. 64 columns for every
//     slot of a token and sums them itself, so the outputs never cross workgroups.
// No workgroup ever waits for a later phase of another one, so the grid drains whatever the residency; the waits are
// bounded all the same (spin_limit polls, then the error word of the scratch is set and the wave goes on).
//
// Row arithmetic is that of the separate dispatches — the same piece dot products, the same reduction order, the
// same SwiGLU rounding, the same order of the weighted sum — so the block's output has the bits of
// hq_dense_gemv_bf16_pair + hq_qmatmul_batch_ggml x 2 + hq_moe_weighted_reduce.
//
// Shapes: K-quant experts (Q4_K, Q5_K or Q6_K; gate / up of one type, down of the same or -- the mix GGUF files of the
// reference's model hold, docs/ADR-028...:4942-4946 -- Q4_K / Q5_K gate / up with a Q6_K down), hidden = 2048 (32 lanes
// per gate / up row: a wave step is one gate row and the up row of the same index), expert FFN = shared FFN = 512 (8
// lanes per down row), <= 256 experts, bf16 activations.
#include <math.h>

#include "hq_internal.h"
#include "moe_topk.h"

#include "gemv_pieces.h"

namespace hq {
namespace {

constexpr uint32_t FH = 2048, FI = 512;               // hidden, expert FFN width
template <int TYPE>
constexpr uint32_t kRowBytesH = FH / 256 * kBlockBytes<TYPE>;  // bytes of a gate / up row
template <int TYPE>
constexpr uint32_t kRowBytesI = FI / 256 * kBlockBytes<TYPE>;  // bytes of a down row
constexpr uint32_t MAX_T = 8;                         // tokens per call
// Two shapes of workgroup (template arguments WAVES_, RING_ of the kernel): 8 waves with four weight fetches in flight
// each -- one token: the phases are round trips, few rows per wave -- and 12 waves with two -- several tokens: the
// phases are bound by VALU issue, and three waves per SIMD keep it a little busier than two (16 waves leave 128
// registers per lane and spill 60 .. 200 of them).
// A logit is stored LG_COPIES times and a workgroup polls copy (its index among its token's workgroups) % LG_COPIES: at
// one token 256 workgroups would otherwise poll the same 2 KB (sixteen cache lines, a few memory channels).
constexpr uint32_t LG_COPIES = 8;

struct FusedArgs {
    const uint16_t* x;       // [T][H] bf16
    const uint16_t* router;  // [E][H] bf16
    const uint16_t* sh_lw;   // [H] bf16 or null: shared-expert gate logit
    const uint8_t *eg, *eu, *ed, *sg, *su, *sd;
    const float* residual;
    float* out;
    uint32_t* route_ids;
    float* route_w;
    uint8_t* scratch;
    uint32_t T, E, K;
    uint64_t stride_gu, stride_d;
    uint32_t m4, m2, magic, spin_limit;
};

// Scratch layout (byte offsets), the same on host and device: call counter and error word, then the two hand-over
// areas, both of (tag << 32 | value bits) words.
struct Layout {
    uint32_t T, E, K;
    __host__ __device__ uint32_t slots() const { return K + 1; }  // routed slots + the shared expert
    __host__ __device__ size_t logits() const { return 64; }  // u64 [LG_COPIES][T][E + 1]
    __host__ __device__ size_t act() const { return logits() + (size_t)LG_COPIES * T * (E + 1) * 8; }  // u64 [T][K + 1][I]
    __host__ __device__ size_t total() const { return act() + (size_t)T * slots() * FI * 8; }
};

template <typename V>
__device__ __forceinline__ void st_dev(V* p, V v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename V>
__device__ __forceinline__ V ld_dev(const V* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The value of a (tag, value) word once its tag is `tag`; polls at most `limit` times, then reports through *err.
__device__ __forceinline__ uint32_t wait_tagged(const uint64_t* p, uint32_t tag, uint32_t limit, uint32_t* err) {
    uint64_t got = ld_dev(p);
    for (uint32_t n = 0; (uint32_t)(got >> 32) != tag; ++n) {
        if (n >= limit) {
            st_dev(err, 1u);
            break;
        }
        __builtin_amdgcn_s_sleep(1);
        got = ld_dev(p);
    }
    return (uint32_t)got;
}

// LDS slot of 16-byte chunk ch of the staged activations.  Lanes that read together differ in the piece index (ch / 8)
// or, Q6_K, whose lane reads four runs of sixteen at a stride of 32 inside one half of a super-block, in bits 1, 4, 5, 6.
template <int TYPE>
__device__ __forceinline__ uint32_t swz8(uint32_t ch) {
    if constexpr (TYPE == HQ_Q6_K) return ch ^ (((ch >> 4) & 1u) | (((ch >> 5) & 3u) << 2));
    return ch ^ ((ch >> 4) & 7u);
}
// First float4 of run r (sixteen activations) of a lane's 64 activations of a row of FI: lane li = (super-block, quarter).
template <int TYPE>
__device__ __forceinline__ uint32_t act_run(uint32_t li, uint32_t r) {
    if constexpr (TYPE == HQ_Q6_K) return (li >> 2) * 64u + ((li >> 1) & 1u) * 32u + (li & 1u) * 4u + 8u * r;
    return li * 16u + 4u * r;
}

template <int TG, int TD, int WAVES_, int RING_>  // types of gate / up and of down; waves per workgroup; fetches in flight per wave
__global__ __launch_bounds__(64 * WAVES_) void moe_fused_kernel(FusedArgs a) {
    constexpr uint32_t WAVES = WAVES_, THREADS = 64 * WAVES;
    constexpr int RING = RING_;
    // activation loads of a thread per polling pass: (8 + 1) slots x 512 / 2 words = 4.5 per thread of 512, 2.25 of 1024
    constexpr int POLL = WAVES_ == 8 ? 5 : 3;
    constexpr uint32_t ROWB_H = kRowBytesH<TG>, ROWB_I = kRowBytesI<TD>;
    extern __shared__ uint4 smem[];
    const Layout L{a.T, a.E, a.K};
    const uint32_t T = a.T, E = a.E, K = a.K, S = K + 1;
    // After phase 1 a workgroup works for ONE token, token b % T: it needs that token's logits, activations and routing
    // only (eight tokens: an eighth of the words to poll for).
    // LDS: [the token's staged activations | later: its SwiGLU activations of all slots] | logits | ids | weights | partials
    uint4* lds_x = smem;                                                       // H/8 chunks (paired bf16 words)
    float* lds_sx = reinterpret_cast<float*>(lds_x + FH / 8);                  // H/16 per-16 sums
    const uint32_t area = (FH / 8) * 16 + (FH / 16) * 4, act_bytes = S * (FI * 4 + FI / 16 * 4);
    uint8_t* after = reinterpret_cast<uint8_t*>(smem) + (area > act_bytes ? area : act_bytes);
    float4* lds_act = reinterpret_cast<float4*>(smem);                         // S * I floats (over the activations, after phase 2)
    float* lds_as = reinterpret_cast<float*>(lds_act + (size_t)S * (FI / 4));  // S * I/16 sums
    float* lds_lg = reinterpret_cast<float*>(after);                           // E + 1
    uint32_t* lds_id = reinterpret_cast<uint32_t*>(lds_lg + (E + 1));          // K
    float* lds_w = reinterpret_cast<float*>(lds_id + K);                       // K + 1: slot K = shared gate
    float* lds_part = lds_w + S;                                               // S * 64 down partials of one unit
    uint32_t* lds_gath = reinterpret_cast<uint32_t*>(lds_part + S * 64);       // 64 * WAVES: the workgroup's SwiGLU activations

    const uint32_t tid = threadIdx.x, lane = tid & 63u, b = blockIdx.x, G = gridDim.x;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));  // known to be the same in a wave: scalar branches
    const uint32_t tok = b % T, jb = b / T, nb = (G - tok + T - 1u) / T;  // the token, this workgroup among its nb workgroups
    const uint32_t tw = jb * WAVES + wv, NTW = nb * WAVES;               // this wave among the token's waves
    uint32_t* s_epoch = reinterpret_cast<uint32_t*>(a.scratch);
    uint32_t* s_err = s_epoch + 1;
    uint64_t* s_lg = reinterpret_cast<uint64_t*>(a.scratch + L.logits());
    uint64_t* s_act = reinterpret_cast<uint64_t*>(a.scratch + L.act());

    const uint32_t tag = ld_dev(s_epoch) + 1u;
    const uint64_t tag_hi = (uint64_t)tag << 32;

    // the activations of all tokens, requested first and staged while the logits travel (the layout and sums of
    // stage_store); 16 activations per thread and pass
    static_assert(FH / 16 <= THREADS, "one pass stages a token");
    XRaw<true> xraw;
    xraw.fetch(a.x + (size_t)tok * FH, tid < FH / 16 ? tid : 0u);  // (no branch around the load)

    // ---- phase 1: router logits and the shared-gate logit, one (row, token) per wave and turn, with the arithmetic of
    // dense_gemv_bf16_kernel. ----
    const uint32_t n_rows = E + (a.sh_lw ? 1u : 0u);
    // Workgroup b takes the rows b, b + G, ... for every token (G <= n_rows: it has at least one row), its waves the
    // (row, token) pairs in turn.  Every workgroup so delivers logits of EVERY token, which matters for the call
    // counter: a workgroup cannot get past its token's routing before all workgroups have started and read it.
    const uint32_t rows_mine = (n_rows - b + G - 1u) / G;
    for (uint32_t q = wv; q < rows_mine * T; q += WAVES) {
        const uint32_t r = b + G * (q / T), t = q % T;
        const uint4* wr = reinterpret_cast<const uint4*>(r < E ? a.router + (size_t)r * FH : a.sh_lw);
        const uint4* xr = reinterpret_cast<const uint4*>(a.x + (size_t)t * FH);
        uint4 wq[FH / 8 / 64], xq[FH / 8 / 64];
#pragma unroll
        for (uint32_t c = 0; c < FH / 8 / 64; ++c) {
            wq[c] = wr[lane + 64 * c];
            xq[c] = xr[lane + 64 * c];
        }
        float acc = 0.f;
#pragma unroll
        for (uint32_t c = 0; c < FH / 8 / 64; ++c) {
            const uint32_t ww[4] = {wq[c].x, wq[c].y, wq[c].z, wq[c].w}, tw[4] = {xq[c].x, xq[c].y, xq[c].z, xq[c].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc = fmaf(bf16_bits_to_f32(ww[i] & 0xffffu), bf16_bits_to_f32(tw[i] & 0xffffu), acc);
                acc = fmaf(bf16_bits_to_f32(ww[i] >> 16), bf16_bits_to_f32(tw[i] >> 16), acc);
            }
        }
        acc = wave_sum(acc);
        if (lane < LG_COPIES) st_dev(&s_lg[((size_t)lane * T + t) * (E + 1) + r], tag_hi | __float_as_uint(acc));
    }

    // ---- while the logits travel: the staged activations go to LDS ----
    if (tid < FH / 16) {
        const uint32_t j = tid;
        const uint4 p = xraw.r[0], q = xraw.r[1];
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
        lds_x[swz8<TG>(2 * j)] = o0;
        lds_x[swz8<TG>(2 * j + 1)] = o1;
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            sum += bf16_bits_to_f32(w[e] & 0xffffu);
            sum += bf16_bits_to_f32(w[e] >> 16);
        }
        lds_sx[j] = sum;
    }

    // ---- the token's logits, then its routing (every workgroup of the token for itself, one wave) ----
    for (uint32_t i = tid; i < E + 1; i += THREADS)
        lds_lg[i] = i < n_rows ? __uint_as_float(wait_tagged(&s_lg[((size_t)(jb % LG_COPIES) * T + tok) * (E + 1) + i], tag, a.spin_limit, s_err)) : 0.f;
    __syncthreads();
    if (wv == 0) {
        uint32_t id;
        float wt;
        softmax_topk_lane<4>(lds_lg, E, K, lane, id, wt);
        if (lane < K) {
            id = id < E ? id : E - 1u;  // (the selection only yields indices below E; a bound the fetch addresses can rely on)
            lds_id[lane] = id;
            lds_w[lane] = wt;
            if (jb == 0 && a.route_ids) {
                a.route_ids[tok * K + lane] = id;
                a.route_w[tok * K + lane] = wt;
            }
        }
        if (lane == 0) lds_w[K] = a.sh_lw ? 1.f / (1.f + expf(-lds_lg[E])) : 1.f;  // ffn.rs:28-30
    }
    __syncthreads();

    uint32_t m4, m2, magic;
    asm volatile("v_mov_b32 %0, %3\n\tv_mov_b32 %1, %4\n\tv_mov_b32 %2, %5"
                 : "=v"(m4), "=v"(m2), "=v"(magic)
                 : "s"(a.m4), "s"(a.m2), "s"(a.magic));

    // ---- phase 2: gate and up row p % I of slot p / I of the token, lanes 0-31 the gate row and 32-63 the up row, then
    // the SwiGLU; the waves of the token's workgroups take the rows in turn, RING fetches ahead ----
    // The activations are not stored where they arise.  Loads and stores are counted by one counter and return in order,
    // and a write-through store is acknowledged by memory a microsecond or more after its issue (several under load): a
    // store among the fetches holds back every fetch behind it.  Lane n keeps the activation of the wave's row n; after
    // the phase the waves put theirs together in LDS and ONE wave stores the workgroup's rows (eight consecutive words
    // per row index: 64-byte pieces instead of 8-byte ones), after the next phase's first weight fetches have been issued.
    // (A wave with more than 64 rows, which takes a small grid and many slots, stores for itself.)
    uint32_t keep = 0;
    const uint32_t P = S * FI;
    const uint32_t rows2 = tw < P ? (P - tw + NTW - 1u) / NTW : 0u;
    const uint32_t rows2_wg = jb * WAVES < P ? (P - jb * WAVES + NTW - 1u) / NTW : 0u;  // of the workgroup's first wave: the most
    const bool gather = rows2_wg <= 64u;
    auto flush = [&](uint32_t first, uint32_t count) {
        if (lane < count) st_dev(&s_act[(size_t)tok * P + tw + (first + lane) * NTW], tag_hi | keep);
    };
    {
        const uint32_t li = lane & 31u, hf = lane >> 5;
        const int c4 = (int)(li & 3u);
        const uint32_t mine = rows2;
        const uint32_t lane_off = (li >> 2) * kBlockBytes<TG>;
        auto fetch = [&](Piece<TG>& pc, uint32_t p) {
            const uint32_t r = p % FI, s = p / FI;
            const uint8_t* base = s < K ? (hf ? a.eu : a.eg) + (size_t)lds_id[s] * a.stride_gu : (hf ? a.su : a.sg);
            pc.load(base + (size_t)r * ROWB_H + lane_off, c4);
        };
        Piece<TG> ring[RING];
#pragma unroll
        for (int i = 0; i < RING; ++i)
            if ((uint32_t)i < mine) fetch(ring[i], tw + (uint32_t)i * NTW);
        uint32_t xp[32];
        float sx[4];
        {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t ch = act_run<TG>(li, (uint32_t)r) / 2u;  // two chunks of eight per run
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const uint4 v = lds_x[swz8<TG>(ch + u)];
                    xp[8 * r + 4 * u] = v.x;
                    xp[8 * r + 4 * u + 1] = v.y;
                    xp[8 * r + 4 * u + 2] = v.z;
                    xp[8 * r + 4 * u + 3] = v.w;
                }
                sx[r] = lds_sx[ch / 2];
            }
        }
        float keep_g = 0.f, keep_u = 0.f;
        for (uint32_t i0 = 0; i0 < mine; i0 += RING) {
#pragma unroll
            for (int i = 0; i < RING; ++i) {
                const uint32_t n = i0 + (uint32_t)i;
                if (n < mine) {
                    const uint32_t p = tw + n * NTW;
                    const float v = group_sum(dot_pair(ring[i], c4, xp, sx, m4, m2, magic), 5);
                    const float gate = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
                    const float up = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
                    if (n + RING < mine) {
                        float tie = v;
                        asm volatile("" : "+v"(tie));
                        fetch(ring[i], p + RING * NTW);
                    }
                    keep_g = lane == (n & 63u) ? gate : keep_g;  // the SwiGLU of up to 64 rows is one pass at the end
                    keep_u = lane == (n & 63u) ? up : keep_u;
                    if ((n & 63u) == 63u && n + 1u < mine) {
                        keep = __float_as_uint(silu_mul_f32(keep_g, keep_u));
                        flush(n - 63u, 64u);
                    }
                }
            }
        }
        keep = __float_as_uint(silu_mul_f32(keep_g, keep_u));
    }
    if (gather && lane < rows2) lds_gath[lane * WAVES + wv] = keep;
    // The workgroup's activations go out by its last wave (or by every wave for itself), which then waits for the stores'
    // acknowledgement while the other waves issue the next phase's first weight fetches; nobody polls before that: the
    // other workgroups' stores were issued at about the same time, so the first poll finds nearly everything, and polls
    // that start earlier only get in the way of the stores.
    const bool storing = !gather || wv == WAVES - 1u;
    auto store_acts = [&]() {
        if (gather) {
            if (storing)
                for (uint32_t idx = lane; idx < rows2_wg * WAVES; idx += 64u) {
                    const uint32_t p = jb * WAVES + idx % WAVES + idx / WAVES * NTW;
                    if (p < P) st_dev(&s_act[(size_t)tok * P + p], tag_hi | lds_gath[idx]);
                }
        } else if (rows2) {
            flush((rows2 - 1u) & ~63u, ((rows2 - 1u) & 63u) + 1u);
        }
    };
    auto await_acts_stored = [&]() {
        if (storing) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (gather) __syncthreads();
    };
    // Every fetch of the phase has been consumed: a wait that costs nothing and tells the compiler so (it cannot see it
    // from the loop's conditions), or it would make the next phase's fetches wait for each other for the sake of the
    // registers they share with these.
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    __syncthreads();  // the staged activations are dead from here on: their LDS holds the SwiGLU activations next

    // ---- phases 3 + 4: unit (token t, column slice c): the down rows of the slice for every slot of the token, then
    // the weighted sum over the slots in slot order, the shared expert last (the order of moe_weighted_reduce_kernel) ----
    {
        constexpr int RD = TD == HQ_Q5_K && RING > 3 ? 3 : RING;  // (a ring of four Q5_K pieces beside the 64 activations spills)
        const uint32_t li = lane & 7u, sub = lane >> 3;
        const int c4 = (int)(li & 3u);
        const uint32_t groups = T <= 1 ? 1u : T <= 2 ? 2u : T <= 4 ? 4u : 8u, cols = 8u * groups;  // columns per unit: about one unit per workgroup
        const uint32_t units_per_t = FH / cols, t = tok;
        store_acts();
        if (jb >= units_per_t) await_acts_stored();  // a workgroup without a unit
        for (uint32_t c = jb; c < units_per_t; c += nb) {
            // steps (slot s, row group g) = step index s * groups + g.  With several row groups a wave takes a run of
            // consecutive steps, so that it changes slot (and reloads the slot's activations from LDS) as seldom as
            // possible; with one row group (one token) every step is another slot and the waves take the steps in turn.
            const uint32_t n_steps = S * groups;
            const bool runs = groups > 1;
            const uint32_t st0 = runs ? wv * n_steps / WAVES : wv, stp = runs ? 1u : WAVES;
            const uint32_t mine = runs ? (wv + 1u) * n_steps / WAVES - st0 : wv < n_steps ? (n_steps - wv + WAVES - 1u) / WAVES : 0u;
            auto fetch = [&](Piece<TD>& pc, uint32_t n) {
                const uint32_t st = st0 + n * stp, s = st / groups, g = st % groups;
                const uint8_t* base = s < K ? a.ed + (size_t)lds_id[s] * a.stride_d : a.sd;
                pc.load(base + (size_t)(cols * c + 8 * g + sub) * ROWB_I + (li >> 2) * kBlockBytes<TD>, c4);
            };
            Piece<TD> ring[RD];
            auto prefetch = [&]() {
#pragma unroll
                for (int i = 0; i < RD; ++i)
                    if ((uint32_t)i < mine) fetch(ring[i], (uint32_t)i);
            };
            if (c == jb && storing) {  // (a storing wave's fetches would stand in the queue in front of the acknowledgement's wait)
                await_acts_stored();
                prefetch();
            } else {
                prefetch();
                if (c == jb) await_acts_stored();
            }
            // the token's SwiGLU activations of every slot: (tag, value) words, two per 16-byte load, all of a thread's
            // loads of a pass in flight at once; a load whose words are not both fresh is asked for again
            {
                typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                const uint64_t* src = s_act + (size_t)(t * S) * FI;
                const uint32_t n2 = S * FI / 2;
                for (uint32_t base = 0; base < n2; base += POLL * THREADS) {
                    u32x4 got[POLL];
                    uint32_t off[POLL];
#pragma unroll
                    for (int i = 0; i < POLL; ++i) {
                        const uint32_t e2 = base + tid + (uint32_t)i * THREADS;
                        off[i] = 16u * (e2 < n2 ? e2 : tid);  // past the end: a word of the thread's own, not used
                        asm volatile("global_load_dwordx4 %0, %1, %2 sc0 sc1" : "=v"(got[i]) : "v"(off[i]), "s"(src) : "memory");
                    }
                    for (uint32_t tries = 0;; ++tries) {
                        // the results exist once the counter has drained; naming them keeps their uses below the wait
                        if constexpr (POLL == 5)
                            asm volatile("s_waitcnt vmcnt(0)" : "+v"(got[0]), "+v"(got[1]), "+v"(got[2]), "+v"(got[3]), "+v"(got[4]) : : "memory");
                        else
                            asm volatile("s_waitcnt vmcnt(0)" : "+v"(got[0]), "+v"(got[1]), "+v"(got[2]) : : "memory");
                        bool fresh = true;
#pragma unroll
                        for (int i = 0; i < POLL; ++i) {
                            if (got[i].y != tag || got[i].w != tag) {
                                fresh = false;
                                asm volatile("global_load_dwordx4 %0, %1, %2 sc0 sc1" : "+v"(got[i]) : "v"(off[i]), "s"(src) : "memory");
                            }
                        }
                        if (fresh) break;
                        if (tries >= a.spin_limit) {
                            st_dev(s_err, 2u);
                            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                            break;
                        }
                    }
#pragma unroll
                    for (int i = 0; i < POLL; ++i) {
                        const uint32_t e2 = base + tid + (uint32_t)i * THREADS;
                        if (e2 < n2) {
                            const uint32_t e = 2 * e2, sl = e / FI, k = e % FI, q = k >> 2;  // piece p = q / 16 reads float4 slot q ^ p
                            float* dst = reinterpret_cast<float*>(lds_act) + sl * FI + (((q ^ (q >> 4)) << 2) | (k & 3u));
                            dst[0] = __uint_as_float(got[i].x);
                            dst[1] = __uint_as_float(got[i].z);
                        }
                    }
                }
            }
            __syncthreads();
            for (uint32_t e = tid; e < S * (FI / 16); e += THREADS) {  // per-16 sums in the order one thread adds them (stage_swiglu)
                const uint32_t s = e / (FI / 16), j = e % (FI / 16);
                float sum = 0.f;
#pragma unroll
                for (uint32_t k = 0; k < 16; ++k) {
                    const uint32_t q = (j * 16 + k) >> 2;
                    sum += reinterpret_cast<float*>(lds_act)[s * FI + (((q ^ (q >> 4)) << 2) | (k & 3u))];
                }
                lds_as[e] = sum;
            }
            __syncthreads();
            float xf[64], sx[4];
            uint32_t cur_s = ~0u;
            for (uint32_t i0 = 0; i0 < mine; i0 += RD) {
#pragma unroll
                for (int i = 0; i < RD; ++i) {
                    const uint32_t n = i0 + (uint32_t)i;
                    if (n < mine) {
                        const uint32_t st = st0 + n * stp, s = st / groups, g = st % groups;
                        if (s != cur_s) {  // uniform
                            cur_s = s;
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                const uint32_t f0 = act_run<TD>(li, (uint32_t)r);
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    const uint32_t f = f0 + (uint32_t)j;
                                    const float4 v = lds_act[s * (FI / 4) + (f ^ (f >> 4))];
                                    xf[16 * r + 4 * j] = v.x;
                                    xf[16 * r + 4 * j + 1] = v.y;
                                    xf[16 * r + 4 * j + 2] = v.z;
                                    xf[16 * r + 4 * j + 3] = v.w;
                                }
                                sx[r] = lds_as[s * (FI / 16) + f0 / 4];
                            }
                        }
                        const float v = group_sum(dot_f32(ring[i], c4, xf, sx), 3);
                        if (n + RD < mine) {
                            float tie = v;
                            asm volatile("" : "+v"(tie));
                            fetch(ring[i], n + RD);
                        }
                        if (li == 0) lds_part[s * cols + 8 * g + sub] = v;
                    }
                }
            }
            // (every fetch has been consumed: a free wait that tells the compiler so, or it would make the next unit's first
            // fetches wait for the output store below)
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
            __syncthreads();
            if (tid < cols) {
                const uint32_t col = cols * c + tid;
                float acc = 0.f;
                for (uint32_t s = 0; s < S; ++s) acc = fmaf(lds_w[s], lds_part[s * cols + tid], acc);
                if (a.residual) acc += a.residual[(size_t)t * FH + col];
                a.out[(size_t)t * FH + col] = acc;
            }
            __syncthreads();  // lds_act / lds_part are rewritten by the next unit
        }
    }
    if (b == 0 && tid == 0) st_dev(s_epoch, tag);
}

}  // namespace

size_t moe_fused_scratch_bytes(uint32_t n_tokens, uint32_t n_experts, uint32_t top_k) {
    return (Layout{n_tokens, n_experts, top_k}.total() + 255) & ~(size_t)255;
}

namespace {
// The kernel instantiated for (gate / up type, down type), or null: one K-quant for all three, or Q4_K / Q5_K gate / up
// with a Q6_K down.
template <int W, int R>
void (*fused_kernel_of(hq_ggml_type t, hq_ggml_type td))(FusedArgs) {
    if (t == HQ_Q4_K && td == HQ_Q4_K) return moe_fused_kernel<HQ_Q4_K, HQ_Q4_K, W, R>;
    if (t == HQ_Q5_K && td == HQ_Q5_K) return moe_fused_kernel<HQ_Q5_K, HQ_Q5_K, W, R>;
    if (t == HQ_Q6_K && td == HQ_Q6_K) return moe_fused_kernel<HQ_Q6_K, HQ_Q6_K, W, R>;
    if (t == HQ_Q4_K && td == HQ_Q6_K) return moe_fused_kernel<HQ_Q4_K, HQ_Q6_K, W, R>;
    if (t == HQ_Q5_K && td == HQ_Q6_K) return moe_fused_kernel<HQ_Q5_K, HQ_Q6_K, W, R>;
    return nullptr;
}
// wide: the 12-wave form
void (*fused_kernel_for(hq_ggml_type t, hq_ggml_type td, bool wide = false))(FusedArgs) {
    return wide ? fused_kernel_of<12, 2>(t, td) : fused_kernel_of<8, 4>(t, td);
}
}  // namespace

bool moe_fused_supported(uint32_t n_tokens, uint32_t hidden, uint32_t n_experts, uint32_t top_k, uint32_t inter,
                         uint32_t shared_inter, hq_ggml_type t, hq_ggml_type t_down, hq_act_dtype xdt) {
    return fused_kernel_for(t, t_down) != nullptr && xdt == HQ_BF16 && hidden == FH && inter == FI && shared_inter == FI && n_tokens >= 1 &&
           n_tokens <= MAX_T && n_experts >= n_tokens && n_experts <= 256 && top_k >= 1 && top_k <= 64 && top_k <= n_experts;
}

int launch_moe_fused(hipStream_t s, const MoeFusedArgs& m) {
    FusedArgs a{};
    a.x = static_cast<const uint16_t*>(m.x);
    a.router = static_cast<const uint16_t*>(m.router);
    a.sh_lw = static_cast<const uint16_t*>(m.shared_gate_logit);
    a.eg = static_cast<const uint8_t*>(m.expert_gate);
    a.eu = static_cast<const uint8_t*>(m.expert_up);
    a.ed = static_cast<const uint8_t*>(m.expert_down);
    a.sg = static_cast<const uint8_t*>(m.shared_gate);
    a.su = static_cast<const uint8_t*>(m.shared_up);
    a.sd = static_cast<const uint8_t*>(m.shared_down);
    a.residual = m.residual;
    a.out = m.out;
    a.route_ids = m.route_ids;
    a.route_w = m.route_weights;
    a.scratch = static_cast<uint8_t*>(m.scratch);
    a.T = m.n_tokens;
    a.E = m.n_experts;
    a.K = m.top_k;
    a.stride_gu = m.stride_gate_up;
    a.stride_d = m.stride_down;
    a.m4 = m.t_gate_up == HQ_Q6_K ? N4 : M4;
    a.m2 = m.t_gate_up == HQ_Q5_K ? M1 : m.t_gate_up == HQ_Q6_K ? N2 : M2;
    a.magic = MAGIC;
    a.spin_limit = m.spin_limit ? m.spin_limit : (1u << 20);
    // from two tokens on the 12-wave form (17.8 / 22.5 / 34.3 us at 2 / 4 / 8 tokens against 19.0 / 24.2 / 34.8; one token: the same)
    const bool wide = m.n_tokens >= 2u;
    const uint32_t WAVES = wide ? 12u : 8u, THREADS = 64u * WAVES;
    auto kern = fused_kernel_for(m.t_gate_up, m.t_down, wide);
    if (!kern) return fail(HQ_ERR_UNSUPPORTED, "fused MoE block: gate / up type %d with down type %d", (int)m.t_gate_up, (int)m.t_down);
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    // every workgroup must deliver at least one logit row (see the header comment), and one workgroup per CU
    const uint32_t rows = m.n_experts + (m.shared_gate_logit ? 1u : 0u);
    const uint32_t grid = cus < rows ? cus : rows;
    if (grid < m.n_tokens)  // after the logits a workgroup works for one token: every token needs a workgroup
        return fail(HQ_ERR_UNSUPPORTED, "fused MoE block: %u tokens over %u router rows", m.n_tokens, rows);
    const uint32_t S = m.top_k + 1;
    const size_t area = (size_t)(FH / 8) * 16 + (size_t)(FH / 16) * 4, act_bytes = (size_t)S * (FI * 4 + FI / 16 * 4);
    const size_t lds = (area > act_bytes ? area : act_bytes) + (size_t)(m.n_experts + 1) * 4 + (size_t)m.top_k * 4 + (size_t)S * 4 +
                       (size_t)S * 64 * 4 + (size_t)64 * WAVES * 4;
    if (lds > 64 * 1024) return fail(HQ_ERR_UNSUPPORTED, "fused MoE block: %zu bytes of LDS", lds);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(THREADS), lds, s, a);
    return check_launch("fused MoE block launch");
}

}  // namespace hq

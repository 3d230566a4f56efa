// The dense SwiGLU FFN of one decode token as ONE launch:  out = W_down . (silu(W_gate . x) * (W_up . x)) (+ residual).
//
// Three dequant-fused GEMVs of 28 MB each (hidden 4096, inter 12288, Q4_K) cost a launch and a memory round trip apiece
// when they are dispatched one by one; here one grid of one workgroup (16 waves) per CU streams all three matrices:
//   phase 1  every wave walks its rows of W_gate and the same rows of W_up (gemv_walk.h, the two-matrix walk of the
//            batched gate + up launch), forms silu(g) * u for them and stores the activations as (call number << 32 |
//            float bits) words into the scratch;
//   between  it requests the first windows of its W_down rows -- they depend on nothing, so the memory pipe keeps
//            streaming while the activations travel -- then collects all `inter` activations (16-byte cache-bypassing
//            loads, asked for again until both words carry this call's number) into LDS with their per-16 sums;
//   phase 2  it walks its rows of W_down over those f32 activations and stores the outputs.
// A word either carries this call's number or it is stale: nothing is cleared between calls and no fence is executed (a
// device-scope release fence writes the whole L2 back on this part).  The call number lives in the scratch (zeroed once by
// the caller; workgroup 0 stores the new number at its end, which it cannot reach before every workgroup has delivered
// activations, i.e. has read the old one).  Waits are bounded: after spin_limit polls the scratch's error word is set and
// the wave goes on, so every wave exits whatever happens.
//
// Every product runs the code of the separate kernels in the same order, so the result has the bits of
// hq_qmatmul_batch_ggml(gate, up) + hq_silu_mul + hq_qmatmul_ggml(down, f32 activations).
#include "hq_internal.h"
#include "gemv_pieces.h"
#include "gemv_walk.h"

namespace hq {
namespace {

constexpr int WAVES = 16, THREADS = 64 * WAVES;
constexpr int POLL = 4;  // activation loads a thread keeps in flight per polling pass

// Windows of W_down a wave requests before it waits for the activations.  One: every window more that is asked for while
// other waves still walk their gate / up rows stands in the memory queue in front of those rows (three windows per wave
// are the whole 28 MB matrix: the last gate / up row then ends 3 us later, 14.5 -> 17.5 us into the kernel, and the block
// 1.5 us later); the rest of the matrix streams while the VALU-bound second phase computes.
template <int TYPE>
constexpr int kDownRing = 1;

struct DArgs {
    const void* x;
    const uint8_t *wg, *wu, *wd;
    const float* residual;
    float* out;
    uint8_t* scratch;
    uint32_t hidden, inter;
    FlatGeom ggu, gdn;
    uint32_t m4, m2, magic, spin_limit;
};

// scratch: call number (u32), error word (u32), padding | u64 done[kMaxGrid]: a mark per workgroup | u64 act[inter]
constexpr uint32_t kMaxGrid = 512;
constexpr size_t kDoneOffset = 256, kActOffset = kDoneOffset + (size_t)kMaxGrid * 8;

template <typename V>
__device__ __forceinline__ void st_dev(V* p, V v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename V>
__device__ __forceinline__ V ld_dev(const V* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int TGU, int TDN, bool X_BF16>
__global__ __launch_bounds__(THREADS) void dense_ffn_kernel(DArgs a) {
    using X1 = FlatX<TGU, X_BF16>;
    using X2 = FlatX<TDN, false>;
    extern __shared__ uint4 smem[];
    uint4* lds_x1 = smem;
    float* lds_s1 = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(smem) + X1::value_bytes(a.hidden));
    uint8_t* area2 = reinterpret_cast<uint8_t*>(smem) + ((X1::lds_bytes(a.hidden) + 15u) & ~(size_t)15);
    uint4* lds_x2 = reinterpret_cast<uint4*>(area2);
    float* lds_s2 = reinterpret_cast<float*>(area2 + X2::value_bytes(a.inter));

    const uint32_t tid = threadIdx.x, lane = tid & 63u, b = blockIdx.x, G = gridDim.x;
    const uint32_t wv = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    uint32_t* s_epoch = reinterpret_cast<uint32_t*>(a.scratch);
    uint32_t* s_err = s_epoch + 1;
    uint64_t* s_done = reinterpret_cast<uint64_t*>(a.scratch + kDoneOffset);
    uint64_t* s_act = reinterpret_cast<uint64_t*>(a.scratch + kActOffset);
    __shared__ uint32_t lds_out;  // waves of this workgroup that are through phase 1
    if (tid == 0) lds_out = 0;
    const uint32_t tag = ld_dev(s_epoch) + 1u;
    const uint64_t tag_hi = (uint64_t)tag << 32;

    // ---- phase 1: gate and up rows, SwiGLU, activations out ----
    X1::stage(a.x, a.hidden, lds_x1, lds_s1, tid, THREADS);
    FlatWalk<TGU, X_BF16, 1> w1;
    w1.init(a.wg, a.wu, a.inter, 2, a.ggu, wv * G + b, WAVES * G);
    w1.prime();
    __syncthreads();
    w1.load_masks(a.m4, a.m2, a.magic);
    w1.run(lds_x1, lds_s1, [&](uint32_t cnt, float g, float u, uint32_t row) {
        if (lane < cnt && row < a.inter) st_dev(&s_act[row], tag_hi | (uint64_t)__float_as_uint(silu_mul_f32(g, u)));
    });

    // The workgroup's last wave out of phase 1 marks the workgroup: the marks only say WHEN collecting is worth starting
    // (2 KB to poll instead of 8 bytes per activation; polls that start early find little and get in the way of the
    // stores); what makes an activation valid is its own tag.
    {
        uint32_t prev = 0;
        if (lane == 0) prev = __hip_atomic_fetch_add(&lds_out, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        prev = (uint32_t)__builtin_amdgcn_readfirstlane((int)prev);
        if (prev == WAVES - 1u && lane == 0) st_dev(&s_done[b], tag_hi | 1u);
    }

    // ---- the first windows of the down rows: requested before the wait, they travel with the activations ----
    FlatWalk<TDN, false, kDownRing<TDN>, true> w2;
    w2.init(a.wd, a.wd, a.hidden, 1, a.gdn, wv * G + b, WAVES * G);
    w2.prime();

    if (wv == 0) {
        for (uint32_t i = lane; i < G; i += 64u) {
            uint64_t got = ld_dev(&s_done[i]);
            for (uint32_t n = 0; (uint32_t)(got >> 32) != tag; ++n) {
                if (n >= a.spin_limit) {
                    st_dev(s_err, 2u);
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
                got = ld_dev(&s_done[i]);
            }
        }
    }
    __syncthreads();

    // ---- all activations into LDS (f32, the layout of the down walk): coalesced 16-byte loads of two words, each asked for
    // again until it is fresh.  Eight consecutive lanes hold a run of sixteen activations; its sum is chained through them
    // in index order, as the staging of a stored row adds it. ----
    {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const uint32_t n2 = a.inter / 2u;
        for (uint32_t base = 0; base < n2; base += POLL * THREADS) {
            u32x4 got[POLL];
            uint32_t off[POLL];
#pragma unroll
            for (int i = 0; i < POLL; ++i) {
                const uint32_t e2 = base + tid + (uint32_t)i * THREADS;
                off[i] = 16u * (e2 < n2 ? e2 : 0u);  // past the end: the first words again, not used
                asm volatile("global_load_dwordx4 %0, %1, %2 sc0 sc1" : "=v"(got[i]) : "v"(off[i]), "s"(s_act) : "memory");
            }
            for (uint32_t tries = 0;; ++tries) {
                // the results exist once the counter has drained; naming them keeps their uses below the wait
                asm volatile("s_waitcnt vmcnt(0)" : "+v"(got[0]), "+v"(got[1]), "+v"(got[2]), "+v"(got[3]) : : "memory");
                bool fresh = true;
#pragma unroll
                for (int i = 0; i < POLL; ++i) {
                    if (got[i].y != tag || got[i].w != tag) {
                        fresh = false;
                        asm volatile("global_load_dwordx4 %0, %1, %2 sc0 sc1" : "+v"(got[i]) : "v"(off[i]), "s"(s_act) : "memory");
                    }
                }
                if (fresh) break;
                if (tries >= a.spin_limit) {
                    st_dev(s_err, 1u);
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
#pragma unroll
            for (int i = 0; i < POLL; ++i) {
                const uint32_t e2 = base + tid + (uint32_t)i * THREADS;  // (inter % 16 == 0: the eight lanes of a run are in or out together)
                const float v0 = __uint_as_float(got[i].x), v1 = __uint_as_float(got[i].z);
                float s = 0.f;
#pragma unroll
                for (uint32_t step = 0; step < 8; ++step) {
                    const float carry = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(s), 0x111 /* row_shr:1 */, 0xf, 0xf, false));
                    if ((lane & 7u) == step) s = ((step ? carry : 0.f) + v0) + v1;
                }
                if (e2 < n2) {
                    const uint32_t e = 2u * e2;
                    float* dst = reinterpret_cast<float*>(lds_x2) + X2::slot(e >> 2) * 4u + (e & 3u);
                    dst[0] = v0;
                    dst[1] = v1;
                    if ((lane & 7u) == 7u) lds_s2[e2 >> 3] = s;
                }
            }
        }
    }
    __syncthreads();

    // ---- phase 2: the down rows ----
    w2.load_masks(a.m4, a.m2, a.magic);
    w2.run(lds_x2, lds_s2, [&](uint32_t cnt, float y, float, uint32_t row) {
        if (lane < cnt && row < a.hidden) a.out[row] = a.residual ? y + a.residual[row] : y;
    });
    if (b == 0 && tid == 0) st_dev(s_epoch, tag);
}

template <int TYPE>
bool type_fits(uint32_t k) {
    return k % kUnitElems<TYPE> == 0 && k / kUnitElems<TYPE> >= 2;
}

template <int TGU, int TDN, bool X_BF16>
size_t lds_need(uint32_t hidden, uint32_t inter) {
    return ((FlatX<TGU, X_BF16>::lds_bytes(hidden) + 15u) & ~(size_t)15) + FlatX<TDN, false>::lds_bytes(inter);
}

template <int TGU, int TDN, bool X_BF16>
int launch_t(hipStream_t s, const DenseFfnArgs& d, uint32_t cus, bool dry) {
    if (!type_fits<TGU>(d.hidden) || !type_fits<TDN>(d.inter)) return fail(HQ_ERR_UNSUPPORTED, "dense FFN block: hidden %u / inter %u are not whole blocks", d.hidden, d.inter);
    const size_t lds = lds_need<TGU, TDN, X_BF16>(d.hidden, d.inter);
    if (lds > 160 * 1024 - 512) return fail(HQ_ERR_UNSUPPORTED, "dense FFN block: %zu bytes of LDS (hidden %u, inter %u)", lds, d.hidden, d.inter);
    if ((uint64_t)d.inter * (d.hidden / kUnitElems<TGU>) >= 0x7fff0000ull || (uint64_t)d.hidden * (d.inter / kUnitElems<TDN>) >= 0x7fff0000ull)
        return fail(HQ_ERR_UNSUPPORTED, "dense FFN block: matrices too large");
    // Every workgroup must deliver activations (see the header comment): no more workgroups than the gate / up walk has
    // super-tasks.
    const FlatGeom ggu = flat_geom(d.hidden, kUnitElems<TGU>, kUnitsPerWindow<TGU>, d.inter, 2, cus * WAVES);
    const uint32_t n_super = (d.inter + (1u << ggu.log_r) - 1u) >> ggu.log_r;
    uint32_t grid = cus < n_super ? cus : n_super;
    if (grid > kMaxGrid) grid = kMaxGrid;
    if (dry) return HQ_OK;
    DArgs a{};
    a.x = d.x;
    a.wg = static_cast<const uint8_t*>(d.w_gate);
    a.wu = static_cast<const uint8_t*>(d.w_up);
    a.wd = static_cast<const uint8_t*>(d.w_down);
    a.residual = d.residual;
    a.out = d.out;
    a.scratch = static_cast<uint8_t*>(d.scratch);
    a.hidden = d.hidden;
    a.inter = d.inter;
    a.ggu = ggu;
    a.gdn = flat_geom(d.inter, kUnitElems<TDN>, kUnitsPerWindow<TDN>, d.hidden, 1, grid * WAVES);
    a.m4 = TGU == HQ_Q6_K ? N4 : M4;
    a.m2 = TGU == HQ_Q5_K ? M1 : TGU == HQ_Q6_K ? N2 : M2;
    a.magic = MAGIC;
    a.spin_limit = d.spin_limit ? d.spin_limit : (1u << 20);
    auto kern = dense_ffn_kernel<TGU, TDN, X_BF16>;
    size_t lds_launch = lds < 81 * 1024 ? 81 * 1024 : lds;  // more than half a CU's LDS: one workgroup per CU
    if (int rc = ensure_lds_limit(reinterpret_cast<const void*>(kern), lds_launch, "hipFuncSetAttribute(dense FFN LDS)")) return rc;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(THREADS), lds_launch, s, a);
    return check_launch("dense FFN block launch");
}

// Q8_0 / Q4_0: the walk's own rule for doubled pieces, per matrix (gate and up are walked side by side).
template <int T, bool X_BF16>
int route_blocks(hipStream_t s, const DenseFfnArgs& d, uint32_t cus, bool dry) {
    const bool pg = walk_doubled<T, X_BF16>(2ull * d.inter, d.hidden), pd = walk_doubled<T, false>(d.hidden, d.inter);
    if (pg && pd) return launch_t<kX2 + T, kX2 + T, X_BF16>(s, d, cus, dry);
    if (pg) return launch_t<kX2 + T, T, X_BF16>(s, d, cus, dry);
    if (pd) return launch_t<T, kX2 + T, X_BF16>(s, d, cus, dry);
    return launch_t<T, T, X_BF16>(s, d, cus, dry);
}

template <bool X_BF16>
int route(hipStream_t s, const DenseFfnArgs& d, uint32_t cus, bool dry) {
    const hq_ggml_type g = d.t_gate_up, n = d.t_down;
    if (g == n) {
        switch (g) {
            case HQ_Q4_K: return launch_t<HQ_Q4_K, HQ_Q4_K, X_BF16>(s, d, cus, dry);
            case HQ_Q5_K: return launch_t<HQ_Q5_K, HQ_Q5_K, X_BF16>(s, d, cus, dry);
            case HQ_Q6_K: return launch_t<HQ_Q6_K, HQ_Q6_K, X_BF16>(s, d, cus, dry);
            case HQ_Q8_0: return route_blocks<HQ_Q8_0, X_BF16>(s, d, cus, dry);
            case HQ_Q4_0: return route_blocks<HQ_Q4_0, X_BF16>(s, d, cus, dry);
        }
    }
    // the mixes GGUF files of the reference's models hold: down in Q6_K over Q4_K or Q5_K gate / up
    if (g == HQ_Q4_K && n == HQ_Q6_K) return launch_t<HQ_Q4_K, HQ_Q6_K, X_BF16>(s, d, cus, dry);
    if (g == HQ_Q5_K && n == HQ_Q6_K) return launch_t<HQ_Q5_K, HQ_Q6_K, X_BF16>(s, d, cus, dry);
    return fail(HQ_ERR_UNSUPPORTED, "dense FFN block: gate / up type %d with down type %d", (int)g, (int)n);
}

}  // namespace

size_t dense_ffn_scratch_bytes(uint32_t inter) { return (kActOffset + (size_t)inter * 8 + 255) & ~(size_t)255; }

int launch_dense_ffn(hipStream_t s, const DenseFfnArgs& d, bool dry) {
    uint32_t cus = 256;
    if (!dry)
        if (int rc = cu_count(&cus)) return rc;
    return d.xdt == HQ_BF16 ? route<true>(s, d, cus, dry) : route<false>(s, d, cus, dry);
}

}  // namespace hq

// C entry points of libhf2q_hip.so: argument validation and routing.  Every
// check that the reference performs on the host before it dispatches (shape
// alignment, supported types, cache bounds) happens here and turns into an
// error code; kernels are only launched with shapes they were written for.
#include <stdarg.h>
#include <stdio.h>

#include <atomic>
#include <mutex>

#include "hq_internal.h"

namespace hq {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return HQ_OK;
    return fail(HQ_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

static bool known_type(hq_ggml_type t) {
    return t == HQ_Q8_0 || t == HQ_Q4_K || t == HQ_Q6_K || t == HQ_Q5_K || t == HQ_Q4_0;
}

// Largest activation-row count the GEMV kernels take; above it the MFMA GEMM
// runs (MM_ROUTING_THRESHOLD = 8, src/serve/forward_mlx.rs:9791).
constexpr uint32_t kGemvMaxRows = 8;

static int check_weight_alignment(const void* w, hq_ggml_type t) {
    const size_t need = (t == HQ_Q4_K || t == HQ_Q5_K) ? 16 : 2;
    if (!is_aligned(w, need))
        return fail(HQ_ERR_INVALID_ARGUMENT, "weight pointer must be %zu-byte aligned for ggml type %d",
                    need, (int)t);
    return HQ_OK;
}

// The device's CU count, cached per device.
int ensure_lds_limit(const void* kernel, size_t bytes, const char* what) {
    if (bytes < 64 * 1024) return HQ_OK;  // below the default limit
    struct Entry {
        const void* fn;
        int dev;
        size_t bytes;
    };
    static std::mutex mu;
    static Entry table[256];
    static int used = 0;
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    std::lock_guard<std::mutex> lock(mu);
    Entry* e = nullptr;
    for (int i = 0; i < used; ++i)
        if (table[i].fn == kernel && table[i].dev == dev) e = &table[i];
    if (e && e->bytes >= bytes) return HQ_OK;
    if (int rc = check_hip(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes), what)) return rc;
    if (!e && used < 256) e = &table[used++];
    if (e) *e = Entry{kernel, dev, bytes};  // a full table only means the attribute is set again next time
    return HQ_OK;
}

int cu_count(uint32_t* out) {
    static std::mutex mu;
    static int cached[64] = {};
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    std::lock_guard<std::mutex> lock(mu);
    if (dev < 0 || dev >= 64 || cached[dev] == 0) {
        int cus = 0;
        if (int rc = check_hip(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev),
                               "hipDeviceGetAttribute(CU count)"))
            return rc;
        if (cus <= 0) cus = 256;
        if (dev < 0 || dev >= 64) {
            *out = (uint32_t)cus;
            return HQ_OK;
        }
        cached[dev] = cus;
    }
    *out = (uint32_t)cached[dev];
    return HQ_OK;
}

// hq_stream_read_probe: a fixed grid of waves, each reading runs of 8 KiB (eight 16-byte non-temporal loads per lane, all
// issued before the first is used) a grid's width apart, front to back through the buffer.  Non-temporal, whole lines
// once each: the fastest way found to read on this device (510 MB in 74 us; 84 with plain loads).
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ p, uint64_t n16, uint32_t* sink) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t wave = (uint64_t)blockIdx.x * 4u + (threadIdx.x >> 6), waves = (uint64_t)gridDim.x * 4u;
    const uint64_t chunks = (n16 + 511u) / 512u;
    uint32_t acc = 0;
    for (uint64_t c = wave; c < chunks; c += waves) {
        uint4 v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint64_t j = c * 512u + 64u * i + lane;
            v[i] = ldnt16(reinterpret_cast<const uint8_t*>(p + (j < n16 ? j : n16 - 1u)));
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) acc ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    }
    if (acc == 0x9e3779b9u && *sink != acc) *sink = acc;  // keeps the loads; practically never taken
}

}  // namespace hq

using namespace hq;

// Polling limit of the in-launch hand-overs (0: the kernels' default); see hq_set_handover_spin_limit.
static std::atomic<uint32_t> g_spin_limit{0};

extern "C" {

const char* hq_last_error(void) { return g_err; }

int hq_version(void) { return 100; }

uint32_t hq_block_elems(hq_ggml_type t) {
    return (t == HQ_Q8_0 || t == HQ_Q4_0) ? 32u : (t == HQ_Q4_K || t == HQ_Q5_K || t == HQ_Q6_K) ? 256u : 0u;
}

uint32_t hq_block_bytes(hq_ggml_type t) {
    return t == HQ_Q8_0 ? Q8_0_BYTES : t == HQ_Q4_K ? Q4K_BYTES : t == HQ_Q6_K ? Q6K_BYTES : t == HQ_Q5_K ? Q5K_BYTES
           : t == HQ_Q4_0 ? Q4_0_BYTES : 0u;
}

int hq_dequant_ggml(void* stream, const void* w_blocks, void* out, hq_act_dtype out_dtype,
                    uint64_t n_elems, hq_ggml_type t) {
    if (!known_type(t)) return fail(HQ_ERR_UNSUPPORTED, "hq_dequant_ggml: unsupported ggml type %d", (int)t);
    if (out_dtype != HQ_F32 && out_dtype != HQ_BF16 && out_dtype != HQ_F16)
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_dequant_ggml: out_dtype %d", (int)out_dtype);
    if (n_elems % hq_block_elems(t))
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_dequant_ggml: n_elems %llu is not a multiple of the block size %u",
                    (unsigned long long)n_elems, hq_block_elems(t));
    if (n_elems == 0) return HQ_OK;
    if (!w_blocks || !out) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_dequant_ggml: null buffer");
    if (int rc = check_weight_alignment(w_blocks, t)) return rc;
    if (!is_aligned(out, 16)) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_dequant_ggml: out must be 16-byte aligned");
    return launch_dequant((hipStream_t)stream, w_blocks, out, out_dtype, n_elems, t);
}

static int quantize_common(const char* fn, void* stream, const float* src, uint64_t n_elems, uint64_t n_per_row, hq_ggml_type t,
                           void* out_blocks, const float* imatrix, bool with_imatrix, void* scratch, size_t scratch_bytes) {
    if (!known_type(t)) return fail(HQ_ERR_UNSUPPORTED, "%s: unsupported ggml type %d", fn, (int)t);
    const uint32_t be = hq_block_elems(t);
    // Same two shape rules as GgmlQuantizer::quantize (quantizer.rs:57-71).
    if (n_per_row == 0 || n_per_row % be)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: n_per_row %llu not a multiple of block size %u", fn, (unsigned long long)n_per_row, be);
    if (n_elems % n_per_row)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: n_elems %llu not a multiple of n_per_row %llu", fn, (unsigned long long)n_elems,
                    (unsigned long long)n_per_row);
    if (n_per_row / be > 0xffffffffull) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: n_per_row %llu", fn, (unsigned long long)n_per_row);
    if (n_elems == 0) return HQ_OK;
    if (!src || !out_blocks) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!is_aligned(src, 16)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: src must be 16-byte aligned", fn);
    if (int rc = check_weight_alignment(out_blocks, t)) return rc;
    float* rows = nullptr;
    if (with_imatrix) {
        if (!imatrix || !is_aligned(imatrix, 4)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: imatrix is null or not 4-byte aligned", fn);
        const size_t need = hq_quantize_ggml_imatrix_scratch_bytes(n_elems, n_per_row, t);
        if (need) {
            if (!scratch || !is_aligned(scratch, 4) || scratch_bytes < need)
                return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch of %zu bytes, %zu needed (4-byte aligned)", fn, scratch_bytes, need);
            rows = static_cast<float*>(scratch);
        }
    }
    return launch_quantize((hipStream_t)stream, src, n_elems, n_per_row, t, out_blocks, with_imatrix ? imatrix : nullptr, rows);
}

int hq_quantize_ggml(void* stream, const float* src, uint64_t n_elems, uint64_t n_per_row,
                     hq_ggml_type t, void* out_blocks) {
    return quantize_common("hq_quantize_ggml", stream, src, n_elems, n_per_row, t, out_blocks, nullptr, false, nullptr, 0);
}

size_t hq_quantize_ggml_imatrix_scratch_bytes(uint64_t n_elems, uint64_t n_per_row, hq_ggml_type t) {
    if (t != HQ_Q4_0 || n_per_row == 0) return 0;
    return (size_t)(n_elems / n_per_row) * sizeof(float);  // the mean square of every row
}

int hq_quantize_ggml_imatrix(void* stream, const float* src, uint64_t n_elems, uint64_t n_per_row, hq_ggml_type t,
                             const float* imatrix, void* out_blocks, void* scratch, size_t scratch_bytes) {
    return quantize_common("hq_quantize_ggml_imatrix", stream, src, n_elems, n_per_row, t, out_blocks, imatrix, true, scratch, scratch_bytes);
}

static int check_matmul_common(const char* fn, const void* x, hq_act_dtype xdt, const void* w,
                               const float* y, uint32_t n, uint32_t k, hq_ggml_type t) {
    if (!known_type(t)) return fail(HQ_ERR_UNSUPPORTED, "%s: unsupported ggml type %d", fn, (int)t);
    if (xdt != HQ_F32 && xdt != HQ_BF16) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: activation dtype %d", fn, (int)xdt);
    if (k == 0 || k % hq_block_elems(t))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: k %u is not a multiple of the block size %u", fn, k,
                    hq_block_elems(t));
    if (n == 0) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: n is 0", fn);
    if (!x || !w || !y) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!is_aligned(x, 16)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: x must be 16-byte aligned", fn);
    if (!is_aligned(y, 4)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: y must be 4-byte aligned", fn);
    return check_weight_alignment(w, t);
}

#ifndef HQ_CHUNK_LIMIT_Q4K
#define HQ_CHUNK_LIMIT_Q4K 2
#endif
#ifndef HQ_CHUNK_LIMIT_Q6K
#define HQ_CHUNK_LIMIT_Q6K 1
#endif
#ifndef HQ_CHUNK_LIMIT_Q80
#define HQ_CHUNK_LIMIT_Q80 1
#endif
namespace {

// Rows past the GEMV limit.  Every type has small tiles (Q4_K / Q5_K: 64 token rows, the others 128) whose one launch
// for any m <= 128 costs about what one to two chunks of kGemvMaxRows rows through the small-batch kernel cost
// (measured at 12288 x 4096: Q4_K 34 us against 15.5 us per chunk; Q6_K 44 against 32; Q8_0 43 against 33; Q4_0 33
// against 30), so Q4_K / Q5_K run two chunks before the tiles take over and the other types one.  Where a type has no
// small-batch kernel for this k (K-quants with k % 1024 != 0) two rounds of per-row GEMVs run first.
uint32_t chunked_rows_limit(uint32_t k, hq_ggml_type t) {
    if (!gemv_rows_supported(t, kGemvMaxRows, k) && !gemv_rows32_supported(t, kGemvMaxRows, k)) return 2 * kGemvMaxRows;
    if (t == HQ_Q4_K || t == HQ_Q5_K) return HQ_CHUNK_LIMIT_Q4K * kGemvMaxRows;
    return t == HQ_Q6_K ? HQ_CHUNK_LIMIT_Q6K * kGemvMaxRows : HQ_CHUNK_LIMIT_Q80 * kGemvMaxRows;
}

bool f16_tile_route(uint32_t m, uint32_t k, hq_ggml_type t) {
    return m > chunked_rows_limit(k, t) && gemm_f16_tile_supported(t, k);
}

// All routes of the dense product; `workspace` is only read on the f16 tile route.
int qmatmul_routes(hipStream_t stream, const void* x, hq_act_dtype xdt, const void* w_blocks, float* y, uint32_t m,
                   uint32_t n, uint32_t k, hq_ggml_type t, void* workspace, const float* w_scales = nullptr) {
    if (f16_tile_route(m, k, t)) return launch_gemm_f16_tile(stream, x, xdt, w_blocks, y, m, n, k, t, workspace, 0, w_scales);
    if (m > chunked_rows_limit(k, t) && gemm_supported(t, k)) return launch_gemm(stream, x, xdt, w_blocks, y, m, n, k, t);
    // kGemvMaxRows activation rows per launch: the small-batch kernel where it exists for the chunk, else one GEMV
    // per row (also the route of shapes the tile kernels do not cover).
    const size_t xrow_bytes = (size_t)k * (xdt == HQ_BF16 ? 2 : 4);
    for (uint32_t r0 = 0; r0 < m; r0 += kGemvMaxRows) {
        const uint32_t rows = m - r0 < kGemvMaxRows ? m - r0 : kGemvMaxRows;
        if ((gemv_rows_supported(t, rows, k) || gemv_rows_stream_fast(t, xdt, rows, n, k) || gemv_rows_stream_takes(t, xdt, rows, n, k)) &&
            !gemv_stream_passes_preferred(t, xdt, rows, n, k)) {
            if (int rc = launch_gemv_rows(stream, static_cast<const uint8_t*>(x) + (size_t)r0 * xrow_bytes, xdt, w_blocks,
                                          y + (size_t)r0 * n, rows, n, k, t))
                return rc;
            continue;
        }
        // five to eight f32 rows over Q8_0 / Q4_0: two passes of up to four rows on the matrix cores where that form fits
        // on a large matrix (lm_head 262144 x 2816: 2 x 141 us against 392 .. 428 with the kernel of exact f32 products below;
        // 12288 x 4096: 34 against 26 .. 27 us)
        if ((t == HQ_Q8_0 || t == HQ_Q4_0) && xdt != HQ_BF16 && rows > 4 && n >= 32768 && gemv_rows_stream_takes(t, xdt, 4, n, k)) {
            for (uint32_t h0 = 0; h0 < rows; h0 += 4) {
                const uint32_t hr = rows - h0 < 4 ? rows - h0 : 4;
                if (int rc = launch_gemv_rows(stream, static_cast<const uint8_t*>(x) + (size_t)(r0 + h0) * xrow_bytes, xdt, w_blocks,
                                              y + (size_t)(r0 + h0) * n, hr, n, k, t))
                    return rc;
            }
            continue;
        }
        if (gemv_rows32_supported(t, rows, k)) {
            if (int rc = launch_gemv_rows32(stream, static_cast<const uint8_t*>(x) + (size_t)r0 * xrow_bytes, xdt, w_blocks,
                                            y + (size_t)r0 * n, rows, n, k, t))
                return rc;
            continue;
        }
        GemvArgs a{};
        a.x = static_cast<const uint8_t*>(x) + (size_t)r0 * xrow_bytes;
        a.w = static_cast<const uint8_t*>(w_blocks);
        a.ids = nullptr;
        a.y = y + (size_t)r0 * n;
        a.pairs = m - r0 < kGemvMaxRows ? m - r0 : kGemvMaxRows;
        a.top_k = 1;
        a.n = n;
        a.k = k;
        a.n_experts = 1;
        a.expert_stride = 0;
        if (int rc = launch_gemv(stream, a, xdt, t)) return rc;
    }
    return HQ_OK;
}

}  // namespace

size_t hq_qmatmul_ggml_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt, hq_ggml_type t) {
    (void)n;
    (void)xdt;
    return f16_tile_route(m, k, t) ? gemm_f16_tile_workspace_bytes(m, n, k, t) : 0;
}

namespace {
int qmatmul_ws(const char* fn, void* stream, const void* x, hq_act_dtype xdt, const void* w_blocks, const float* w_scales,
               float* y, uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t, void* workspace, size_t workspace_bytes) {
    if (int rc = check_matmul_common(fn, x, xdt, w_blocks, y, n, k, t)) return rc;
    if (m == 0) return HQ_OK;
    const size_t need = hq_qmatmul_ggml_workspace_bytes(m, n, k, xdt, t);
    if (need) {
        if (!workspace || workspace_bytes < need)
            return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace of %zu bytes, %zu needed", fn,
                        workspace ? workspace_bytes : (size_t)0, need);
        if (reinterpret_cast<uintptr_t>(workspace) % 256)
            return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace must be 256-byte aligned", fn);
    }
    return qmatmul_routes((hipStream_t)stream, x, xdt, w_blocks, y, m, n, k, t, workspace, w_scales);
}
}  // namespace

int hq_qmatmul_ggml_k_slices(uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t, uint32_t* slices, uint32_t* blocks_per_slice) {
    if (!slices || !blocks_per_slice) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_qmatmul_ggml_k_slices: null output");
    if (!known_type(t) || n == 0 || k == 0 || k % hq_block_elems(t))
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_qmatmul_ggml_k_slices: type %d, n %u, k %u", (int)t, n, k);
    *slices = 1;
    *blocks_per_slice = (k + 255u) / 256u;
    if (f16_tile_route(m, k, t) && m <= 256) gemm_f16_small_tile_slices(t, m, n, k, slices, blocks_per_slice);
    return HQ_OK;
}

int hq_gemv_flat_plan(uint32_t n, uint32_t k, hq_ggml_type t, uint32_t waves, uint32_t* units_per_row, uint32_t* rows_per_task,
                      uint32_t* windows_per_task, uint32_t* units_per_window, uint32_t* window_capacity) {
    if (!units_per_row || !rows_per_task || !windows_per_task || !units_per_window || !window_capacity)
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gemv_flat_plan: null output");
    const uint32_t ue = t == HQ_Q8_0 || t == HQ_Q4_0 ? 32u : 256u;
    if (!known_type(t) || n == 0 || waves == 0 || k % ue || k / ue < 2)
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_gemv_flat_plan: type %d, n %u, k %u, waves %u", (int)t, n, k, waves);
    gemv_flat_plan(t, n, k, waves, units_per_row, rows_per_task, windows_per_task, units_per_window, window_capacity);
    return HQ_OK;
}

int hq_qmatmul_ggml_ws(void* stream, const void* x, hq_act_dtype xdt, const void* w_blocks, float* y, uint32_t m,
                       uint32_t n, uint32_t k, hq_ggml_type t, void* workspace, size_t workspace_bytes) {
    return qmatmul_ws("hq_qmatmul_ggml_ws", stream, x, xdt, w_blocks, nullptr, y, m, n, k, t, workspace, workspace_bytes);
}

int hq_qmatmul_ggml_ws_prepared(void* stream, const void* x, hq_act_dtype xdt, const void* w_blocks, const float* w_row_scales,
                                float* y, uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t, void* workspace,
                                size_t workspace_bytes) {
    if (!w_row_scales || !is_aligned(w_row_scales, 4))
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_qmatmul_ggml_ws_prepared: w_row_scales is null or not 4-byte aligned");
    return qmatmul_ws("hq_qmatmul_ggml_ws_prepared", stream, x, xdt, w_blocks, w_row_scales, y, m, n, k, t, workspace,
                      workspace_bytes);
}

int hq_weight_row_scales_ggml(void* stream, const void* w_blocks, float* scales, uint64_t n_rows, uint32_t k, hq_ggml_type t) {
    const char* fn = "hq_weight_row_scales_ggml";
    if (hq_block_elems(t) == 0) return fail(HQ_ERR_UNSUPPORTED, "%s: ggml type %d", fn, (int)t);
    if (k == 0 || k % hq_block_elems(t)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: k = %u is not a multiple of the block", fn, k);
    if (n_rows == 0) return HQ_OK;
    if (n_rows > 0x7fffffffull) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: %llu rows", fn, (unsigned long long)n_rows);
    if (!w_blocks || !scales || !is_aligned(scales, 4)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null or misaligned buffer", fn);
    if (int rc = check_weight_alignment(w_blocks, t)) return rc;
    return launch_weight_row_scales((hipStream_t)stream, w_blocks, scales, (uint32_t)n_rows, k, t);
}

int hq_qmatmul_ggml(void* stream, const void* x, hq_act_dtype xdt, const void* w_blocks, float* y,
                    uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t) {
    if (int rc = check_matmul_common("hq_qmatmul_ggml", x, xdt, w_blocks, y, n, k, t)) return rc;
    if (m == 0) return HQ_OK;
    const size_t need = hq_qmatmul_ggml_workspace_bytes(m, n, k, xdt, t);
    if (!need) return qmatmul_routes((hipStream_t)stream, x, xdt, w_blocks, y, m, n, k, t, nullptr);
    void* ws = nullptr;
    if (int rc = check_hip(hipMallocAsync(&ws, need, (hipStream_t)stream), "hipMallocAsync(qmatmul workspace)"))
        return rc;
    const int rc = qmatmul_routes((hipStream_t)stream, x, xdt, w_blocks, y, m, n, k, t, ws);
    const int rc_free = check_hip(hipFreeAsync(ws, (hipStream_t)stream), "hipFreeAsync(qmatmul workspace)");
    return rc ? rc : rc_free;
}

size_t hq_qmatmul_gated_ggml_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt, hq_ggml_type t) {
    if (hq_block_elems(t) == 0 || n == 0 || k == 0 || k % hq_block_elems(t)) return 0;
    return f16_tile_route(m, k, t) && gemm_f16_tile_gated_supported(t, m, n, k) ? hq_qmatmul_ggml_workspace_bytes(m, n, k, xdt, t) : 0;
}

int hq_qmatmul_gated_ggml_ws(void* stream, const void* x, hq_act_dtype xdt, const void* w_blocks, const float* w_row_scales,
                             const float* gate, float* y, uint32_t m, uint32_t n, uint32_t k, hq_ggml_type t, void* workspace,
                             size_t workspace_bytes) {
    const char* fn = "hq_qmatmul_gated_ggml_ws";
    if (int rc = check_matmul_common(fn, x, xdt, w_blocks, y, n, k, t)) return rc;
    if (!gate || !is_aligned(gate, 4)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: gate is null or not 4-byte aligned", fn);
    if (w_row_scales && !is_aligned(w_row_scales, 4)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: w_row_scales must be 4-byte aligned", fn);
    if (m == 0) return HQ_OK;
    const size_t need = hq_qmatmul_gated_ggml_workspace_bytes(m, n, k, xdt, t);
    if (!need)
        return fail(HQ_ERR_UNSUPPORTED,
                    "%s: this shape or type has no gated tile form (hq_qmatmul_gated_ggml_workspace_bytes is 0): "
                    "hq_qmatmul_ggml and hq_silu_mul give the same result", fn);
    if (!workspace || workspace_bytes < need)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace of %zu bytes, %zu needed", fn, workspace ? workspace_bytes : (size_t)0, need);
    if (reinterpret_cast<uintptr_t>(workspace) % 256) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace must be 256-byte aligned", fn);
    return launch_gemm_f16_tile((hipStream_t)stream, x, xdt, w_blocks, y, m, n, k, t, workspace, 0, w_row_scales, gate);
}

size_t hq_qmatmul_swiglu_ggml_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt, hq_ggml_type t) {
    (void)xdt;
    if (hq_block_elems(t) == 0 || n == 0 || k == 0 || k % hq_block_elems(t)) return 0;
    return (t == HQ_Q4_K || t == HQ_Q5_K) && f16_tile_route(m, k, t) ? gemm_f16_swiglu_workspace_bytes(m, n, k) : 0;
}

int hq_qmatmul_swiglu_ggml_ws(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up,
                              const float* gate_row_scales, const float* up_row_scales, float* y, uint32_t m, uint32_t n,
                              uint32_t k, hq_ggml_type t, void* workspace, size_t workspace_bytes) {
    const char* fn = "hq_qmatmul_swiglu_ggml_ws";
    if (int rc = check_matmul_common(fn, x, xdt, w_gate, y, n, k, t)) return rc;
    if (!w_up) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (int rc = check_weight_alignment(w_up, t)) return rc;
    if ((gate_row_scales == nullptr) != (up_row_scales == nullptr))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: the row scales of both matrices, or of neither", fn);
    if (gate_row_scales && (!is_aligned(gate_row_scales, 4) || !is_aligned(up_row_scales, 4)))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: row scales must be 4-byte aligned", fn);
    if (m == 0) return HQ_OK;
    const size_t need = hq_qmatmul_swiglu_ggml_workspace_bytes(m, n, k, xdt, t);
    if (!need)
        return fail(HQ_ERR_UNSUPPORTED,
                    "%s: this shape or type has no SwiGLU tile form (hq_qmatmul_swiglu_ggml_workspace_bytes is 0): two "
                    "hq_qmatmul_ggml calls and hq_silu_mul give the same result", fn);
    if (!workspace || workspace_bytes < need)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace of %zu bytes, %zu needed", fn, workspace ? workspace_bytes : (size_t)0, need);
    if (reinterpret_cast<uintptr_t>(workspace) % 256) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace must be 256-byte aligned", fn);
    return launch_gemm_f16_swiglu((hipStream_t)stream, x, xdt, w_gate, w_up, y, m, n, k, t, workspace, gate_row_scales, up_row_scales);
}

int hq_qmatmul_swiglu_decode_supported(uint32_t n, uint32_t k, hq_ggml_type t, hq_act_dtype xdt) {
    if (!known_type(t) || (xdt != HQ_F32 && xdt != HQ_BF16) || n == 0 || k == 0 || k % hq_block_elems(t)) return 0;
    return launch_gemv_swiglu(nullptr, nullptr, xdt, nullptr, nullptr, nullptr, 1, n, k, t, true) == HQ_OK;
}

int hq_qmatmul_swiglu_decode(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up, float* y, uint32_t m,
                             uint32_t n, uint32_t k, hq_ggml_type t) {
    const char* fn = "hq_qmatmul_swiglu_decode";
    if (int rc = check_matmul_common(fn, x, xdt, w_gate, y, n, k, t)) return rc;
    if (!w_up) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (int rc = check_weight_alignment(w_up, t)) return rc;
    if (m > kGemvMaxRows) return fail(HQ_ERR_UNSUPPORTED, "%s: %u rows (limit %u; hq_qmatmul_swiglu_ggml_ws is the prefill form)", fn, m, kGemvMaxRows);
    if (m == 0) return HQ_OK;
    return launch_gemv_swiglu((hipStream_t)stream, x, xdt, w_gate, w_up, y, m, n, k, t, false);
}

size_t hq_qmatmul_perm021_ggml_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt, hq_ggml_type t) {
    // the tile GEMM gathers while it converts; every other route first copies the activations into row-major order
    if (f16_tile_route(m, k, t)) return gemm_f16_tile_workspace_bytes(m, n, k, t);
    return (((size_t)m * k * (xdt == HQ_BF16 ? 2 : 4)) + 255) & ~(size_t)255;
}

int hq_qmatmul_perm021_ggml_ws(void* stream, const void* x_perm, hq_act_dtype xdt, const void* w_blocks, float* y, uint32_t m,
                               uint32_t n, uint32_t k, uint32_t head_dim, hq_ggml_type t, void* workspace,
                               size_t workspace_bytes) {
    const char* fn = "hq_qmatmul_perm021_ggml_ws";
    if (int rc = check_matmul_common(fn, x_perm, xdt, w_blocks, y, n, k, t)) return rc;
    if (head_dim == 0 || head_dim % 8 || k % head_dim)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: head_dim %u must be a multiple of 8 that divides k = %u", fn, head_dim, k);
    if (m == 0) return HQ_OK;
    const size_t need = hq_qmatmul_perm021_ggml_workspace_bytes(m, n, k, xdt, t);
    if (!workspace || workspace_bytes < need)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace of %zu bytes, %zu needed", fn, workspace ? workspace_bytes : (size_t)0, need);
    if (reinterpret_cast<uintptr_t>(workspace) % 256) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace must be 256-byte aligned", fn);
    if (f16_tile_route(m, k, t))
        return launch_gemm_f16_tile((hipStream_t)stream, x_perm, xdt, w_blocks, y, m, n, k, t, workspace, head_dim);
    if (int rc = launch_unpermute021((hipStream_t)stream, x_perm, workspace, m, k, head_dim, xdt == HQ_BF16 ? 2 : 4)) return rc;
    return qmatmul_routes((hipStream_t)stream, workspace, xdt, w_blocks, y, m, n, k, t, nullptr);
}

size_t hq_qmatmul_id_scratch_bytes(uint32_t n_experts, uint32_t max_rows) {
    (void)n_experts;
    (void)max_rows;
    return 0;
}

namespace {
// Routed rows per expert from which the grouped tile GEMM takes over from one GEMV per row (256 experts of 512 x 2048
// Q4_K, top-8: the MoE block takes 310 us against 346 at 96 tokens, 319 against 412 at 128; at 64 tokens, two rows per
// expert, the GEMVs are ahead, 257 against 315).
constexpr uint64_t kGroupedRowsPerExpert = 3;
bool grouped_route(uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k, uint32_t n_experts, uint64_t expert_stride,
                   hq_ggml_type t) {
    const uint64_t pairs = (uint64_t)n_tokens * top_k;
    return pairs >= 256 && pairs >= kGroupedRowsPerExpert * n_experts &&
           gemm_f16_grouped_supported(t, n, k, n_experts, expert_stride, pairs);
}
}  // namespace

size_t hq_qmatmul_id_ggml_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k, uint32_t n_experts,
                                          uint64_t expert_stride, hq_ggml_type t) {
    if (hq_block_elems(t) == 0) return 0;  // not a type of this library
    if (n == 0 || k == 0 || k % hq_block_elems(t)) return 0;
    return grouped_route(n_tokens, top_k, n, k, n_experts, expert_stride, t)
               ? gemm_f16_grouped_workspace_bytes(n_tokens, top_k, n_experts, n, k) : 0;
}

namespace {
int qmatmul_id(const char* fn, void* stream, const void* x, hq_act_dtype xdt, const void* w_stack, const float* w_scales,
               const uint32_t* ids, float* y, void* scratch, size_t scratch_bytes, uint32_t n_tokens, uint32_t top_k, uint32_t n,
               uint32_t k, uint32_t n_experts, uint64_t expert_stride, hq_ggml_type t);
}  // namespace

int hq_qmatmul_id_ggml(void* stream, const void* x, hq_act_dtype xdt, const void* w_stack,
                       const uint32_t* ids, float* y, void* scratch, size_t scratch_bytes,
                       uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k,
                       uint32_t n_experts, uint64_t expert_stride, hq_ggml_type t) {
    return qmatmul_id("hq_qmatmul_id_ggml", stream, x, xdt, w_stack, nullptr, ids, y, scratch, scratch_bytes, n_tokens, top_k, n, k,
                      n_experts, expert_stride, t);
}

int hq_qmatmul_id_ggml_prepared(void* stream, const void* x, hq_act_dtype xdt, const void* w_stack, const float* w_row_scales,
                                const uint32_t* ids, float* y, void* scratch, size_t scratch_bytes, uint32_t n_tokens,
                                uint32_t top_k, uint32_t n, uint32_t k, uint32_t n_experts, uint64_t expert_stride,
                                hq_ggml_type t) {
    if (!w_row_scales || !is_aligned(w_row_scales, 4))
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_qmatmul_id_ggml_prepared: w_row_scales is null or not 4-byte aligned");
    return qmatmul_id("hq_qmatmul_id_ggml_prepared", stream, x, xdt, w_stack, w_row_scales, ids, y, scratch, scratch_bytes, n_tokens,
                      top_k, n, k, n_experts, expert_stride, t);
}

namespace {
int qmatmul_id(const char* fn, void* stream, const void* x, hq_act_dtype xdt, const void* w_stack, const float* w_scales,
               const uint32_t* ids, float* y, void* scratch, size_t scratch_bytes, uint32_t n_tokens, uint32_t top_k, uint32_t n,
               uint32_t k, uint32_t n_experts, uint64_t expert_stride, hq_ggml_type t) {
    if (int rc = check_matmul_common(fn, x, xdt, w_stack, y, n, k, t)) return rc;
    if (!ids) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null ids", fn);
    if (n_experts == 0 || top_k == 0)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: n_experts %u, top_k %u", fn, n_experts, top_k);
    const uint64_t expert_bytes = (uint64_t)n * (k / hq_block_elems(t)) * hq_block_bytes(t);
    if (expert_stride < expert_bytes)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: expert_stride %llu < one expert's %llu bytes", fn,
                    (unsigned long long)expert_stride, (unsigned long long)expert_bytes);
    if (expert_stride % ((t == HQ_Q4_K || t == HQ_Q5_K) ? 16 : 2))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: expert_stride %llu breaks block alignment", fn,
                    (unsigned long long)expert_stride);
    const uint64_t pairs = (uint64_t)n_tokens * top_k;
    if (pairs == 0) return HQ_OK;
    // Many rows per expert and a workspace from the caller: rows sorted by expert, tile GEMM per expert.
    if (scratch && grouped_route(n_tokens, top_k, n, k, n_experts, expert_stride, t)) {
        const size_t need = gemm_f16_grouped_workspace_bytes(n_tokens, top_k, n_experts, n, k);
        if (scratch_bytes < need)
            return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch of %zu bytes, %zu needed", fn, scratch_bytes, need);
        if (reinterpret_cast<uintptr_t>(scratch) % 256)
            return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch must be 256-byte aligned", fn);
        return launch_gemm_f16_grouped((hipStream_t)stream, x, xdt, w_stack, ids, y, scratch, n_tokens, top_k, n, k, n_experts,
                                       expert_stride, t, w_scales);
    }
    // One GEMV per routed row, up to 65535 rows per launch (grid.y).  Rows that share an expert read
    // its weights through L2.
    const size_t xrow_bytes = (size_t)k * (xdt == HQ_BF16 ? 2 : 4);
    constexpr uint64_t kMaxPerLaunch = 65535u / 1u;
    for (uint64_t p0 = 0; p0 < pairs;) {
        // keep launches aligned to whole tokens so that the x row of pair p is (p0 + p) / top_k
        uint64_t cnt = pairs - p0 < kMaxPerLaunch ? pairs - p0 : kMaxPerLaunch;
        if (cnt < pairs - p0) cnt -= cnt % top_k;
        if (cnt == 0) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: top_k %u too large", fn, top_k);
        GemvArgs a{};
        a.x = static_cast<const uint8_t*>(x) + (size_t)(p0 / top_k) * xrow_bytes;
        a.w = static_cast<const uint8_t*>(w_stack);
        a.ids = ids + p0;
        a.y = y + (size_t)p0 * n;
        a.pairs = (uint32_t)cnt;
        a.top_k = top_k;
        a.n = n;
        a.k = k;
        a.n_experts = n_experts;
        a.expert_stride = expert_stride;
        if (int rc = launch_gemv((hipStream_t)stream, a, xdt, t)) return rc;
        p0 += cnt;
    }
    return HQ_OK;
}
}  // namespace

size_t hq_qmatmul_id_swiglu_ggml_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k, uint32_t n_experts,
                                                 uint64_t expert_stride, hq_ggml_type t) {
    if (hq_block_elems(t) == 0 || n == 0 || k == 0 || k % hq_block_elems(t)) return 0;
    return gemm_f16_grouped_swiglu_supported(t) && grouped_route(n_tokens, top_k, n, k, n_experts, expert_stride, t)
               ? gemm_f16_grouped_workspace_bytes(n_tokens, top_k, n_experts, n, k, 2) : 0;
}

int hq_qmatmul_id_swiglu_ggml(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate_stack, const void* w_up_stack,
                              const float* gate_row_scales, const float* up_row_scales, const uint32_t* ids, float* y,
                              void* scratch, size_t scratch_bytes, uint32_t n_tokens, uint32_t top_k, uint32_t n, uint32_t k,
                              uint32_t n_experts, uint64_t expert_stride, hq_ggml_type t) {
    const char* fn = "hq_qmatmul_id_swiglu_ggml";
    if (int rc = check_matmul_common(fn, x, xdt, w_gate_stack, y, n, k, t)) return rc;
    if (!w_up_stack) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (int rc = check_weight_alignment(w_up_stack, t)) return rc;
    if (!ids) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null ids", fn);
    if (n_experts == 0 || top_k == 0) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: n_experts %u, top_k %u", fn, n_experts, top_k);
    if ((gate_row_scales == nullptr) != (up_row_scales == nullptr))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: the row scales of both stacks, or of neither", fn);
    if (gate_row_scales && (!is_aligned(gate_row_scales, 4) || !is_aligned(up_row_scales, 4)))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: row scales must be 4-byte aligned", fn);
    if ((uint64_t)n_tokens * top_k == 0) return HQ_OK;
    const size_t need = hq_qmatmul_id_swiglu_ggml_workspace_bytes(n_tokens, top_k, n, k, n_experts, expert_stride, t);
    if (!need)
        return fail(HQ_ERR_UNSUPPORTED,
                    "%s: this shape or type has no grouped SwiGLU form (hq_qmatmul_id_swiglu_ggml_workspace_bytes is 0): "
                    "two hq_qmatmul_id_ggml calls and hq_silu_mul give the same result", fn);
    if (!scratch || scratch_bytes < need)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch of %zu bytes, %zu needed", fn, scratch ? scratch_bytes : (size_t)0, need);
    if (reinterpret_cast<uintptr_t>(scratch) % 256) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch must be 256-byte aligned", fn);
    return launch_gemm_f16_grouped((hipStream_t)stream, x, xdt, w_gate_stack, ids, y, scratch, n_tokens, top_k, n, k, n_experts,
                                   expert_stride, t, gate_row_scales, w_up_stack, up_row_scales);
}

int hq_qmatmul_batch_ggml(void* stream, const hq_qmatmul_job* jobs, uint32_t n_jobs, hq_act_dtype xdt,
                          hq_ggml_type t) {
    const char* fn = "hq_qmatmul_batch_ggml";
    if (n_jobs == 0) return HQ_OK;
    if (!jobs) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null jobs", fn);
    if (n_jobs > HQ_QMATMUL_BATCH_MAX_JOBS)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: %u jobs (limit %d)", fn, n_jobs, HQ_QMATMUL_BATCH_MAX_JOBS);
    GemvArgs ga[HQ_QMATMUL_BATCH_MAX_JOBS];
    uint32_t live = 0;
    for (uint32_t i = 0; i < n_jobs; ++i) {
        const hq_qmatmul_job& j = jobs[i];
        if (int rc = check_matmul_common(fn, j.x, xdt, j.w, j.y, j.n, j.k, t)) return rc;
        if (j.x_up) {
            if (xdt != HQ_F32) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: job %u: x_up needs f32 activations", fn, i);
            if (!is_aligned(j.x_up, 16)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: job %u: x_up must be 16-byte aligned", fn, i);
        }
        GemvArgs a{};
        a.x = j.x;
        a.x2 = j.x_up;
        a.w = static_cast<const uint8_t*>(j.w);
        a.y = j.y;
        a.n = j.n;
        a.k = j.k;
        if (j.route_logits) {
            if (j.ids) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: job %u: ids and route_logits are both set", fn, i);
            if (j.n_experts > 256 || j.top_k > 64 || j.top_k > j.n_experts)
                return fail(HQ_ERR_UNSUPPORTED, "%s: job %u: in-launch routing takes n_experts <= 256 and top_k <= min(64, n_experts)", fn, i);
            if (!j.route_ids != !j.route_weights)
                return fail(HQ_ERR_INVALID_ARGUMENT, "%s: job %u: route_ids and route_weights go together", fn, i);
        }
        if (j.ids || j.route_logits) {
            if (j.n_experts == 0 || j.top_k == 0)
                return fail(HQ_ERR_INVALID_ARGUMENT, "%s: job %u: n_experts %u, top_k %u", fn, i, j.n_experts, j.top_k);
            const uint64_t expert_bytes = (uint64_t)j.n * (j.k / hq_block_elems(t)) * hq_block_bytes(t);
            if (j.expert_stride < expert_bytes || j.expert_stride % ((t == HQ_Q4_K || t == HQ_Q5_K) ? 16 : 2))
                return fail(HQ_ERR_INVALID_ARGUMENT, "%s: job %u: expert_stride %llu (one expert is %llu bytes)", fn, i,
                            (unsigned long long)j.expert_stride, (unsigned long long)expert_bytes);
            const uint64_t pairs = (uint64_t)j.rows * j.top_k;
            if (pairs > 65535) return fail(HQ_ERR_UNSUPPORTED, "%s: job %u: %llu routed rows (limit 65535)", fn, i, (unsigned long long)pairs);
            a.ids = j.ids;
            a.route_logits = j.route_logits;
            a.route_ids = j.route_ids;
            a.route_w = j.route_weights;
            a.pairs = (uint32_t)pairs;
            a.top_k = j.top_k;
            a.n_experts = j.n_experts;
            a.expert_stride = j.expert_stride;
        } else {
            // the dense form is the decode route only: more rows belong to the tile kernels
            if (j.rows > kGemvMaxRows)
                return fail(HQ_ERR_UNSUPPORTED, "%s: job %u: %u dense rows (limit %u; use hq_qmatmul_ggml)", fn, i, j.rows, kGemvMaxRows);
            a.pairs = j.rows;
            a.top_k = 1;
            a.n_experts = 1;
        }
        if (a.pairs == 0) continue;
        ga[live++] = a;
    }
    return launch_gemv_jobs((hipStream_t)stream, ga, live, xdt, t);
}

size_t hq_moe_ffn_decode_scratch_bytes(uint32_t n_tokens, uint32_t hidden, uint32_t n_experts, uint32_t top_k, uint32_t inter,
                                       uint32_t shared_inter, hq_ggml_type t, hq_act_dtype xdt) {
    if (!moe_fused_supported(n_tokens, hidden, n_experts, top_k, inter, shared_inter, t, t, xdt)) return 0;
    return moe_fused_scratch_bytes(n_tokens, n_experts, top_k);
}

size_t hq_moe_ffn_decode_layer_scratch_bytes(const hq_moe_ffn_layer* l, uint32_t n_tokens, hq_act_dtype xdt) {
    if (!l) return 0;
    const hq_ggml_type td = l->down_type ? (hq_ggml_type)l->down_type : l->ggml_type;
    if (!moe_fused_supported(n_tokens, l->hidden, l->n_experts, l->top_k, l->inter, l->shared_inter, l->ggml_type, td, xdt)) return 0;
    return moe_fused_scratch_bytes(n_tokens, l->n_experts, l->top_k);
}

int hq_moe_ffn_decode(void* stream, const hq_moe_ffn_layer* l, const void* x, hq_act_dtype xdt, const float* residual,
                      float* out, uint32_t n_tokens, void* scratch, size_t scratch_bytes, uint32_t* route_ids,
                      float* route_weights) {
    const char* fn = "hq_moe_ffn_decode";
    if (!l) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null layer", fn);
    if (n_tokens == 0) return HQ_OK;
    const hq_ggml_type t_down = l->down_type ? (hq_ggml_type)l->down_type : l->ggml_type;
    if (!moe_fused_supported(n_tokens, l->hidden, l->n_experts, l->top_k, l->inter, l->shared_inter, l->ggml_type, t_down, xdt))
        return fail(HQ_ERR_UNSUPPORTED,
                    "%s: takes 1..8 tokens of bf16 activations, K-quant experts (one type, or Q4_K / Q5_K gate / up with a Q6_K down), "
                    "hidden 2048, expert and shared FFN width 512, <= 256 experts (got %u tokens, dtype %d, types %d / %d, hidden %u, "
                    "inter %u / %u, %u experts, top-%u); run the block as separate dispatches",
                    fn, n_tokens, (int)xdt, (int)l->ggml_type, (int)t_down, l->hidden, l->inter, l->shared_inter, l->n_experts, l->top_k);
    if (!x || !out || !scratch || !l->router || !l->expert_gate || !l->expert_up || !l->expert_down || !l->shared_gate ||
        !l->shared_up || !l->shared_down)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!route_ids != !route_weights) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: route_ids and route_weights go together", fn);
    const void* al16[] = {x, out, l->router, l->shared_gate_logit, l->expert_gate, l->expert_up, l->expert_down,
                          l->shared_gate, l->shared_up, l->shared_down, residual};
    for (const void* p : al16)
        if (!is_aligned(p, 16)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: every buffer must be 16-byte aligned", fn);
    if (!is_aligned(scratch, 256)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch must be 256-byte aligned", fn);
    const size_t need = moe_fused_scratch_bytes(n_tokens, l->n_experts, l->top_k);
    if (scratch_bytes < need) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch of %zu bytes, %zu needed", fn, scratch_bytes, need);
    const uint64_t gu_bytes = (uint64_t)l->inter * (l->hidden / 256) * hq_block_bytes(l->ggml_type),
                   d_bytes = (uint64_t)l->hidden * (l->inter / 256) * hq_block_bytes(t_down);
    if (l->expert_stride_gate_up < gu_bytes || l->expert_stride_gate_up % 16 || l->expert_stride_down < d_bytes || l->expert_stride_down % 16)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: expert strides %llu / %llu (one expert is %llu / %llu bytes)", fn,
                    (unsigned long long)l->expert_stride_gate_up, (unsigned long long)l->expert_stride_down,
                    (unsigned long long)gu_bytes, (unsigned long long)d_bytes);
    MoeFusedArgs a{};
    a.x = x;
    a.router = l->router;
    a.shared_gate_logit = l->shared_gate_logit;
    a.expert_gate = l->expert_gate;
    a.expert_up = l->expert_up;
    a.expert_down = l->expert_down;
    a.shared_gate = l->shared_gate;
    a.shared_up = l->shared_up;
    a.shared_down = l->shared_down;
    a.residual = residual;
    a.out = out;
    a.route_ids = route_ids;
    a.route_weights = route_weights;
    a.scratch = scratch;
    a.n_tokens = n_tokens;
    a.n_experts = l->n_experts;
    a.top_k = l->top_k;
    a.stride_gate_up = l->expert_stride_gate_up;
    a.stride_down = l->expert_stride_down;
    a.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
    a.t_gate_up = l->ggml_type;
    a.t_down = t_down;
    return launch_moe_fused((hipStream_t)stream, a);
}

size_t hq_matmul_f16_shadow_workspace_bytes(uint32_t m, uint32_t n, uint32_t k) {
    if (m == 0 || n == 0 || k == 0) return 0;
    return f16_shadow_workspace_bytes(m, k);
}

int hq_matmul_f16_shadow(void* stream, const void* x, hq_act_dtype xdt, const void* w_f16, float* y, uint32_t m, uint32_t n, uint32_t k,
                         void* workspace, size_t workspace_bytes) {
    const char* fn = "hq_matmul_f16_shadow";
    if (m == 0 || n == 0) return HQ_OK;
    if (xdt != HQ_F32 && xdt != HQ_BF16) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: activation dtype %d", fn, (int)xdt);
    if (k == 0 || k % 8) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: k = %u is not a positive multiple of 8", fn, k);
    if (!x || !w_f16 || !y || !workspace) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
    if (!is_aligned(x, 16) || !is_aligned(w_f16, 16) || !is_aligned(y, 16) || !is_aligned(workspace, 256))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: x, w_f16 and y must be 16-byte aligned, workspace 256-byte aligned", fn);
    const size_t need = f16_shadow_workspace_bytes(m, k);
    if (workspace_bytes < need) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace of %zu bytes, %zu needed", fn, workspace_bytes, need);
    return launch_f16_shadow_matmul((hipStream_t)stream, x, xdt, w_f16, y, m, n, k, workspace, need);
}

// Rows that take the GEMV of dense.hip (the reference's matvec kernels serve m = 1; a few rows are as many passes).
static bool dense_rows_as_gemv(uint32_t m, uint32_t k, hq_act_dtype wdt) { return m <= kGemvMaxRows && dense_gemv_takes(k, wdt); }

size_t hq_dense_matmul_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, hq_act_dtype xdt, hq_act_dtype wdt) {
    if (m == 0 || n == 0 || k == 0 || (wdt != HQ_F16 && wdt != HQ_F32) || dense_rows_as_gemv(m, k, wdt)) return 0;
    return wdt == HQ_F16 ? f16_shadow_workspace_bytes(m, k) : f32_dense_workspace_bytes(m, k, xdt);
}

int hq_dense_matmul(void* stream, const void* x, hq_act_dtype xdt, const void* w, hq_act_dtype wdt, float* y, uint32_t m, uint32_t n,
                    uint32_t k, void* workspace, size_t workspace_bytes) {
    const char* fn = "hq_dense_matmul";
    if (m == 0 || n == 0) return HQ_OK;
    if (xdt != HQ_F32 && xdt != HQ_BF16) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: activation dtype %d", fn, (int)xdt);
    if (wdt != HQ_F32 && wdt != HQ_F16) return fail(HQ_ERR_UNSUPPORTED, "%s: weight dtype %d (f32 or f16)", fn, (int)wdt);
    if (k == 0 || k % 8) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: k = %u is not a positive multiple of 8", fn, k);
    if (!x || !w || !y) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
    if (!is_aligned(x, 16) || !is_aligned(w, 16) || !is_aligned(y, 16))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: x, w and y must be 16-byte aligned", fn);
    if (dense_rows_as_gemv(m, k, wdt)) return launch_dense_gemv((hipStream_t)stream, x, xdt, w, wdt, y, m, n, k);
    const size_t need = hq_dense_matmul_workspace_bytes(m, n, k, xdt, wdt);
    if (!workspace || !is_aligned(workspace, 256) || workspace_bytes < need)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: workspace of %zu bytes (256-byte aligned), %zu needed", fn, workspace ? workspace_bytes : (size_t)0, need);
    if (wdt == HQ_F16) return launch_f16_shadow_matmul((hipStream_t)stream, x, xdt, w, y, m, n, k, workspace, need);
    return launch_f32_dense_matmul((hipStream_t)stream, x, xdt, w, y, m, n, k, workspace, need);
}

int hq_stream_read_probe(void* stream, const void* buf, size_t bytes, uint32_t* sink) {
    if (bytes == 0) return HQ_OK;
    if (!buf || !sink || bytes % 16 || !is_aligned(buf, 16))
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_stream_read_probe: buf / sink null, or buf / bytes not multiples of 16");
    const uint64_t n16 = bytes / 16, chunks = (n16 + 511) / 512;
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    const uint64_t blocks = chunks / 4 + 1 < 8ull * cus ? chunks / 4 + 1 : 8ull * cus;  // eight workgroups of four waves per CU
    hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, static_cast<const uint4*>(buf), n16, sink);
    return check_launch("stream read probe launch");
}

void hq_set_handover_spin_limit(uint32_t limit) { g_spin_limit.store(limit, std::memory_order_relaxed); }

int hq_handover_status(void* stream, const void* scratch, uint32_t* error) {
    if (!scratch || !error) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_handover_status: null argument");
    if (int rc = check_hip(hipMemcpyAsync(error, static_cast<const uint8_t*>(scratch) + 4, 4, hipMemcpyDeviceToHost, (hipStream_t)stream),
                           "hipMemcpyAsync(hand-over error word)"))
        return rc;
    return check_hip(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize(hand-over status)");
}

static int dense_ffn_args(const char* fn, DenseFfnArgs* a, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up,
                          const void* w_down, hq_ggml_type t_gate_up, hq_ggml_type t_down, const float* residual, float* out,
                          uint32_t hidden, uint32_t inter, void* scratch) {
    if (!known_type(t_gate_up) || !known_type(t_down)) return fail(HQ_ERR_UNSUPPORTED, "%s: ggml types %d / %d", fn, (int)t_gate_up, (int)t_down);
    if (xdt != HQ_F32 && xdt != HQ_BF16) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: activation dtype %d", fn, (int)xdt);
    *a = DenseFfnArgs{x, xdt, w_gate, w_up, w_down, t_gate_up, t_down, residual, out, scratch, hidden, inter,
                      g_spin_limit.load(std::memory_order_relaxed)};
    return HQ_OK;
}

size_t hq_dense_ffn_decode_scratch_bytes(uint32_t hidden, uint32_t inter, hq_ggml_type t_gate_up, hq_ggml_type t_down, hq_act_dtype xdt) {
    DenseFfnArgs a;
    if (hidden == 0 || inter == 0) return 0;
    if (dense_ffn_args("hq_dense_ffn_decode_scratch_bytes", &a, nullptr, xdt, nullptr, nullptr, nullptr, t_gate_up, t_down, nullptr,
                       nullptr, hidden, inter, nullptr))
        return 0;
    return launch_dense_ffn(nullptr, a, true) == HQ_OK ? dense_ffn_scratch_bytes(inter) : 0;
}

int hq_dense_ffn_decode(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up, const void* w_down,
                        hq_ggml_type t_gate_up, hq_ggml_type t_down, const float* residual, float* out, uint32_t hidden,
                        uint32_t inter, void* scratch, size_t scratch_bytes) {
    const char* fn = "hq_dense_ffn_decode";
    DenseFfnArgs a;
    if (int rc = dense_ffn_args(fn, &a, x, xdt, w_gate, w_up, w_down, t_gate_up, t_down, residual, out, hidden, inter, scratch)) return rc;
    if (hidden == 0 || inter == 0) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: hidden %u, inter %u", fn, hidden, inter);
    if (int rc = launch_dense_ffn(nullptr, a, true)) return rc;  // shape and types
    if (!x || !w_gate || !w_up || !w_down || !out || !scratch) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!is_aligned(x, 16) || !is_aligned(out, 4) || !is_aligned(residual, 4))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: x needs 16-byte, out / residual 4-byte alignment", fn);
    if (int rc = check_weight_alignment(w_gate, t_gate_up)) return rc;
    if (int rc = check_weight_alignment(w_up, t_gate_up)) return rc;
    if (int rc = check_weight_alignment(w_down, t_down)) return rc;
    if (!is_aligned(scratch, 256)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch must be 256-byte aligned", fn);
    if (scratch_bytes < dense_ffn_scratch_bytes(inter))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch of %zu bytes, %zu needed", fn, scratch_bytes, dense_ffn_scratch_bytes(inter));
    return launch_dense_ffn((hipStream_t)stream, a, false);
}

static int check_fwht(const char* fn, const float* buf, uint32_t n_heads, uint32_t head_dim) {
    if (head_dim != 256 && head_dim != 512) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: head_dim %u (256 or 512)", fn, head_dim);
    if (n_heads && !buf) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!is_aligned(buf, 16)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: buffer must be 16-byte aligned", fn);
    return HQ_OK;
}

int hq_fwht_sign_premult_f32(void* stream, float* buf, uint32_t n_heads, uint32_t head_dim) {
    if (int rc = check_fwht("hq_fwht_sign_premult_f32", buf, n_heads, head_dim)) return rc;
    if (n_heads == 0) return HQ_OK;
    return launch_fwht_sign((hipStream_t)stream, buf, n_heads, head_dim, false);
}

int hq_fwht_sign_undo_f32(void* stream, float* buf, uint32_t n_heads, uint32_t head_dim) {
    if (int rc = check_fwht("hq_fwht_sign_undo_f32", buf, n_heads, head_dim)) return rc;
    if (n_heads == 0) return HQ_OK;
    return launch_fwht_sign((hipStream_t)stream, buf, n_heads, head_dim, true);
}

int hq_tq_encode_kv(void* stream, const float* src, uint8_t* codes, float* norms, uint32_t n_tokens,
                    uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t write_pos) {
    if (head_dim != 256 && head_dim != 512)
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_tq_encode_kv: head_dim %u (256 or 512)", head_dim);
    if (capacity == 0 || n_tokens > capacity)
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_tq_encode_kv: %u tokens into a cache of capacity %u", n_tokens, capacity);
    if (n_tokens == 0 || n_kv_heads == 0) return HQ_OK;
    if (!src || !codes || !norms) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_tq_encode_kv: null buffer");
    if (!is_aligned(src, 16) || !is_aligned(codes, 4) || !is_aligned(norms, 4))
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_tq_encode_kv: src needs 16-byte, codes / norms 4-byte alignment");
    return launch_tq_encode((hipStream_t)stream, src, codes, norms, n_tokens, n_kv_heads, head_dim, capacity,
                            write_pos % capacity);
}

int hq_tq_dequantize_kv_seq(void* stream, const uint8_t* codes, const float* norms, const float* lut256, float* dst,
                            uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t start_pos,
                            uint32_t n_tokens, float scale_factor_d512, uint32_t codebook_bits, int unrotate) {
    const char* fn = "hq_tq_dequantize_kv_seq";
    if (head_dim != 256 && head_dim != 512) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: head_dim %u (256 or 512)", fn, head_dim);
    if (codebook_bits != 5 && codebook_bits != 6 && codebook_bits != 8)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: codebook_bits %u (5, 6 or 8)", fn, codebook_bits);
    if ((uint64_t)start_pos + n_tokens > capacity)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: positions %u..%llu past the capacity %u", fn, start_pos,
                    (unsigned long long)start_pos + n_tokens, capacity);
    if (codebook_bits != 8 && !lut256)
        return fail(HQ_ERR_UNSUPPORTED, "%s: a %u-bit cache needs its centroid table (lut256)", fn, codebook_bits);
    if (n_kv_heads == 0 || n_tokens == 0) return HQ_OK;
    if ((uint64_t)n_kv_heads * n_tokens * (head_dim / 256) > 0x7fffffffull)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: %u heads x %u tokens is too large for one call", fn, n_kv_heads, n_tokens);
    if (!codes || !norms || !dst) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!is_aligned(codes, 4) || !is_aligned(norms, 4) || !is_aligned(dst, 16))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: codes / norms need 4-byte, dst 16-byte alignment", fn);
    return launch_tq_dequantize((hipStream_t)stream, codes, norms, lut256, dst, n_kv_heads, head_dim, capacity, start_pos,
                                n_tokens, scale_factor_d512, unrotate != 0);
}

size_t hq_flash_attn_vec_tq_tmp_bytes(uint32_t num_heads, uint32_t head_dim, uint32_t kv_seq_len) {
    return tq_attn_tmp_bytes(num_heads, head_dim, kv_seq_len);
}

static int flash_attn_vec_tq(const char* fn, bool undo_rotation, void* stream, const float* q, const uint8_t* k_codes,
                             const float* k_norms, const uint8_t* v_codes, const float* v_norms, const float* lut256,
                             float* out, void* tmp, size_t tmp_bytes, const hq_tq_attn_params* p) {
    if (!p) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null params", fn);
    if (p->head_dim != 256 && p->head_dim != 512)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: head_dim %u (256 or 512)", fn, p->head_dim);
    if (p->kv_seq_len == 0) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: kv_seq_len is 0", fn);
    if (p->kv_capacity < p->kv_seq_len)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: kv_capacity %u < kv_seq_len %u", fn, p->kv_capacity, p->kv_seq_len);
    if (p->codebook_bits != 5 && p->codebook_bits != 6 && p->codebook_bits != 8)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: codebook_bits %u (5, 6 or 8)", fn, p->codebook_bits);
    if (p->num_kv_heads == 0 || p->num_heads == 0 || p->num_heads % p->num_kv_heads)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: %u heads over %u kv heads", fn, p->num_heads, p->num_kv_heads);
    if (p->mask_type > 2) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: mask_type %u", fn, p->mask_type);
    if (p->ring_start >= p->kv_capacity) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: ring_start %u >= capacity", fn, p->ring_start);
    if (!q || !k_codes || !k_norms || !v_codes || !v_norms || !out || !tmp)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!is_aligned(q, 16) || !is_aligned(out, 16) || !is_aligned(k_codes, 16) || !is_aligned(v_codes, 16) ||
        !is_aligned(tmp, 16))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: q / out / codes / tmp need 16-byte alignment", fn);
    // 5- and 6-bit caches store one code per byte like the 8-bit one and differ only in the centroid
    // table, which the caller supplies (its first 2^bits entries); the linear int8 map is 8-bit only.
    if (p->codebook_bits != 8 && !lut256)
        return fail(HQ_ERR_UNSUPPORTED, "%s: a %u-bit cache needs its centroid table (lut256)", fn, p->codebook_bits);
    if (tmp_bytes < tq_attn_tmp_bytes(p->num_heads, p->head_dim, p->kv_seq_len))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: tmp holds %zu bytes, %zu needed", fn, tmp_bytes,
                    tq_attn_tmp_bytes(p->num_heads, p->head_dim, p->kv_seq_len));
    return launch_tq_attention((hipStream_t)stream, q, k_codes, k_norms, v_codes, v_norms, lut256, out,
                               static_cast<float*>(tmp), *p, undo_rotation);
}

int hq_flash_attn_vec_tq(void* stream, const float* q, const uint8_t* k_codes, const float* k_norms,
                         const uint8_t* v_codes, const float* v_norms, const float* lut256, float* out,
                         void* tmp, size_t tmp_bytes, const hq_tq_attn_params* p) {
    return flash_attn_vec_tq("hq_flash_attn_vec_tq", false, stream, q, k_codes, k_norms, v_codes, v_norms, lut256, out, tmp,
                             tmp_bytes, p);
}

int hq_flash_attn_vec_tq_undo(void* stream, const float* q, const uint8_t* k_codes, const float* k_norms,
                              const uint8_t* v_codes, const float* v_norms, const float* lut256, float* out,
                              void* tmp, size_t tmp_bytes, const hq_tq_attn_params* p) {
    return flash_attn_vec_tq("hq_flash_attn_vec_tq_undo", true, stream, q, k_codes, k_norms, v_codes, v_norms, lut256, out,
                             tmp, tmp_bytes, p);
}

// Scratch of hq_flash_attn_vec_tq_static: one copy per GPU, held until the process ends.  In host code the array's
// name is only a handle for hipGetSymbolAddress; the address the kernels get is looked up once per device.
static __device__ __align__(256) unsigned char scratch[HQ_TQ_STATIC_TMP_BYTES];

static int static_scratch(void** out) {
    static std::mutex mu;
    static void* ptr[64] = {};
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (dev < 0 || dev >= 64) return fail(HQ_ERR_UNSUPPORTED, "hq_flash_attn_vec_tq_static: device ordinal %d (0..63)", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr[dev]) {
        void* p = nullptr;
        if (int rc = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(static attention scratch)"))
            return rc;
        if (!p) return fail(HQ_ERR_HIP, "hq_flash_attn_vec_tq_static: no address for the static scratch");
        ptr[dev] = p;
    }
    *out = ptr[dev];
    return HQ_OK;
}

int hq_flash_attn_vec_tq_static(void* stream, const float* q, const uint8_t* k_codes, const float* k_norms,
                                const uint8_t* v_codes, const float* v_norms, const float* lut256, float* out,
                                const hq_tq_attn_params* p, int undo_rotation) {
    const char* fn = "hq_flash_attn_vec_tq_static";
    if (!p) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null params", fn);
    // sizes first: the scratch is fixed, so the shape check does not depend on the other arguments being sane
    if ((p->head_dim == 256 || p->head_dim == 512) && p->kv_seq_len != 0) {
        const size_t need = tq_attn_tmp_bytes(p->num_heads, p->head_dim, p->kv_seq_len);
        if (need > HQ_TQ_STATIC_TMP_BYTES)
            return fail(HQ_ERR_INVALID_ARGUMENT,
                        "%s: %u heads x head_dim %u over %u positions need %zu bytes of scratch, the static buffer holds %zu; "
                        "use hq_flash_attn_vec_tq with caller scratch",
                        fn, p->num_heads, p->head_dim, p->kv_seq_len, need, (size_t)HQ_TQ_STATIC_TMP_BYTES);
    }
    void* tmp = nullptr;
    if (int rc = static_scratch(&tmp)) return rc;
    return flash_attn_vec_tq(fn, undo_rotation != 0, stream, q, k_codes, k_norms, v_codes, v_norms, lut256, out, tmp,
                             HQ_TQ_STATIC_TMP_BYTES, p);
}

int hq_dense_gemv_bf16(void* stream, const void* x, hq_act_dtype xdt, const void* w_bf16, float* y, uint32_t m,
                       uint32_t n, uint32_t k) {
    if (xdt != HQ_F32 && xdt != HQ_BF16) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_dense_gemv_bf16: activation dtype %d", (int)xdt);
    if (k == 0 || k % 8) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_dense_gemv_bf16: k %u is not a multiple of 8", k);
    if (m == 0 || n == 0) return HQ_OK;
    if (!x || !w_bf16 || !y) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_dense_gemv_bf16: null buffer");
    if (!is_aligned(x, 16) || !is_aligned(w_bf16, 16))
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_dense_gemv_bf16: x and w must be 16-byte aligned");
    if (m > 65535) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_dense_gemv_bf16: m %u too large", m);
    return launch_dense_gemv_bf16((hipStream_t)stream, x, xdt, w_bf16, y, m, n, k);
}

int hq_dense_gemv_bf16_pair(void* stream, const void* x, hq_act_dtype xdt, const void* w_a, float* y_a, uint32_t n_a,
                            const void* w_b, float* y_b, uint32_t n_b, uint32_t m, uint32_t k) {
    const char* fn = "hq_dense_gemv_bf16_pair";
    if (xdt != HQ_F32 && xdt != HQ_BF16) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: activation dtype %d", fn, (int)xdt);
    if (k == 0 || k % 8) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: k %u is not a multiple of 8", fn, k);
    if (m == 0 || (n_a == 0 && n_b == 0)) return HQ_OK;
    if (!x || (n_a && (!w_a || !y_a)) || (n_b && (!w_b || !y_b))) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!is_aligned(x, 16) || !is_aligned(w_a, 16) || !is_aligned(w_b, 16))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: x and both weight matrices must be 16-byte aligned", fn);
    if (m > 65535) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: m %u too large", fn, m);
    return launch_dense_gemv_bf16_pair((hipStream_t)stream, x, xdt, w_a, y_a, n_a, w_b, y_b, n_b, m, k);
}

int hq_moe_softmax_topk(void* stream, const float* logits, uint32_t* ids, float* weights, uint32_t n_tokens,
                        uint32_t n_experts, uint32_t top_k) {
    if (n_experts == 0 || n_experts > 1024) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_moe_softmax_topk: n_experts %u (1..1024)", n_experts);
    // ffn.rs:203-204: top-k must be positive and cannot exceed num_experts
    if (top_k == 0 || top_k > n_experts || top_k > 64)
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_moe_softmax_topk: top_k %u with %u experts (1..min(64, n_experts))", top_k, n_experts);
    if (n_tokens == 0) return HQ_OK;
    if (!logits || !ids || !weights) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_moe_softmax_topk: null buffer");
    return launch_moe_softmax_topk((hipStream_t)stream, logits, ids, weights, n_tokens, n_experts, top_k);
}

int hq_silu_mul(void* stream, const float* gate, const float* up, float* out, uint64_t n) {
    if (n % 4) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_silu_mul: n %llu is not a multiple of 4", (unsigned long long)n);
    if (n == 0) return HQ_OK;
    if (!gate || !up || !out) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_silu_mul: null buffer");
    if (!is_aligned(gate, 16) || !is_aligned(up, 16) || !is_aligned(out, 16))
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_silu_mul: buffers must be 16-byte aligned");
    return launch_silu_mul((hipStream_t)stream, gate, up, out, n);
}

int hq_moe_weighted_reduce(void* stream, const float* y, const float* w, const float* shared, const float* shared_logit,
                           const float* residual, float* out, uint32_t n_tokens, uint32_t top_k, uint32_t hidden) {
    if (hidden == 0 || hidden % 4) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_moe_weighted_reduce: hidden %u is not a multiple of 4", hidden);
    if (n_tokens == 0) return HQ_OK;
    if (n_tokens > 65535) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_moe_weighted_reduce: n_tokens %u too large", n_tokens);
    if ((top_k && (!y || !w)) || !out) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_moe_weighted_reduce: null buffer");
    if (shared_logit && !shared) return fail(HQ_ERR_INVALID_ARGUMENT, "hq_moe_weighted_reduce: shared_logit without shared");
    if (!is_aligned(y, 16) || !is_aligned(shared, 16) || !is_aligned(residual, 16) || !is_aligned(out, 16))
        return fail(HQ_ERR_INVALID_ARGUMENT, "hq_moe_weighted_reduce: buffers must be 16-byte aligned");
    return launch_moe_weighted_reduce((hipStream_t)stream, y, w, shared, shared_logit, residual, out, n_tokens, top_k, hidden);
}

}  // extern "C"

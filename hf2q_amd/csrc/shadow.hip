// The prefill product over the F16 shadow of a weight: y[m][n] = x[m][k] . W[n][k]^T with W already dequantised to f16
// (hq_dequant_ggml with HQ_F16 at load time).  Replaces the route dispatch_qmatmul takes for m > 8 when the weight has
// a shadow (src/serve/forward_mlx.rs:9790-9817 -> dispatch_mm_v2_f16: F16 weight x F32 input -> F32 output).  With the
// dequantisation out of the way this is a plain dense GEMM, which is the vendor library's business: the activations are
// cast to f16 by a small kernel here (f32 or bf16 -> f16, round to nearest even), and hipBLASLt multiplies with f32
// accumulation and f32 output.  The library is bound at load time (libhipblaslt.so.1); its handle is created once per
// device, the algorithm it picks is remembered per (m, n, k, workspace) and reused.
#include <hip/hip_fp16.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

#include "hq_internal.h"

namespace hq {
namespace {

// 8 activations per thread: two 16-byte loads (f32) or one (bf16), one 16-byte store.
template <bool X_BF16>
__global__ __launch_bounds__(256) void cast_to_f16_kernel(const void* __restrict__ x, __half* __restrict__ out, uint64_t n8) {
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= n8) return;
    float v[8];
    if constexpr (X_BF16) {
        const uint4 r = static_cast<const uint4*>(x)[i];
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = __uint_as_float(w[j] << 16);
            v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
    } else {
        const float4 a = static_cast<const float4*>(x)[2 * i], b = static_cast<const float4*>(x)[2 * i + 1];
        v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
    }
    union {
        __half h[8];
        uint4 u;
    } o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o.h[j] = __float2half_rn(v[j]);
    reinterpret_cast<uint4*>(out)[i] = o.u;
}

int check_lt(hipblasStatus_t st, const char* what) {
    if (st == HIPBLAS_STATUS_SUCCESS) return HQ_OK;
    return fail(HQ_ERR_HIP, "%s: hipBLASLt status %d", what, (int)st);
}

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t ws = 0;
};
struct PerDevice {
    hipblasLtHandle_t handle = nullptr;
    std::map<std::tuple<uint32_t, uint32_t, uint32_t, size_t, bool>, Plan> plans;  // (m, n, k, workspace, f32 operands)
};
std::mutex g_mu;
std::map<int, PerDevice> g_dev;

// The plan for (m, n, k) with at most `ws_cap` bytes of library workspace, made on first use.  Column-major reading of
// the row-major operands: D (n x m, ld n) = op_T(A = W as k x n, ld k) . (B = X as k x m, ld k).
// f32_operands: both operands f32 (weights that are stored as f32) instead of f16.
int plan_for(uint32_t m, uint32_t n, uint32_t k, size_t ws_cap, bool f32_operands, hipblasLtHandle_t* handle, Plan* out) {
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    std::lock_guard<std::mutex> lock(g_mu);
    PerDevice& pd = g_dev[dev];
    if (!pd.handle)
        if (int rc = check_lt(hipblasLtCreate(&pd.handle), "hipblasLtCreate")) return rc;
    *handle = pd.handle;
    const auto key = std::make_tuple(m, n, k, ws_cap, f32_operands);
    const hipDataType op_type = f32_operands ? HIP_R_32F : HIP_R_16F;
    auto it = pd.plans.find(key);
    if (it != pd.plans.end()) {
        *out = it->second;
        return HQ_OK;
    }
    Plan p;
    if (int rc = check_lt(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate")) return rc;
    const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    int rc = check_lt(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)), "hipblasLtMatmulDescSetAttribute(TRANSA)");
    if (!rc) rc = check_lt(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)), "hipblasLtMatmulDescSetAttribute(TRANSB)");
    if (!rc) rc = check_lt(hipblasLtMatrixLayoutCreate(&p.a, op_type, k, n, k), "hipblasLtMatrixLayoutCreate(weights)");
    if (!rc) rc = check_lt(hipblasLtMatrixLayoutCreate(&p.b, op_type, k, m, k), "hipblasLtMatrixLayoutCreate(activations)");
    if (!rc) rc = check_lt(hipblasLtMatrixLayoutCreate(&p.c, HIP_R_32F, n, m, n), "hipblasLtMatrixLayoutCreate(output)");
    hipblasLtMatmulPreference_t pref = nullptr;
    if (!rc) rc = check_lt(hipblasLtMatmulPreferenceCreate(&pref), "hipblasLtMatmulPreferenceCreate");
    if (!rc) rc = check_lt(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws_cap, sizeof(ws_cap)),
                           "hipblasLtMatmulPreferenceSetAttribute(workspace)");
    hipblasLtMatmulHeuristicResult_t res[1];
    int found = 0;
    if (!rc) rc = check_lt(hipblasLtMatmulAlgoGetHeuristic(pd.handle, p.desc, p.a, p.b, p.c, p.c, pref, 1, res, &found), "hipblasLtMatmulAlgoGetHeuristic");
    if (pref) hipblasLtMatmulPreferenceDestroy(pref);
    if (!rc && found < 1) rc = fail(HQ_ERR_UNSUPPORTED, "dense matmul: the vendor library has no %s kernel for %u x %u x %u", f32_operands ? "f32" : "f16", m, n, k);
    if (rc) {
        if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
        if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
        if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
        if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
        return rc;
    }
    p.algo = res[0].algo;
    p.ws = res[0].workspaceSize;
    pd.plans.emplace(key, p);
    *out = p;
    return HQ_OK;
}

constexpr size_t kLibraryWorkspace = 32u << 20;  // what the vendor library may use beside the f16 activations
inline size_t cast_bytes(uint32_t m, uint32_t k) { return ((size_t)m * k * 2 + 255) & ~(size_t)255; }

}  // namespace

size_t f16_shadow_workspace_bytes(uint32_t m, uint32_t k) { return cast_bytes(m, k) + kLibraryWorkspace; }

int launch_f16_shadow_matmul(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_f16, float* y, uint32_t m, uint32_t n,
                             uint32_t k, void* workspace, size_t workspace_bytes) {
    const size_t xb = cast_bytes(m, k);
    __half* xh = static_cast<__half*>(workspace);
    const uint64_t n8 = (uint64_t)m * k / 8;
    const unsigned blocks = (unsigned)((n8 + 255) / 256);
    if (xdt == HQ_BF16)
        hipLaunchKernelGGL(cast_to_f16_kernel<true>, dim3(blocks), dim3(256), 0, s, x, xh, n8);
    else
        hipLaunchKernelGGL(cast_to_f16_kernel<false>, dim3(blocks), dim3(256), 0, s, x, xh, n8);
    if (int rc = check_launch("f16 cast kernel launch")) return rc;
    const size_t ws_cap = workspace_bytes - xb;
    hipblasLtHandle_t handle = nullptr;
    Plan p;
    if (int rc = plan_for(m, n, k, ws_cap, false, &handle, &p)) return rc;
    const float alpha = 1.f, beta = 0.f;
    return check_lt(hipblasLtMatmul(handle, p.desc, &alpha, w_f16, p.a, xh, p.b, &beta, y, p.c, y, p.c, &p.algo,
                                    static_cast<uint8_t*>(workspace) + xb, ws_cap, s),
                    "hipblasLtMatmul");
}

// The same product over weights stored as f32 (dense_matmul_f32_f32_tensor, src/serve/forward_mlx.rs:9851-9866): f32
// operands, f32 accumulation.  bf16 activations are widened into the workspace first (exact).
namespace {
__global__ __launch_bounds__(256) void widen_bf16_kernel(const uint4* __restrict__ x, float4* __restrict__ out, uint64_t n8) {
    const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= n8) return;
    const uint4 r = x[i];
    out[2 * i] = make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                             __uint_as_float(r.y & 0xffff0000u));
    out[2 * i + 1] = make_float4(__uint_as_float(r.z << 16), __uint_as_float(r.z & 0xffff0000u), __uint_as_float(r.w << 16),
                                 __uint_as_float(r.w & 0xffff0000u));
}
inline size_t widen_bytes(uint32_t m, uint32_t k, hq_act_dtype xdt) { return xdt == HQ_BF16 ? ((size_t)m * k * 4 + 255) & ~(size_t)255 : 0; }
}  // namespace

size_t f32_dense_workspace_bytes(uint32_t m, uint32_t k, hq_act_dtype xdt) { return widen_bytes(m, k, xdt) + kLibraryWorkspace; }

int launch_f32_dense_matmul(hipStream_t s, const void* x, hq_act_dtype xdt, const void* w_f32, float* y, uint32_t m, uint32_t n,
                            uint32_t k, void* workspace, size_t workspace_bytes) {
    const size_t xb = widen_bytes(m, k, xdt);
    const void* xf = x;
    if (xdt == HQ_BF16) {
        const uint64_t n8 = (uint64_t)m * k / 8;
        hipLaunchKernelGGL(widen_bf16_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, s, static_cast<const uint4*>(x),
                           static_cast<float4*>(workspace), n8);
        if (int rc = check_launch("bf16 widening kernel launch")) return rc;
        xf = workspace;
    }
    const size_t ws_cap = workspace_bytes - xb;
    hipblasLtHandle_t handle = nullptr;
    Plan p;
    if (int rc = plan_for(m, n, k, ws_cap, true, &handle, &p)) return rc;
    const float alpha = 1.f, beta = 0.f;
    return check_lt(hipblasLtMatmul(handle, p.desc, &alpha, w_f32, p.a, xf, p.b, &beta, y, p.c, y, p.c, &p.algo,
                                    static_cast<uint8_t*>(workspace) + xb, ws_cap, s),
                    "hipblasLtMatmul(f32)");
}

}  // namespace hq

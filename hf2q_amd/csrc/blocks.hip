// Whole FFN blocks behind one C call each (host code only): the sequences of library calls that stand for hf2q's
// build_dense_ffn_layer_gpu_q (gpu_ffn.rs:1017-1351) and build_moe_ffn_layer_gpu_q_into (gpu_ffn.rs:2313-2802) at any
// token count, with every intermediate buffer and workspace carved out of ONE caller scratch.  Each step is a public entry
// point of this library called with the arguments a caller issuing the steps one by one would pass, so a block's result
// has the bits of that hand-written sequence.
#include "hq_internal.h"

namespace hq {
namespace {

constexpr uint32_t kDecodeRows = 8;            // up to here the GEMV routes (MM_ROUTING_THRESHOLD, forward_mlx.rs:9791)
constexpr uint32_t kFusedSwigluMaxK = 8192;    // the down GEMV that forms silu(gate) * up while it stages them: up to this k
constexpr uint32_t kRouteInLaunchMaxTokens = 4, kRouteInLaunchMaxExperts = 256;

size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }
size_t max3(size_t a, size_t b, size_t c) { return a > b ? (a > c ? a : c) : (b > c ? b : c); }

// Carves 256-byte aligned pieces off a scratch (or only adds their sizes up when base is null).
struct Carver {
    uint8_t* base;
    size_t used = 0;
    template <typename T>
    T* take(size_t count) {
        T* p = base ? reinterpret_cast<T*>(base + used) : nullptr;
        used += up256(count * sizeof(T));
        return p;
    }
    void* bytes(size_t n) { return take<uint8_t>(n); }
};



// ---- dense SwiGLU FFN ----
struct DenseBufs {
    float *gate, *up, *act;
    void* ws;
    size_t ws_bytes;
};

size_t dense_ws_bytes(uint32_t m, uint32_t hidden, uint32_t inter, hq_ggml_type tg, hq_ggml_type td, hq_act_dtype xdt) {
    return max3(hq_qmatmul_ggml_workspace_bytes(m, inter, hidden, xdt, tg), hq_qmatmul_gated_ggml_workspace_bytes(m, inter, hidden, xdt, tg),
                hq_qmatmul_ggml_workspace_bytes(m, hidden, inter, HQ_F32, td));
}

DenseBufs carve_dense(Carver& c, uint32_t m, uint32_t hidden, uint32_t inter, hq_ggml_type tg, hq_ggml_type td, hq_act_dtype xdt) {
    DenseBufs b{};
    const size_t n = (size_t)m * inter;
    b.gate = c.take<float>(n);
    b.up = c.take<float>(n);
    b.act = c.take<float>(n);
    b.ws_bytes = dense_ws_bytes(m, hidden, inter, tg, td, xdt);
    b.ws = b.ws_bytes ? c.bytes(b.ws_bytes) : nullptr;
    return b;
}

int dense_ffn_steps(void* stream, const void* x, hq_act_dtype xdt, const void* wg, const void* wu, const void* wd, hq_ggml_type tg,
                    hq_ggml_type td, const float* sg, const float* su, const float* sd, float* out, uint32_t m, uint32_t hidden,
                    uint32_t inter, const DenseBufs& b) {
    if (m <= kDecodeRows) {
        // decode: gate + up + SwiGLU as one launch per row where the streaming GEMV takes the pair, else gate and up as one
        // batched launch; then down (with the SwiGLU folded into its staging where that pays)
        if (hq_qmatmul_swiglu_decode_supported(inter, hidden, tg, xdt)) {
            if (int rc = hq_qmatmul_swiglu_decode(stream, x, xdt, wg, wu, b.act, m, inter, hidden, tg)) return rc;
            return hq_qmatmul_ggml(stream, b.act, HQ_F32, wd, out, m, hidden, inter, td);
        }
        hq_qmatmul_job jobs[2] = {};
        jobs[0].x = jobs[1].x = x;
        jobs[0].w = wg;
        jobs[1].w = wu;
        jobs[0].y = b.gate;
        jobs[1].y = b.up;
        jobs[0].rows = jobs[1].rows = m;
        jobs[0].n = jobs[1].n = inter;
        jobs[0].k = jobs[1].k = hidden;
        if (int rc = hq_qmatmul_batch_ggml(stream, jobs, 2, xdt, tg)) return rc;
        if (inter <= kFusedSwigluMaxK) {
            hq_qmatmul_job dn = {};
            dn.x = b.gate;
            dn.x_up = b.up;
            dn.w = wd;
            dn.y = out;
            dn.rows = m;
            dn.n = hidden;
            dn.k = inter;
            return hq_qmatmul_batch_ggml(stream, &dn, 1, HQ_F32, td);
        }
        if (int rc = hq_silu_mul(stream, b.gate, b.up, b.act, (uint64_t)m * inter)) return rc;
        return hq_qmatmul_ggml(stream, b.act, HQ_F32, wd, out, m, hidden, inter, td);
    }
    // prefill: gate, then the up projection finishing the gating in its epilogue where the tile route offers that, then down
    auto mm = [&](const void* xin, hq_act_dtype dt, const void* w, const float* sc, float* y, uint32_t n, uint32_t k, hq_ggml_type t) {
        return sc ? hq_qmatmul_ggml_ws_prepared(stream, xin, dt, w, sc, y, m, n, k, t, b.ws, b.ws_bytes)
                  : hq_qmatmul_ggml_ws(stream, xin, dt, w, y, m, n, k, t, b.ws, b.ws_bytes);
    };
    if (int rc = mm(x, xdt, wg, sg, b.gate, inter, hidden, tg)) return rc;
    if (hq_qmatmul_gated_ggml_workspace_bytes(m, inter, hidden, xdt, tg)) {
        if (int rc = hq_qmatmul_gated_ggml_ws(stream, x, xdt, wu, su, b.gate, b.act, m, inter, hidden, tg, b.ws, b.ws_bytes)) return rc;
    } else {
        if (int rc = mm(x, xdt, wu, su, b.up, inter, hidden, tg)) return rc;
        if (int rc = hq_silu_mul(stream, b.gate, b.up, b.act, (uint64_t)m * inter)) return rc;
    }
    return mm(b.act, HQ_F32, wd, sd, out, hidden, inter, td);
}

int check_dense(const char* fn, uint32_t hidden, uint32_t inter, hq_ggml_type tg, hq_ggml_type td, hq_act_dtype xdt) {
    if (!hq_block_elems(tg) || !hq_block_elems(td)) return fail(HQ_ERR_UNSUPPORTED, "%s: ggml types %d / %d", fn, (int)tg, (int)td);
    if (xdt != HQ_F32 && xdt != HQ_BF16) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: activation dtype %d", fn, (int)xdt);
    if (hidden == 0 || inter == 0 || hidden % hq_block_elems(tg) || inter % hq_block_elems(td) || inter % 4)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: hidden %u / inter %u are not whole blocks of types %d / %d", fn, hidden, inter, (int)tg, (int)td);
    return HQ_OK;
}

// ---- MoE FFN ----
struct MoeBufs {
    float *logits, *sh_logit, *topk_w, *gate, *up, *act, *down, *sh_gate, *sh_up, *sh_act, *sh_down;
    uint32_t* ids;
    void *id_ws, *dense_ws;
    size_t id_ws_bytes, dense_ws_bytes;
};

hq_ggml_type down_type(const hq_moe_ffn_layer& l) { return l.down_type ? (hq_ggml_type)l.down_type : l.ggml_type; }

MoeBufs carve_moe(Carver& c, const hq_moe_ffn_layer& l, uint32_t T, hq_act_dtype xdt) {
    MoeBufs b{};
    const uint32_t K = l.top_k, E = l.n_experts, H = l.hidden, I = l.inter, SI = l.shared_inter;
    const hq_ggml_type t = l.ggml_type, td = down_type(l);
    const size_t TK = (size_t)T * K;
    b.logits = c.take<float>((size_t)T * E);
    b.sh_logit = c.take<float>(T);
    b.ids = c.take<uint32_t>(TK);
    b.topk_w = c.take<float>(TK);
    b.gate = c.take<float>(TK * I);
    b.up = c.take<float>(TK * I);
    b.act = c.take<float>(TK * I);
    b.down = c.take<float>(TK * H);
    b.sh_gate = c.take<float>((size_t)T * SI);
    b.sh_up = c.take<float>((size_t)T * SI);
    b.sh_act = c.take<float>((size_t)T * SI);
    b.sh_down = c.take<float>((size_t)T * H);
    b.id_ws_bytes = max3(hq_qmatmul_id_swiglu_ggml_workspace_bytes(T, K, I, H, E, l.expert_stride_gate_up, t),
                         hq_qmatmul_id_ggml_workspace_bytes(T, K, I, H, E, l.expert_stride_gate_up, t),
                         hq_qmatmul_id_ggml_workspace_bytes((uint32_t)TK, 1, H, I, E, l.expert_stride_down, td));
    b.id_ws = b.id_ws_bytes ? c.bytes(b.id_ws_bytes) : nullptr;
    b.dense_ws_bytes = max3(hq_qmatmul_swiglu_ggml_workspace_bytes(T, SI, H, xdt, t), hq_qmatmul_ggml_workspace_bytes(T, SI, H, xdt, t),
                            hq_qmatmul_ggml_workspace_bytes(T, H, SI, HQ_F32, td));
    b.dense_ws = b.dense_ws_bytes ? c.bytes(b.dense_ws_bytes) : nullptr;
    return b;
}

int check_moe(const char* fn, const hq_moe_ffn_layer* l, uint32_t T, hq_act_dtype xdt) {
    if (!l) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null layer", fn);
    const hq_ggml_type t = l->ggml_type, td = down_type(*l);
    if (!hq_block_elems(t) || !hq_block_elems(td)) return fail(HQ_ERR_UNSUPPORTED, "%s: ggml types %d / %d", fn, (int)t, (int)td);
    if (xdt != HQ_F32 && xdt != HQ_BF16) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: activation dtype %d", fn, (int)xdt);
    if (l->hidden == 0 || l->inter == 0 || l->shared_inter == 0 || l->hidden % hq_block_elems(t) || l->hidden % 8 || l->inter % hq_block_elems(td) ||
        l->shared_inter % hq_block_elems(td) || l->inter % 4 || l->shared_inter % 4)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: hidden %u / inter %u / shared inter %u are not whole blocks of types %d / %d", fn, l->hidden,
                    l->inter, l->shared_inter, (int)t, (int)td);
    if (l->n_experts == 0 || l->n_experts > 1024 || l->top_k == 0 || l->top_k > l->n_experts || l->top_k > 64)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: top-%u of %u experts", fn, l->top_k, l->n_experts);
    if ((uint64_t)T * l->top_k > 0x7fffffffull) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: %u tokens x top-%u", fn, T, l->top_k);
    return HQ_OK;
}

int moe_steps(void* stream, const hq_moe_ffn_layer& l, const hq_moe_ffn_row_scales* rs, const void* x, hq_act_dtype xdt, const float* residual,
              float* out, uint32_t T, const MoeBufs& b) {
    const uint32_t K = l.top_k, E = l.n_experts, H = l.hidden, I = l.inter, SI = l.shared_inter, TK = T * K;
    const hq_ggml_type t = l.ggml_type, td = down_type(l);
    const float* no = nullptr;
    const float *rs_eg = rs ? rs->expert_gate : no, *rs_eu = rs ? rs->expert_up : no, *rs_ed = rs ? rs->expert_down : no;
    const float *rs_sg = rs ? rs->shared_gate : no, *rs_su = rs ? rs->shared_up : no, *rs_sd = rs ? rs->shared_down : no;
    const float* sh_logit = l.shared_gate_logit ? b.sh_logit : nullptr;
    if (T <= kDecodeRows) {
        // decode-sized: the dispatches of a phase that the reference encodes without a barrier between them as one launch
        // each (gpu_ffn.rs:2485, 2546), the SwiGLU passes folded into the staging of the down projections
        if (l.shared_gate_logit) {
            if (int rc = hq_dense_gemv_bf16_pair(stream, x, xdt, l.router, b.logits, E, l.shared_gate_logit, b.sh_logit, 1, T, H)) return rc;
        } else if (int rc = hq_dense_gemv_bf16(stream, x, xdt, l.router, b.logits, T, E, H)) {
            return rc;
        }
        hq_qmatmul_job j[4] = {};
        const bool route_in_launch = T <= kRouteInLaunchMaxTokens && E <= kRouteInLaunchMaxExperts;
        if (!route_in_launch)
            if (int rc = hq_moe_softmax_topk(stream, b.logits, b.ids, b.topk_w, T, E, K)) return rc;
        for (int i = 0; i < 2; ++i) {
            j[i].x = x;
            j[i].w = i ? l.expert_up : l.expert_gate;
            j[i].y = i ? b.up : b.gate;
            j[i].rows = T;
            j[i].top_k = K;
            j[i].n = I;
            j[i].k = H;
            j[i].n_experts = E;
            j[i].expert_stride = l.expert_stride_gate_up;
            if (route_in_launch)
                j[i].route_logits = b.logits;
            else
                j[i].ids = b.ids;
        }
        if (route_in_launch) {
            j[0].route_ids = b.ids;
            j[0].route_weights = b.topk_w;
        }
        for (int i = 2; i < 4; ++i) {
            j[i].x = x;
            j[i].w = i == 3 ? l.shared_up : l.shared_gate;
            j[i].y = i == 3 ? b.sh_up : b.sh_gate;
            j[i].rows = T;
            j[i].n = SI;
            j[i].k = H;
        }
        if (int rc = hq_qmatmul_batch_ggml(stream, j, 4, xdt, t)) return rc;
        hq_qmatmul_job d[2] = {};
        d[0].x = b.gate;
        d[0].x_up = b.up;
        d[0].w = l.expert_down;
        d[0].ids = b.ids;
        d[0].y = b.down;
        d[0].rows = TK;
        d[0].top_k = 1;
        d[0].n = H;
        d[0].k = I;
        d[0].n_experts = E;
        d[0].expert_stride = l.expert_stride_down;
        d[1].x = b.sh_gate;
        d[1].x_up = b.sh_up;
        d[1].w = l.shared_down;
        d[1].y = b.sh_down;
        d[1].rows = T;
        d[1].n = H;
        d[1].k = SI;
        if (int rc = hq_qmatmul_batch_ggml(stream, d, 2, HQ_F32, td)) return rc;
        return hq_moe_weighted_reduce(stream, b.down, b.topk_w, b.sh_down, sh_logit, residual, out, T, K, H);
    }
    // A: router and shared-gate logits
    if (int rc = hq_dense_gemv_bf16(stream, x, xdt, l.router, b.logits, T, E, H)) return rc;
    if (l.shared_gate_logit)
        if (int rc = hq_dense_gemv_bf16(stream, x, xdt, l.shared_gate_logit, b.sh_logit, T, 1, H)) return rc;
    const bool shared_one_call = b.dense_ws && hq_qmatmul_swiglu_ggml_workspace_bytes(T, SI, H, xdt, t) > 0;
    auto mm = [&](const void* xin, hq_act_dtype dt, const void* w, const float* sc, float* y, uint32_t n, uint32_t k, hq_ggml_type ty) {
        return sc ? hq_qmatmul_ggml_ws_prepared(stream, xin, dt, w, sc, y, T, n, k, ty, b.dense_ws, b.dense_ws_bytes)
                  : hq_qmatmul_ggml_ws(stream, xin, dt, w, y, T, n, k, ty, b.dense_ws, b.dense_ws_bytes);
    };
    if (shared_one_call) {
        const bool both = rs_sg && rs_su;
        if (int rc = hq_qmatmul_swiglu_ggml_ws(stream, x, xdt, l.shared_gate, l.shared_up, both ? rs_sg : no, both ? rs_su : no, b.sh_act, T, SI, H, t,
                                               b.dense_ws, b.dense_ws_bytes))
            return rc;
    } else {
        if (int rc = mm(x, xdt, l.shared_gate, rs_sg, b.sh_gate, SI, H, t)) return rc;
        if (int rc = mm(x, xdt, l.shared_up, rs_su, b.sh_up, SI, H, t)) return rc;
    }
    // B: routing (and the shared expert's SwiGLU)
    if (int rc = hq_moe_softmax_topk(stream, b.logits, b.ids, b.topk_w, T, E, K)) return rc;
    if (!shared_one_call)
        if (int rc = hq_silu_mul(stream, b.sh_gate, b.sh_up, b.sh_act, (uint64_t)T * SI)) return rc;
    // C, D: gate, up and SwiGLU of the routed experts
    auto mm_id = [&](const void* xin, hq_act_dtype dt, const void* w, const float* sc, float* y, uint32_t nt, uint32_t k_top, uint32_t n, uint32_t k,
                     uint64_t stride, hq_ggml_type ty) {
        return sc ? hq_qmatmul_id_ggml_prepared(stream, xin, dt, w, sc, b.ids, y, b.id_ws, b.id_ws_bytes, nt, k_top, n, k, E, stride, ty)
                  : hq_qmatmul_id_ggml(stream, xin, dt, w, b.ids, y, b.id_ws, b.id_ws_bytes, nt, k_top, n, k, E, stride, ty);
    };
    if (b.id_ws && hq_qmatmul_id_swiglu_ggml_workspace_bytes(T, K, I, H, E, l.expert_stride_gate_up, t)) {
        const bool both = rs_eg && rs_eu;
        if (int rc = hq_qmatmul_id_swiglu_ggml(stream, x, xdt, l.expert_gate, l.expert_up, both ? rs_eg : no, both ? rs_eu : no, b.ids, b.act, b.id_ws,
                                               b.id_ws_bytes, T, K, I, H, E, l.expert_stride_gate_up, t))
            return rc;
    } else {
        if (int rc = mm_id(x, xdt, l.expert_gate, rs_eg, b.gate, T, K, I, H, l.expert_stride_gate_up, t)) return rc;
        if (int rc = mm_id(x, xdt, l.expert_up, rs_eu, b.up, T, K, I, H, l.expert_stride_gate_up, t)) return rc;
        if (int rc = hq_silu_mul(stream, b.gate, b.up, b.act, (uint64_t)TK * I)) return rc;
    }
    if (int rc = mm(b.sh_act, HQ_F32, l.shared_down, rs_sd, b.sh_down, H, SI, td)) return rc;
    // E: the down projection of every routed row (n_tokens = T * K, top_k = 1)
    if (int rc = mm_id(b.act, HQ_F32, l.expert_down, rs_ed, b.down, TK, 1, H, I, l.expert_stride_down, td)) return rc;
    // F
    return hq_moe_weighted_reduce(stream, b.down, b.topk_w, b.sh_down, sh_logit, residual, out, T, K, H);
}

}  // namespace
}  // namespace hq

using namespace hq;

extern "C" {

size_t hq_dense_ffn_scratch_bytes(uint32_t m, uint32_t hidden, uint32_t inter, hq_ggml_type t_gate_up, hq_ggml_type t_down, hq_act_dtype xdt) {
    if (m == 0 || check_dense("hq_dense_ffn_scratch_bytes", hidden, inter, t_gate_up, t_down, xdt)) return 0;
    Carver c{nullptr};
    carve_dense(c, m, hidden, inter, t_gate_up, t_down, xdt);
    return c.used;
}

int hq_dense_ffn(void* stream, const void* x, hq_act_dtype xdt, const void* w_gate, const void* w_up, const void* w_down, hq_ggml_type t_gate_up,
                 hq_ggml_type t_down, const float* gate_row_scales, const float* up_row_scales, const float* down_row_scales, float* out,
                 uint32_t m, uint32_t hidden, uint32_t inter, void* scratch, size_t scratch_bytes) {
    const char* fn = "hq_dense_ffn";
    if (int rc = check_dense(fn, hidden, inter, t_gate_up, t_down, xdt)) return rc;
    if (m == 0) return HQ_OK;
    if (!x || !w_gate || !w_up || !w_down || !out || !scratch) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!is_aligned(scratch, 256)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch must be 256-byte aligned", fn);
    Carver c{static_cast<uint8_t*>(scratch)};
    const DenseBufs b = carve_dense(c, m, hidden, inter, t_gate_up, t_down, xdt);
    if (scratch_bytes < c.used) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch of %zu bytes, %zu needed", fn, scratch_bytes, c.used);
    return dense_ffn_steps(stream, x, xdt, w_gate, w_up, w_down, t_gate_up, t_down, gate_row_scales, up_row_scales, down_row_scales, out, m, hidden,
                           inter, b);
}

size_t hq_moe_ffn_prefill_scratch_bytes(const hq_moe_ffn_layer* layer, uint32_t n_tokens, hq_act_dtype xdt) {
    if (n_tokens == 0 || check_moe("hq_moe_ffn_prefill_scratch_bytes", layer, n_tokens, xdt)) return 0;
    Carver c{nullptr};
    carve_moe(c, *layer, n_tokens, xdt);
    return c.used;
}

int hq_moe_ffn_prefill(void* stream, const hq_moe_ffn_layer* layer, const hq_moe_ffn_row_scales* row_scales, const void* x, hq_act_dtype xdt,
                       const float* residual, float* out, uint32_t n_tokens, void* scratch, size_t scratch_bytes, uint32_t* route_ids,
                       float* route_weights) {
    const char* fn = "hq_moe_ffn_prefill";
    if (int rc = check_moe(fn, layer, n_tokens, xdt)) return rc;
    if (n_tokens == 0) return HQ_OK;
    if (!x || !out || !scratch || !layer->router || !layer->expert_gate || !layer->expert_up || !layer->expert_down || !layer->shared_gate ||
        !layer->shared_up || !layer->shared_down)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (!route_ids != !route_weights) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: route_ids and route_weights go together", fn);
    if (!is_aligned(scratch, 256)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch must be 256-byte aligned", fn);
    Carver c{static_cast<uint8_t*>(scratch)};
    const MoeBufs b = carve_moe(c, *layer, n_tokens, xdt);
    if (scratch_bytes < c.used) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: scratch of %zu bytes, %zu needed", fn, scratch_bytes, c.used);
    if (int rc = moe_steps(stream, *layer, row_scales, x, xdt, residual, out, n_tokens, b)) return rc;
    if (route_ids) {
        const size_t n = (size_t)n_tokens * layer->top_k * 4;
        if (int rc = check_hip(hipMemcpyAsync(route_ids, b.ids, n, hipMemcpyDeviceToDevice, (hipStream_t)stream), "hipMemcpyAsync(route ids)")) return rc;
        if (int rc = check_hip(hipMemcpyAsync(route_weights, b.topk_w, n, hipMemcpyDeviceToDevice, (hipStream_t)stream), "hipMemcpyAsync(route weights)"))
            return rc;
    }
    return HQ_OK;
}

}  // extern "C"

/*
 * hf2q_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, scalar CPU restatement of the arithmetic hf2q defines for its
 * quantized-matmul hot path.  It exists only so that tests, the smoke check and
 * the CPU-baseline leg of the benchmark have something independent to compare
 * the HIP kernels with.  Nothing in the shipped library links or calls it.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (see oracle/Makefile).
 * -ffp-contract=off is REQUIRED: the reference fuses multiply-adds only at the
 * sites where it writes `mul_add` explicitly; here those are `fmaf`.
 *
 * Each function cites the reference file:line it follows (paths relative to
 * the hf2q source tree).
 *
 * How each function is pinned (what a wrong sign / index / dropped term trips):
 *   quantize_q4_k / q6_k / q8_0 / q5_k / q4_0 .... byte equality with the
 *       reference's committed golden files tests/fixtures/ggml_quants/{q4_k_512,
 *       q6_k_512,q8_0_64,q5_k_512,q4_0_64}_{noim,im}_{input,expected}.bin
 *       (tests/test_oracle_golden.py).
 *   nearest_int ..................... the RNE table of common.rs:525-539.
 *   dequantize_* .................... exact-rational evaluation of the block
 *       formula rounded once to f32 (Python fractions), RMSE of the golden
 *       blocks against their inputs, re-quantisation idempotence.
 *   gemv_f32 / gemm_f64 ............. numpy float64 matmul.
 *   softmax_topk_renorm, moe_ffn .... known-answer cases of gpu_ffn.rs:3577-3593
 *       and ffn.rs tests, numpy restatement, shared-gate linearity.
 *   fwht / sign tables .............. H*H = I, rotation preserves dot products,
 *       explicit 256x256 Sylvester matrix product.
 *   tq_encode_int8 / tq_attention ... kv_seq_len=1 closed form out[h]=V[kv(h)],
 *       numpy float64 softmax attention, byte count 34,078,720 of the 32K cache.
 *   The Lloyd-Max 8-bit centroid table of the reference's third-party GPU crate
 *   (mlx-native 0.9.1, turboquant.rs, not in the tree) is PARITY UNPINNED: the
 *   oracle only implements the generic code->value LUT form, plus the linear
 *   int8 map the benchmark configuration names.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QK_K 256
#define K_SCALE_SIZE 12
#define Q4K_BYTES 144
#define Q6K_BYTES 210
#define QK8_0 32
#define Q8_0_BYTES 34
#define Q5K_BYTES 176
#define QK4_0 32
#define Q4_0_BYTES 18
#define GROUP_MAX_EPS 1e-15f /* common.rs:15 */

/* ------------------------------------------------------------------ */
/* f16 <-> f32 (IEEE binary16, round-to-nearest-even), as the `half`   */
/* crate's f16::from_f32 / to_f32 used at q4_k.rs:178-184.            */
/* ------------------------------------------------------------------ */
static uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 0xFF) { /* inf / nan */
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        return (uint16_t)(sign | 0x7E00u | (man >> 13));
    }
    int e = (int)exp - 127 + 15;
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
    if (e <= 0) {                                      /* subnormal or zero */
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        int shift = 14 - e; /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++; /* may carry into exp: correct */
    return (uint16_t)(sign | half);
}

static float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                e++;
                man <<= 1;
            } while ((man & 0x400u) == 0);
            man &= 0x3FFu;
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 0x1F) {
        x = sign | 0x7F800000u | (man << 13);
    } else {
        x = sign | ((exp - 15 + 127) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

uint16_t hq_oracle_f32_to_f16(float f) { return f32_to_f16_bits(f); }
float hq_oracle_f16_to_f32(uint16_t h) { return f16_bits_to_f32(h); }

/* bf16 -> f32 is exact (bf16 is the top half of an f32). */
static float bf16_bits_to_f32(uint16_t b) {
    uint32_t x = (uint32_t)b << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* common.rs:23-28 nearest_int: the 2^23+2^22 magic-add, round-half-even. */
static int nearest_int(float fval) {
    float val = fval + 12582912.0f;
    int32_t i;
    memcpy(&i, &val, 4);
    return (i & 0x007fffff) - 0x00400000;
}
int hq_oracle_nearest_int(float f) { return nearest_int(f); }

static int imax(int a, int b) { return a > b ? a : b; }
static int imin(int a, int b) { return a < b ? a : b; }

/* common.rs:61-167 make_qx_quants (rmse_type>=0 callers only: Q6_K uses 1). */
static float make_qx_quants(int n, int nmax, const float *x, int8_t *L, int rmse_type,
                            const float *qw) {
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (amax < GROUP_MAX_EPS) {
        for (int i = 0; i < n; i++) L[i] = 0;
        return 0.0f;
    }
    float nmax_f = (float)nmax;
    float iscale = -nmax_f / max;
    if (rmse_type == 0) {
        for (int i = 0; i < n; i++) {
            int li = nearest_int(iscale * x[i]);
            L[i] = (int8_t)(nmax + imax(-nmax, imin(nmax - 1, li)));
        }
        return 1.0f / iscale;
    }
    int return_early = 0;
    if (rmse_type < 0) {
        rmse_type = -rmse_type;
        return_early = 1;
    }
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int li = nearest_int(iscale * x[i]);
        li = imax(-nmax, imin(nmax - 1, li));
        L[i] = (int8_t)(li + nmax);
        float w = qw ? qw[i]
                     : rmse_type == 1 ? x[i] * x[i]
                     : rmse_type == 2 ? 1.0f
                     : rmse_type == 3 ? fabsf(x[i])
                                      : sqrtf(fabsf(x[i]));
        sumlx = fmaf(w * x[i], (float)li, sumlx);      /* common.rs:120 */
        suml2 = fmaf(w * (float)li, (float)li, suml2); /* common.rs:121 */
    }
    float scale = suml2 != 0.0f ? sumlx / suml2 : 0.0f;
    if (return_early) return suml2 > 0.0f ? 0.5f * (scale + 1.0f / iscale) : 1.0f / iscale;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; is++) {
        if (is == 0) continue;
        iscale = -(nmax_f + 0.1f * (float)is) / max;
        sumlx = 0.0f;
        suml2 = 0.0f;
        for (int i = 0; i < n; i++) {
            int li = nearest_int(iscale * x[i]);
            li = imax(-nmax, imin(nmax - 1, li));
            float w = qw ? qw[i]
                         : rmse_type == 1 ? x[i] * x[i]
                         : rmse_type == 2 ? 1.0f
                         : rmse_type == 3 ? fabsf(x[i])
                                          : sqrtf(fabsf(x[i]));
            sumlx = fmaf(w * x[i], (float)li, sumlx);
            suml2 = fmaf(w * (float)li, (float)li, suml2);
        }
        if (suml2 > 0.0f && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; i++) {
                int li = nearest_int(iscale * x[i]);
                L[i] = (int8_t)(nmax + imax(-nmax, imin(nmax - 1, li)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

/* common.rs:174-286 make_qkx2_quants (weights mandatory) and
 * common.rs:294-408 make_qkx3_quants (weights optional, `max <= min` early out).
 * `variant3` selects the second form. */
static float make_qkx_quants(int variant3, int n, int nmax, const float *x, const float *weights,
                             uint8_t *L, float *the_min, uint8_t *Laux, float rmin, float rdelta,
                             int nstep, int use_mad) {
    float min = x[0], max = x[0];
    float sum_w = weights ? weights[0] : x[0] * x[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        float w = weights ? weights[i] : x[i] * x[i];
        sum_w += w;
        sum_x = fmaf(w, x[i], sum_x); /* common.rs:212 */
    }
    if (min > 0.0f) min = 0.0f;
    if (variant3 ? (max <= min) : (max == min)) { /* common.rs:218 / :331 */
        for (int i = 0; i < n; i++) L[i] = 0;
        *the_min = -min;
        return 0.0f;
    }
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    float best_error = 0.0f;
    for (int i = 0; i < n; i++) {
        int l = nearest_int(iscale * (x[i] - min));
        L[i] = (uint8_t)imax(0, imin(nmax, l));
        float diff = fmaf(scale, (float)L[i], min) - x[i]; /* common.rs:234 */
        diff = use_mad ? fabsf(diff) : diff * diff;
        float w = weights ? weights[i] : x[i] * x[i];
        best_error = fmaf(w, diff, best_error); /* common.rs:236 */
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * (float)is + (float)nmax) / (max - min);
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_xl = 0.0f;
        for (int i = 0; i < n; i++) {
            int l = nearest_int(iscale * (x[i] - min));
            l = imax(0, imin(nmax, l));
            Laux[i] = (uint8_t)l;
            float w = weights ? weights[i] : x[i] * x[i];
            float lf = (float)l;
            sum_l = fmaf(w, lf, sum_l);         /* common.rs:253 */
            sum_l2 = fmaf(w * lf, lf, sum_l2);  /* common.rs:254 */
            sum_xl = fmaf(w * lf, x[i], sum_xl); /* common.rs:255 */
        }
        float D = fmaf(sum_w, sum_l2, -sum_l * sum_l); /* common.rs:260 */
        if (D > 0.0f) {
            float this_scale = fmaf(sum_w, sum_xl, -sum_x * sum_l) / D;
            float this_min = fmaf(sum_l2, sum_x, -sum_l * sum_xl) / D;
            if (this_min > 0.0f) {
                this_min = 0.0f;
                this_scale = sum_xl / sum_l2;
            }
            float cur_error = 0.0f;
            for (int i = 0; i < n; i++) {
                float diff = fmaf(this_scale, (float)Laux[i], this_min) - x[i];
                diff = use_mad ? fabsf(diff) : diff * diff;
                float w = weights ? weights[i] : x[i] * x[i];
                cur_error = fmaf(w, diff, cur_error);
            }
            if (cur_error < best_error) {
                for (int i = 0; i < n; i++) L[i] = Laux[i];
                best_error = cur_error;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

/* common.rs:415-518 make_qp_quants. */
static float make_qp_quants(int n, int nmax, const float *x, uint8_t *L, const float *qw) {
    float max = 0.0f;
    for (int i = 0; i < n; i++)
        if (x[i] > max) max = x[i];
    if (max < GROUP_MAX_EPS) {
        for (int i = 0; i < n; i++) L[i] = 0;
        return 0.0f;
    }
    float iscale = (float)nmax / max;
    for (int i = 0; i < n; i++) L[i] = (uint8_t)nearest_int(iscale * x[i]);
    float scale = 1.0f / iscale;
    float best_mse = 0.0f;
    for (int i = 0; i < n; i++) {
        float diff = fmaf(scale, -(float)L[i], x[i]);
        best_mse = fmaf(qw[i] * diff, diff, best_mse);
    }
    for (int is = -4; is <= 4; is++) {
        if (is == 0) continue;
        float iscale_is = (0.1f * (float)is + (float)nmax) / max;
        float scale_is = 1.0f / iscale_is;
        float mse = 0.0f;
        for (int i = 0; i < n; i++) {
            int l = nearest_int(iscale_is * x[i]);
            if (l > nmax) l = nmax;
            float diff = fmaf(scale_is, -(float)l, x[i]);
            mse = fmaf(qw[i] * diff, diff, mse);
        }
        if (mse < best_mse) {
            best_mse = mse;
            iscale = iscale_is;
        }
    }
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int l = nearest_int(iscale * x[i]);
        if (l > nmax) l = nmax;
        L[i] = (uint8_t)l;
        float w = qw[i];
        sumlx = fmaf(w * x[i], (float)l, sumlx);
        suml2 = fmaf(w * (float)l, (float)l, suml2);
    }
    for (int itry = 0; itry < 5; itry++) {
        int n_changed = 0;
        for (int i = 0; i < n; i++) {
            float w = qw[i];
            float cur_l = (float)L[i];
            float slx = fmaf(w * x[i], -cur_l, sumlx);
            float sl2 = fmaf(w * cur_l, -cur_l, suml2);
            if (slx > 0.0f && sl2 > 0.0f) {
                int new_l = nearest_int(x[i] * sl2 / slx);
                if (new_l > nmax) new_l = nmax;
                if ((uint8_t)new_l != L[i]) {
                    slx = fmaf(w * x[i], (float)new_l, slx);
                    sl2 = fmaf(w * (float)new_l, (float)new_l, sl2);
                    if (slx * slx * suml2 > sumlx * sumlx * sl2) {
                        L[i] = (uint8_t)new_l;
                        sumlx = slx;
                        suml2 = sl2;
                        n_changed++;
                    }
                }
            }
        }
        if (!n_changed) break;
    }
    return suml2 > 0.0f ? sumlx / suml2 : 0.0f;
}

/* q4_k.rs:329-337 get_scale_min_k4. */
static void get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* q4_k.rs:89-217 (quantize_row_ref) and :220-324 (quantize_row_impl), one
 * super-block.  `qw` is the imatrix slice for this block or NULL. */
static void q4k_quantize_block(const float *xb, const float *qw, uint8_t *out) {
    uint8_t L[QK_K], Laux[32], ls_arr[8], lm_arr[8];
    float weights[32], mins[8], scales[8], sw[8];
    uint8_t packed[K_SCALE_SIZE];
    memset(packed, 0, sizeof packed);
    float d_blk, dmin_blk;

    if (!qw) {
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) {
            const float *sub = xb + 32 * j;
            float sum_x2 = 0.0f;
            for (int l = 0; l < 32; l++) sum_x2 = fmaf(sub[l], sub[l], sum_x2); /* q4_k.rs:113 */
            float av_x = sqrtf(sum_x2 / 32.0f);
            for (int l = 0; l < 32; l++) weights[l] = av_x + fabsf(sub[l]);
            scales[j] = make_qkx_quants(0, 32, 15, sub, weights, L + 32 * j, &mins[j], Laux, -1.0f,
                                        0.1f, 20, 0);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)nearest_int(inv_scale * scales[j]);
            uint8_t lm = (uint8_t)nearest_int(inv_min * mins[j]);
            ls_arr[j] = ls > 63 ? 63 : ls;
            lm_arr[j] = lm > 63 ? 63 : lm;
        }
        d_blk = max_scale / 63.0f;
        dmin_blk = max_min / 63.0f;
    } else {
        float sum_x2 = 0.0f;
        for (int l = 0; l < QK_K; l++) sum_x2 = fmaf(xb[l], xb[l], sum_x2); /* q4_k.rs:240 */
        float sigma2 = 2.0f * sum_x2 / (float)QK_K;
        for (int j = 0; j < 8; j++) {
            const float *sub = xb + 32 * j;
            for (int l = 0; l < 32; l++) weights[l] = qw[32 * j + l] * sqrtf(sigma2 + sub[l] * sub[l]);
            float sumw = 0.0f;
            for (int l = 0; l < 32; l++) sumw += weights[l];
            sw[j] = sumw;
            scales[j] = make_qkx_quants(1, 32, 15, sub, weights, L + 32 * j, &mins[j], Laux, -0.9f,
                                        0.05f, 36, 0);
        }
        d_blk = make_qp_quants(8, 63, scales, ls_arr, sw);
        dmin_blk = make_qp_quants(8, 63, mins, lm_arr, sw);
    }
    for (int j = 0; j < 8; j++) { /* q4_k.rs:166-173 */
        uint8_t ls = ls_arr[j], lm = lm_arr[j];
        if (j < 4) {
            packed[j] = ls;
            packed[j + 4] = lm;
        } else {
            packed[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            packed[j - 4] |= (uint8_t)((ls >> 4) << 6);
            packed[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    uint16_t d16 = f32_to_f16_bits(d_blk), dmin16 = f32_to_f16_bits(dmin_blk);
    float d_dq = f16_bits_to_f32(d16), dmin_dq = f16_bits_to_f32(dmin16);
    for (int j = 0; j < 8; j++) { /* q4_k.rs:185-197 */
        uint8_t sc, m;
        get_scale_min_k4(j, packed, &sc, &m);
        float d = d_dq * (float)sc;
        if (d == 0.0f) continue;
        float dm = dmin_dq * (float)m;
        for (int ii = 0; ii < 32; ii++) {
            int l = nearest_int((xb[32 * j + ii] + dm) / d);
            L[32 * j + ii] = (uint8_t)imax(0, imin(15, l));
        }
    }
    out[0] = (uint8_t)(d16 & 0xFF);
    out[1] = (uint8_t)(d16 >> 8);
    out[2] = (uint8_t)(dmin16 & 0xFF);
    out[3] = (uint8_t)(dmin16 >> 8);
    memcpy(out + 4, packed, K_SCALE_SIZE);
    uint8_t *q = out + 16;
    for (int j = 0; j < QK_K; j += 64)
        for (int l = 0; l < 32; l++) *q++ = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
}

/* q5_k.rs:160-243 (quantize_row_q5_k_ref) and :246-311 (quantize_row_q5_k_impl) with the common
 * tail finalize_block (q5_k.rs:88-157), one super-block.  `qw` is the imatrix slice or NULL. */
static void q5k_quantize_block(const float *xb, const float *qw, uint8_t *out) {
    uint8_t L[QK_K], Laux[32], ls_arr[8], lm_arr[8];
    float weights[32], mins[8], scales[8], sw[8];
    uint8_t packed[K_SCALE_SIZE];
    memset(packed, 0, sizeof packed);
    memset(L, 0, sizeof L);
    float d_blk, dmin_blk;
    if (!qw) {
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) {
            const float *sub = xb + 32 * j;
            float sum_x2 = 0.0f;
            for (int l = 0; l < 32; l++) sum_x2 = fmaf(sub[l], sub[l], sum_x2); /* q5_k.rs:183 */
            float av_x = sqrtf(sum_x2 / 32.0f);
            for (int l = 0; l < 32; l++) weights[l] = av_x + fabsf(sub[l]);
            scales[j] = make_qkx_quants(0, 32, 31, sub, weights, L + 32 * j, &mins[j], Laux, -0.5f,
                                        0.1f, 15, 0);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)nearest_int(inv_scale * scales[j]);
            uint8_t lm = (uint8_t)nearest_int(inv_min * mins[j]);
            ls_arr[j] = ls > 63 ? 63 : ls;
            lm_arr[j] = lm > 63 ? 63 : lm;
        }
        d_blk = max_scale / 63.0f;
        dmin_blk = max_min / 63.0f;
    } else {
        float sum_x2 = 0.0f;
        for (int l = 0; l < QK_K; l++) sum_x2 = fmaf(xb[l], xb[l], sum_x2); /* q5_k.rs:261 */
        float sigma2 = 2.0f * sum_x2 / (float)QK_K;
        for (int j = 0; j < 8; j++) {
            const float *sub = xb + 32 * j;
            for (int l = 0; l < 32; l++) weights[l] = qw[32 * j + l] * sqrtf(sigma2 + sub[l] * sub[l]);
            float sumw = 0.0f;
            for (int l = 0; l < 32; l++) sumw += weights[l];
            sw[j] = sumw;
            scales[j] = make_qkx_quants(1, 32, 31, sub, weights, L + 32 * j, &mins[j], Laux, -0.9f,
                                        0.05f, 36, 0);
        }
        d_blk = make_qp_quants(8, 63, scales, ls_arr, sw);
        dmin_blk = make_qp_quants(8, 63, mins, lm_arr, sw);
        for (int j = 0; j < 8; j++) {
            if (ls_arr[j] > 63) ls_arr[j] = 63;
            if (lm_arr[j] > 63) lm_arr[j] = 63;
        }
    }
    for (int j = 0; j < 8; j++) { /* q5_k.rs:72-82 pack_scale_min_k4 */
        uint8_t ls = ls_arr[j], lm = lm_arr[j];
        if (j < 4) {
            packed[j] = ls;
            packed[j + 4] = lm;
        } else {
            packed[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            packed[j - 4] |= (uint8_t)((ls >> 4) << 6);
            packed[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    uint16_t d16 = f32_to_f16_bits(d_blk), dmin16 = f32_to_f16_bits(dmin_blk);
    float d_dq = f16_bits_to_f32(d16), dmin_dq = f16_bits_to_f32(dmin16);
    for (int j = 0; j < 8; j++) { /* q5_k.rs:108-120: sub-blocks with d == 0 keep the search's L */
        uint8_t sc, m;
        get_scale_min_k4(j, packed, &sc, &m);
        float d = d_dq * (float)sc;
        if (d == 0.0f) continue;
        float dm = dmin_dq * (float)m;
        for (int ii = 0; ii < 32; ii++) {
            int l = nearest_int((xb[32 * j + ii] + dm) / d);
            L[32 * j + ii] = (uint8_t)imax(0, imin(31, l));
        }
    }
    out[0] = (uint8_t)(d16 & 0xFF);
    out[1] = (uint8_t)(d16 >> 8);
    out[2] = (uint8_t)(dmin16 & 0xFF);
    out[3] = (uint8_t)(dmin16 >> 8);
    memcpy(out + 4, packed, K_SCALE_SIZE);
    uint8_t *qh = out + 16, *ql = out + 48;
    memset(qh, 0, 32);
    uint8_t m1 = 1, m2 = 2;
    for (int n = 0; n < QK_K; n += 64) { /* q5_k.rs:138-157 */
        for (int j = 0; j < 32; j++) {
            int l1 = L[n + j], l2 = L[n + j + 32];
            if (l1 > 15) {
                l1 -= 16;
                qh[j] |= m1;
            }
            if (l2 > 15) {
                l2 -= 16;
                qh[j] |= m2;
            }
            ql[j] = (uint8_t)(l1 | (l2 << 4));
        }
        ql += 32;
        m1 = (uint8_t)(m1 << 2);
        m2 = (uint8_t)(m2 << 2);
    }
}

/* q4_0.rs:13-50 quantize_row_ref, one block of 32. */
static void q4_0_quantize_block(const float *xb, uint8_t *out) {
    float amax = 0.0f, max = 0.0f;
    for (int j = 0; j < QK4_0; j++) {
        float v = xb[j];
        if (amax < fabsf(v)) {
            amax = fabsf(v);
            max = v;
        }
    }
    float d = max / -8.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint16_t d16 = f32_to_f16_bits(d);
    out[0] = (uint8_t)(d16 & 0xFF);
    out[1] = (uint8_t)(d16 >> 8);
    for (int j = 0; j < QK4_0 / 2; j++) {
        float x0 = xb[j] * id, x1 = xb[QK4_0 / 2 + j] * id;
        int8_t a = (int8_t)(x0 + 8.5f), b = (int8_t)(x1 + 8.5f); /* truncating casts */
        uint8_t xi0 = (uint8_t)(a < 15 ? a : 15), xi1 = (uint8_t)(b < 15 ? b : 15);
        out[2 + j] = (uint8_t)(xi0 | (xi1 << 4));
    }
}

/* q4_0.rs:52-87 quantize_row_impl, one block of a row whose sigma2 = sum(x^2) / n_per_row. */
static void q4_0_quantize_block_im(const float *xb, const float *qw, float sigma2, uint8_t *out) {
    float weight[QK4_0];
    int8_t L[QK4_0];
    for (int j = 0; j < QK4_0; j++) weight[j] = qw[j] * sqrtf(sigma2 + xb[j] * xb[j]);
    float d = make_qx_quants(QK4_0, 8, xb, L, 1, weight);
    uint16_t d16 = f32_to_f16_bits(d);
    out[0] = (uint8_t)(d16 & 0xFF);
    out[1] = (uint8_t)(d16 >> 8);
    for (int j = 0; j < 16; j++) out[2 + j] = (uint8_t)((uint8_t)L[j] | ((uint8_t)L[j + 16] << 4));
}

/* q6_k.rs:40-151 quantize_one_block. */
static void q6k_quantize_block(const float *xb, const float *qw, uint8_t *out) {
    int8_t L[QK_K];
    float scales[16];
    float max_scale = 0.0f, max_abs_scale = 0.0f;
    for (int ib = 0; ib < 16; ib++) {
        float scale = make_qx_quants(16, 32, xb + 16 * ib, L + 16 * ib, 1, qw ? qw + 16 * ib : NULL);
        scales[ib] = scale;
        float a = fabsf(scale);
        if (a > max_abs_scale) {
            max_abs_scale = a;
            max_scale = scale;
        }
    }
    memset(out, 0, Q6K_BYTES);
    if (max_abs_scale < GROUP_MAX_EPS) return;
    float iscale = -128.0f / max_scale;
    uint16_t d16 = f32_to_f16_bits(1.0f / iscale);
    int8_t sc[16];
    for (int ib = 0; ib < 16; ib++) sc[ib] = (int8_t)imin(127, nearest_int(iscale * scales[ib]));
    float d_back = f16_bits_to_f32(d16);
    for (int j = 0; j < 16; j++) {
        float d = d_back * (float)sc[j];
        if (d == 0.0f) continue;
        for (int ii = 0; ii < 16; ii++) {
            int l = nearest_int(xb[16 * j + ii] / d);
            l = imax(-32, imin(31, l));
            L[16 * j + ii] = (int8_t)(l + 32);
        }
    }
    uint8_t *ql = out, *qh = out + 128;
    for (int j = 0; j < QK_K; j += 128) {
        for (int l = 0; l < 32; l++) {
            uint8_t a = (uint8_t)L[j + l], b = (uint8_t)L[j + l + 32], c = (uint8_t)L[j + l + 64],
                    e = (uint8_t)L[j + l + 96];
            ql[l] = (uint8_t)((a & 0xF) | ((c & 0xF) << 4));
            ql[l + 32] = (uint8_t)((b & 0xF) | ((e & 0xF) << 4));
            qh[l] = (uint8_t)((a >> 4) | ((b >> 4) << 2) | ((c >> 4) << 4) | ((e >> 4) << 6));
        }
        ql += 64;
        qh += 32;
    }
    for (int ib = 0; ib < 16; ib++) out[192 + ib] = (uint8_t)sc[ib];
    out[208] = (uint8_t)(d16 & 0xFF);
    out[209] = (uint8_t)(d16 >> 8);
}

/* q8_0.rs:31-72.  Rust's f32::round is half-away-from-zero == C roundf. */
static void q8_0_quantize_block(const float *xb, uint8_t *out) {
    float amax = 0.0f;
    for (int i = 0; i < QK8_0; i++) {
        float a = fabsf(xb[i]);
        if (a > amax) amax = a;
    }
    float d = amax / 127.0f;
    float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint16_t d16 = f32_to_f16_bits(d);
    out[0] = (uint8_t)(d16 & 0xFF);
    out[1] = (uint8_t)(d16 >> 8);
    for (int i = 0; i < QK8_0; i++) {
        float r = roundf(xb[i] * id);
        if (r > 127.0f) r = 127.0f; /* `as i8` saturates */
        if (r < -128.0f) r = -128.0f;
        out[2 + i] = (uint8_t)(int8_t)r;
    }
}

enum { T_Q4_0 = 2, T_Q8_0 = 8, T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14 }; /* ggml_type.rs:18-53 */

static int block_elems(int t) {
    return (t == T_Q8_0 || t == T_Q4_0) ? 32 : (t == T_Q4_K || t == T_Q5_K || t == T_Q6_K) ? 256 : 0;
}
static int block_bytes(int t) {
    return t == T_Q8_0 ? Q8_0_BYTES : t == T_Q4_K ? Q4K_BYTES : t == T_Q6_K ? Q6K_BYTES
           : t == T_Q5_K ? Q5K_BYTES : t == T_Q4_0 ? Q4_0_BYTES : 0;
}

/* quantizer.rs:51-102 dispatch + q4_k.rs:50-86 / q6_k.rs:181-221 / q8_0.rs:31-72.
 * `imatrix` (length n_per_row) is re-used for every row; NULL = reference path.
 * Returns 0, or -1 on a shape the reference rejects (quantizer.rs:57-71). */
int hq_oracle_quantize(const float *src, int64_t n_elems, int64_t n_per_row, int ggml_type,
                       const float *imatrix, uint8_t *out, int n_threads) {
    int be = block_elems(ggml_type), bb = block_bytes(ggml_type);
    if (!be || n_per_row <= 0 || n_per_row % be != 0 || n_elems % n_per_row != 0) return -1;
    int64_t nblocks = n_elems / be;
    int64_t blocks_per_row = n_per_row / be;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (int64_t b = 0; b < nblocks; b++) {
        const float *xb = src + b * be;
        uint8_t *ob = out + b * bb;
        int64_t in_row = b % blocks_per_row;
        const float *qw = imatrix ? imatrix + in_row * be : NULL;
        if (ggml_type == T_Q4_K)
            q4k_quantize_block(xb, qw, ob);
        else if (ggml_type == T_Q5_K)
            q5k_quantize_block(xb, qw, ob);
        else if (ggml_type == T_Q6_K)
            q6k_quantize_block(xb, qw, ob);
        else if (ggml_type == T_Q4_0) {
            if (qw) { /* q4_0.rs:61-65: the row's mean square enters every block's weights */
                const float *row = src + (b / blocks_per_row) * n_per_row;
                float sum_x2 = 0.0f;
                for (int64_t j = 0; j < n_per_row; j++) sum_x2 += row[j] * row[j];
                q4_0_quantize_block_im(xb, qw, sum_x2 / (float)n_per_row, ob);
            } else {
                q4_0_quantize_block(xb, ob);
            }
        } else
            q8_0_quantize_block(xb, ob);
    }
    return 0;
}

/* Dequantisation.  hf2q holds no K-quant dequantiser (its CPU path calls the
 * third-party GGUF reader); the formulas are the inverse of the re-quantisation
 * loops q4_k.rs:185-197 (`L = (x + dmin*m)/(d*sc)`), q6_k.rs:97-110
 * (`L = x/(d*sc) + 32`) and q8_0.rs:59-67 (`q = x/d`), with the block layouts
 * of q4_k.rs:199-215, q6_k.rs:112-150, q8_0.rs:62-68.  Every product below is
 * exact in f32, so each output is one correctly rounded value whatever the
 * association or use of FMA. */
static void q4k_dequant_block(const uint8_t *b, float *y) {
    float d = f16_bits_to_f32((uint16_t)(b[0] | (b[1] << 8)));
    float dmin = f16_bits_to_f32((uint16_t)(b[2] | (b[3] << 8)));
    const uint8_t *q = b + 16;
    int is = 0;
    for (int j = 0; j < QK_K; j += 64) {
        uint8_t sc, m;
        get_scale_min_k4(is, b + 4, &sc, &m);
        float d1 = d * (float)sc, m1 = dmin * (float)m;
        get_scale_min_k4(is + 1, b + 4, &sc, &m);
        float d2 = d * (float)sc, m2 = dmin * (float)m;
        for (int l = 0; l < 32; l++) y[j + l] = d1 * (float)(q[l] & 0xF) - m1;
        for (int l = 0; l < 32; l++) y[j + 32 + l] = d2 * (float)(q[l] >> 4) - m2;
        q += 32;
        is += 2;
    }
}

static void q6k_dequant_block(const uint8_t *b, float *y) {
    float d = f16_bits_to_f32((uint16_t)(b[208] | (b[209] << 8)));
    const uint8_t *ql = b, *qh = b + 128;
    const int8_t *sc = (const int8_t *)(b + 192);
    for (int h = 0; h < 2; h++) {
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int q1 = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
            int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
            int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
            int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            y[l] = d * (float)sc[is] * (float)q1;
            y[l + 32] = d * (float)sc[is + 2] * (float)q2;
            y[l + 64] = d * (float)sc[is + 4] * (float)q3;
            y[l + 96] = d * (float)sc[is + 6] * (float)q4;
        }
        y += 128;
        ql += 64;
        qh += 32;
        sc += 8;
    }
}

/* Inverse of q5_k.rs:108-157: y = d*sc*(ql + 16*hbit) - dmin*m; d*sc*q (11 + 6 + 5 bits) and
 * dmin*m are exact in f32, so y is one rounding of an exact difference. */
static void q5k_dequant_block(const uint8_t *b, float *y) {
    float d = f16_bits_to_f32((uint16_t)(b[0] | (b[1] << 8)));
    float dmin = f16_bits_to_f32((uint16_t)(b[2] | (b[3] << 8)));
    const uint8_t *qh = b + 16, *ql = b + 48;
    int is = 0;
    uint8_t u1 = 1, u2 = 2;
    for (int j = 0; j < QK_K; j += 64) {
        uint8_t sc, m;
        get_scale_min_k4(is, b + 4, &sc, &m);
        float d1 = d * (float)sc, m1 = dmin * (float)m;
        get_scale_min_k4(is + 1, b + 4, &sc, &m);
        float d2 = d * (float)sc, m2 = dmin * (float)m;
        for (int l = 0; l < 32; l++) y[j + l] = d1 * (float)((ql[l] & 0xF) + ((qh[l] & u1) ? 16 : 0)) - m1;
        for (int l = 0; l < 32; l++) y[j + 32 + l] = d2 * (float)((ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - m2;
        ql += 32;
        is += 2;
        u1 = (uint8_t)(u1 << 2);
        u2 = (uint8_t)(u2 << 2);
    }
}

/* Inverse of q4_0.rs:36-46: y = d * (q - 8), low nibbles are elements 0..15, high 16..31. */
static void q4_0_dequant_block(const uint8_t *b, float *y) {
    float d = f16_bits_to_f32((uint16_t)(b[0] | (b[1] << 8)));
    for (int j = 0; j < 16; j++) {
        y[j] = d * (float)((int)(b[2 + j] & 0xF) - 8);
        y[j + 16] = d * (float)((int)(b[2 + j] >> 4) - 8);
    }
}

static void q8_0_dequant_block(const uint8_t *b, float *y) {
    float d = f16_bits_to_f32((uint16_t)(b[0] | (b[1] << 8)));
    for (int i = 0; i < QK8_0; i++) y[i] = d * (float)(int8_t)b[2 + i];
}

static void dequant_block(int ggml_type, const uint8_t *b, float *y) {
    if (ggml_type == T_Q4_K)
        q4k_dequant_block(b, y);
    else if (ggml_type == T_Q5_K)
        q5k_dequant_block(b, y);
    else if (ggml_type == T_Q6_K)
        q6k_dequant_block(b, y);
    else if (ggml_type == T_Q4_0)
        q4_0_dequant_block(b, y);
    else
        q8_0_dequant_block(b, y);
}

int hq_oracle_dequantize(const uint8_t *blocks, int64_t n_elems, int ggml_type, float *out,
                         int n_threads) {
    int be = block_elems(ggml_type), bb = block_bytes(ggml_type);
    if (!be || n_elems % be != 0) return -1;
    int64_t nblocks = n_elems / be;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (int64_t b = 0; b < nblocks; b++) {
        dequant_block(ggml_type, blocks + b * bb, out + b * be);
    }
    return 0;
}

/* ffn.rs:38-50 matmul_a_by_bt: out[i,j] = sum_k lhs[i,k]*rhs[j,k], f32
 * accumulate in k order.  This is "hf2q's scalar matmul" of the CPU baseline. */
void hq_oracle_matmul_a_by_bt(const float *lhs, const float *rhs, int64_t m, int64_t k, int64_t n,
                              float *out, int n_threads) {
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (int64_t j = 0; j < n; j++) {
        for (int64_t i = 0; i < m; i++) {
            float acc = 0.0f;
            for (int64_t kk = 0; kk < k; kk++) acc += lhs[i * k + kk] * rhs[j * k + kk];
            out[i * n + j] = acc;
        }
    }
}

/* The parity gate of the path: y[m,n] = x[m,k] . W[n,k]^T in float64 over the
 * bit-exact dequantised weights, streaming W block-row by block-row so that the
 * 151936x4096 head never has to exist in f32.  x is f32 (xdt=0) or bf16 bits
 * (xdt=1), widened exactly. */
int hq_oracle_qmatmul_f64(const void *x, int xdt, const uint8_t *w_blocks, int64_t m, int64_t n,
                          int64_t k, int ggml_type, double *y, int n_threads) {
    int be = block_elems(ggml_type), bb = block_bytes(ggml_type);
    if (!be || k % be != 0) return -1;
    int64_t row_bytes = k / be * bb;
    double *xd = (double *)malloc(sizeof(double) * (size_t)(m * k));
    if (!xd) return -2;
    for (int64_t i = 0; i < m * k; i++)
        xd[i] = xdt ? (double)bf16_bits_to_f32(((const uint16_t *)x)[i]) : (double)((const float *)x)[i];
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel num_threads(n_threads)
    {
        float *wrow = (float *)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(static)
        for (int64_t j = 0; j < n; j++) {
            const uint8_t *rb = w_blocks + j * row_bytes;
            for (int64_t b = 0; b < k / be; b++) dequant_block(ggml_type, rb + b * bb, wrow + b * be);
            for (int64_t i = 0; i < m; i++) {
                const double *xi = xd + i * k;
                double acc = 0.0;
                for (int64_t kk = 0; kk < k; kk++) acc += xi[kk] * (double)wrow[kk];
                y[i * n + j] = acc;
            }
        }
        free(wrow);
    }
    free(xd);
    return 0;
}

/* mul_mat_id semantics (gpu_ffn.rs:2606-2618, forward_mlx.rs:5237-5245):
 * out[t, s, :] = W[ids[t*top_k+s]] . x[t, :], stack = [n_experts][n][k/QK]. */
int hq_oracle_qmatmul_id_f64(const void *x, int xdt, const uint8_t *w_stack, const uint32_t *ids,
                             int64_t n_tokens, int64_t top_k, int64_t n, int64_t k,
                             int64_t n_experts, int64_t expert_stride, int ggml_type, double *y,
                             int n_threads) {
    size_t xs = xdt ? 2 : 4;
    for (int64_t t = 0; t < n_tokens; t++)
        for (int64_t s = 0; s < top_k; s++) {
            uint32_t e = ids[t * top_k + s];
            if ((int64_t)e >= n_experts) return -3;
            int rc = hq_oracle_qmatmul_f64((const uint8_t *)x + (size_t)(t * k) * xs, xdt,
                                           w_stack + (size_t)e * (size_t)expert_stride, 1, n, k,
                                           ggml_type, y + (t * top_k + s) * n, n_threads);
            if (rc) return rc;
        }
    return 0;
}

/* ffn.rs:24-30 */
static float silu_f(float x) { return x / (1.0f + expf(-x)); }
static float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
float hq_oracle_silu(float x) { return silu_f(x); }

/* gpu_ffn.rs:1879-1924 softmax_topk_renorm_cpu.  Rust's sort_by is stable, so
 * ties keep ascending expert index; an insertion of the k best reproduces it. */
void hq_oracle_softmax_topk_renorm(const float *logits, int64_t seq_len, int64_t n_experts,
                                   int64_t topk, uint32_t *out_idx, float *out_w) {
    float *p = (float *)malloc(sizeof(float) * (size_t)n_experts);
    char *taken = (char *)malloc((size_t)n_experts);
    for (int64_t t = 0; t < seq_len; t++) {
        const float *row = logits + t * n_experts;
        float max_v = -INFINITY;
        for (int64_t e = 0; e < n_experts; e++) max_v = fmaxf(max_v, row[e]);
        float denom = 0.0f;
        for (int64_t e = 0; e < n_experts; e++) {
            p[e] = expf(row[e] - max_v);
            denom += p[e];
        }
        float inv_d = denom > 1e-20f ? 1.0f / denom : 1.0f;
        for (int64_t e = 0; e < n_experts; e++) p[e] *= inv_d;
        memset(taken, 0, (size_t)n_experts);
        float sum_sel = 0.0f;
        for (int64_t s = 0; s < topk; s++) {
            int64_t best = -1;
            for (int64_t e = 0; e < n_experts; e++)
                if (!taken[e] && (best < 0 || p[e] > p[best])) best = e;
            taken[best] = 1;
            out_idx[t * topk + s] = (uint32_t)best;
            sum_sel += p[best];
        }
        float inv_sum = sum_sel > 1e-20f ? 1.0f / sum_sel : 1.0f / (float)topk;
        for (int64_t s = 0; s < topk; s++) out_w[t * topk + s] = p[out_idx[t * topk + s]] * inv_sum;
    }
    free(p);
    free(taken);
}

/* ffn.rs:179-336 moe_ffn_cpu_ref over f32 weights ([out,in] row-major), f32
 * accumulation in the reference's loop order.  router [E,h]; expert_gate/up
 * [E*m,h]; expert_down [E*h,m]; shared_gate_logit [h]; shared_* as dense. */
void hq_oracle_moe_ffn(const float *x, int64_t seq_len, int64_t h, int64_t ne, int64_t topk,
                       int64_t m_moe, int64_t m_sh, const float *router, const float *expert_gate,
                       const float *expert_up, const float *expert_down,
                       const float *shared_gate_logit, const float *shared_gate,
                       const float *shared_up, const float *shared_down, float *output) {
    float *logits = (float *)malloc(sizeof(float) * (size_t)ne);
    uint32_t *idx = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)topk);
    float *w = (float *)malloc(sizeof(float) * (size_t)topk);
    int64_t mm = m_moe > m_sh ? m_moe : m_sh;
    float *a = (float *)malloc(sizeof(float) * (size_t)mm);
    float *b = (float *)malloc(sizeof(float) * (size_t)mm);
    float *moe_out = (float *)malloc(sizeof(float) * (size_t)h);
    for (int64_t t = 0; t < seq_len; t++) {
        const float *xt = x + t * h;
        for (int64_t e = 0; e < ne; e++) {
            float acc = 0.0f;
            for (int64_t i = 0; i < h; i++) acc += router[e * h + i] * xt[i];
            logits[e] = acc;
        }
        /* ffn.rs:228-252: softmax, stable top-k, renormalise (uniform fallback). */
        hq_oracle_softmax_topk_renorm(logits, 1, ne, topk, idx, w);
        for (int64_t i = 0; i < h; i++) moe_out[i] = 0.0f;
        for (int64_t s = 0; s < topk; s++) {
            const float *gw = expert_gate + (int64_t)idx[s] * m_moe * h;
            const float *uw = expert_up + (int64_t)idx[s] * m_moe * h;
            const float *dw = expert_down + (int64_t)idx[s] * h * m_moe;
            for (int64_t i = 0; i < m_moe; i++) {
                float ga = 0.0f, ua = 0.0f;
                for (int64_t j = 0; j < h; j++) ga += gw[i * h + j] * xt[j];
                for (int64_t j = 0; j < h; j++) ua += uw[i * h + j] * xt[j];
                a[i] = silu_f(ga) * ua;
            }
            for (int64_t i = 0; i < h; i++) {
                float acc = 0.0f;
                for (int64_t j = 0; j < m_moe; j++) acc += dw[i * m_moe + j] * a[j];
                moe_out[i] += w[s] * acc;
            }
        }
        float sl = 0.0f;
        for (int64_t i = 0; i < h; i++) sl += shared_gate_logit[i] * xt[i];
        float sg = sigmoid_f(sl);
        for (int64_t i = 0; i < m_sh; i++) {
            float ga = 0.0f, ua = 0.0f;
            for (int64_t j = 0; j < h; j++) ga += shared_gate[i * h + j] * xt[j];
            for (int64_t j = 0; j < h; j++) ua += shared_up[i * h + j] * xt[j];
            b[i] = silu_f(ga) * ua;
        }
        for (int64_t i = 0; i < h; i++) {
            float acc = 0.0f;
            for (int64_t j = 0; j < m_sh; j++) acc += shared_down[i * m_sh + j] * b[j];
            output[t * h + i] = moe_out[i] + sg * acc;
        }
    }
    free(logits);
    free(idx);
    free(w);
    free(a);
    free(b);
    free(moe_out);
}

/* ------------------------------------------------------------------ */
/* TurboQuant-style KV: sign x FWHT rotation and the 8-bit cache.      */
/* ------------------------------------------------------------------ */
/* kv_cache.rs:3871-3876 TBQ_SIGNS_256: bit j of table[j>>3] set => -1. */
static const uint8_t TBQ_SIGNS_256[32] = {
    0xa7, 0x3b, 0x91, 0xf4, 0x6d, 0xc2, 0x58, 0x0e, 0xb3, 0x7f, 0x24, 0xd6, 0x89, 0x45, 0xea, 0x1c,
    0x63, 0xaf, 0xd8, 0x52, 0x97, 0x0b, 0xe1, 0x3d, 0x76, 0xc4, 0x19, 0xfe, 0x4a, 0x85, 0x2c, 0xdb};

/* kv_cache.rs:3879-3888 apply_d1_sign_d256 (per 256-element block). */
static void apply_sign(float *x, int d) {
    for (int j = 0; j < d; j++) {
        int jj = j & 255;
        if ((TBQ_SIGNS_256[jj >> 3] >> (jj & 7)) & 1) x[j] = -x[j];
    }
}

/* Normalised fast Walsh-Hadamard transform (H*H = I), natural (Sylvester)
 * order, over one block of `d` (power of two) elements. */
static void fwht(float *x, int d) {
    for (int h = 1; h < d; h <<= 1)
        for (int i = 0; i < d; i += h << 1)
            for (int j = i; j < i + h; j++) {
                float a = x[j], b = x[j + h];
                x[j] = a + b;
                x[j + h] = a - b;
            }
    float s = 1.0f / sqrtf((float)d);
    for (int i = 0; i < d; i++) x[i] *= s;
}

/* kv_cache.rs:3892-3902: premult = sign then FWHT; undo = FWHT then sign.
 * head_dim 512 is rotated as two independent 256-blocks. */
void hq_oracle_fwht_sign_premult(float *buf, int n_heads, int head_dim) {
    for (int h = 0; h < n_heads; h++)
        for (int o = 0; o < head_dim; o += 256) {
            apply_sign(buf + h * head_dim + o, 256);
            fwht(buf + h * head_dim + o, 256);
        }
}
void hq_oracle_fwht_sign_undo(float *buf, int n_heads, int head_dim) {
    for (int h = 0; h < n_heads; h++)
        for (int o = 0; o < head_dim; o += 256) {
            fwht(buf + h * head_dim + o, 256);
            apply_sign(buf + h * head_dim + o, 256);
        }
}

/* Write-side encode of one (kv_head, position) vector into the 8-bit cache in
 * the linear int8 form the benchmark configuration names: rotate, then per
 * 256-block `scale = amax/127`, `code = round_half_away(x/scale)` (the Q8_0
 * rule of q8_0.rs:59-67 applied per block), stored as a two's-complement byte.
 * Layout: codes [n_kv_heads, capacity, head_dim] u8, norms
 * [n_kv_heads, capacity, head_dim/256] f32 (kv_cache.rs:1982-2012). */
void hq_oracle_tq_encode_int8(const float *kv, int n_kv_heads, int head_dim, int capacity, int pos,
                              uint8_t *codes, float *norms) {
    int npp = head_dim / 256 > 0 ? head_dim / 256 : 1;
    float tmp[512];
    for (int h = 0; h < n_kv_heads; h++) {
        memcpy(tmp, kv + h * head_dim, sizeof(float) * (size_t)head_dim);
        hq_oracle_fwht_sign_premult(tmp, 1, head_dim);
        for (int b = 0; b < npp; b++) {
            float amax = 0.0f;
            for (int i = 0; i < 256; i++) amax = fmaxf(amax, fabsf(tmp[256 * b + i]));
            float d = amax / 127.0f;
            float id = d != 0.0f ? 1.0f / d : 0.0f;
            norms[((int64_t)h * capacity + pos) * npp + b] = d;
            for (int i = 0; i < 256; i++) {
                float r = roundf(tmp[256 * b + i] * id);
                codes[((int64_t)h * capacity + pos) * head_dim + 256 * b + i] = (uint8_t)(int8_t)r;
            }
        }
    }
}

/* Value of one cached element: linear (lut == NULL): norm * int8(code);
 * LUT form: lut[code] * norm / sqrt(256) / scale_factor_d512-per-block. */
static double tq_value(uint8_t code, float norm, const float *lut, float sf) {
    if (!lut) return (double)norm * (double)(int8_t)code;
    return (double)lut[code] * (double)norm / 16.0 / (double)sf;
}

/* Bulk dequantisation of cache positions start_pos .. start_pos + n_tokens - 1 (no wrap:
 * kv_cache.rs:427-428 rejects start_pos + n_tokens > capacity) into out[n_kv_heads][n_tokens][head_dim]
 * f32, rotated domain (dequant_seq_to_temp_f32, kv_cache.rs:431-495): each element is tq_value()
 * rounded once to f32. */
int hq_oracle_tq_dequantize(const uint8_t *codes, const float *norms, const float *lut, int n_kv_heads,
                            int head_dim, int capacity, int start_pos, int n_tokens,
                            float scale_factor_d512, float *out) {
    if (head_dim != 256 && head_dim != 512) return -1;
    if (start_pos < 0 || n_tokens < 0 || (int64_t)start_pos + n_tokens > capacity) return -2;
    int npp = head_dim / 256;
    float sf = head_dim == 512 ? scale_factor_d512 : 1.0f;
    for (int h = 0; h < n_kv_heads; h++)
        for (int t = 0; t < n_tokens; t++) {
            int64_t row = (int64_t)h * capacity + start_pos + t;
            for (int d = 0; d < head_dim; d++)
                out[((int64_t)h * n_tokens + t) * head_dim + d] =
                    (float)tq_value(codes[row * head_dim + d], norms[row * npp + d / 256], lut, sf);
        }
    return 0;
}

/* Single-query attention over the 8-bit cache in float64 (the parity gate for
 * flash_attn_vec_tq_hb, forward_mlx.rs:4687-4742, kv_cache.rs:335-388):
 * out[h] = softmax(scale * q[h] . K[kv(h)]^T [softcapped, masked]) . V[kv(h)],
 * kv(h) = h / (num_heads/num_kv_heads) (kv_cache.rs:4091-4096).  Logical
 * position i lives in physical slot (ring_start + i) % kv_capacity (the inverse of
 * forward_mlx.rs:7299, logical = (k_pos - ring_start + cap) % cap); mask 2
 * keeps only the last `sliding_window` logical positions; masks 0 and 1 keep
 * all kv_seq_len positions for a single query at the end of the sequence. */
int hq_oracle_tq_attention(const float *q, const uint8_t *k_codes, const float *k_norms,
                           const uint8_t *v_codes, const float *v_norms, const float *lut,
                           int num_heads, int num_kv_heads, int head_dim, int kv_seq_len,
                           int kv_capacity, float scale, int mask_type, int sliding_window,
                           float softcap, int ring_start, float scale_factor_d512, double *out) {
    if (head_dim != 256 && head_dim != 512) return -1;
    if (kv_seq_len <= 0 || kv_capacity < kv_seq_len) return -2;
    if (num_kv_heads <= 0 || num_heads % num_kv_heads) return -3;
    int npp = head_dim / 256;
    int group = num_heads / num_kv_heads;
    float sf = head_dim == 512 ? scale_factor_d512 : 1.0f;
    int first = 0;
    if (mask_type == 2 && sliding_window > 0 && kv_seq_len > sliding_window)
        first = kv_seq_len - sliding_window;
    double *s = (double *)malloc(sizeof(double) * (size_t)kv_seq_len);
    for (int h = 0; h < num_heads; h++) {
        int kvh = h / group;
        double mx = -INFINITY;
        for (int i = first; i < kv_seq_len; i++) {
            int64_t slot = ((int64_t)ring_start + i) % kv_capacity;
            const uint8_t *kc = k_codes + ((int64_t)kvh * kv_capacity + slot) * head_dim;
            const float *kn = k_norms + ((int64_t)kvh * kv_capacity + slot) * npp;
            double acc = 0.0;
            for (int d = 0; d < head_dim; d++)
                acc += (double)q[h * head_dim + d] * tq_value(kc[d], kn[d / 256], lut, sf);
            acc *= (double)scale;
            if (softcap != 0.0f) acc = (double)softcap * tanh(acc / (double)softcap);
            s[i] = acc;
            if (acc > mx) mx = acc;
        }
        double denom = 0.0;
        for (int i = first; i < kv_seq_len; i++) {
            s[i] = exp(s[i] - mx);
            denom += s[i];
        }
        for (int d = 0; d < head_dim; d++) out[h * head_dim + d] = 0.0;
        for (int i = first; i < kv_seq_len; i++) {
            int64_t slot = ((int64_t)ring_start + i) % kv_capacity;
            const uint8_t *vc = v_codes + ((int64_t)kvh * kv_capacity + slot) * head_dim;
            const float *vn = v_norms + ((int64_t)kvh * kv_capacity + slot) * npp;
            double p = s[i] / denom;
            for (int d = 0; d < head_dim; d++)
                out[h * head_dim + d] += p * tq_value(vc[d], vn[d / 256], lut, sf);
        }
    }
    free(s);
    return 0;
}

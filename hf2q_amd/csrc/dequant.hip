// Dequantisation of GGML Q4_K / Q6_K / Q8_0 blocks to f32 (bit-exact) or bf16.
//
// hf2q has no K-quant dequantiser of its own; the value of an element is fixed
// by the second-stage loops of its quantizers (q4_k.rs:185-197:
// L = (x + dmin*m)/(d*sc); q6_k.rs:97-110: L = x/(d*sc) + 32; q8_0.rs:59-67):
//   Q4_K  y = (d*sc)*q - dmin*m      Q6_K  y = (d*sc)*(q-32)      Q8_0  y = d*q
//   Q5_K  as Q4_K with q in 0..31 (q5_k.rs:108-157)              Q4_0  y = d*(q-8) (q4_0.rs:36-46)
// d*sc, dmin*m and (d*sc)*q (Q4_K) are exact in f32, so each y below is a
// single rounding of the exact value and does not depend on FMA contraction.
//
// One thread produces four consecutive elements (one 16-byte or 8-byte store),
// so stores are fully coalesced; the handful of header bytes each thread
// re-reads come from cache.  Bandwidth-bound: 4.56 / 4.82 / 5.06 bytes moved
// per element (read + f32 write) for Q4_K / Q6_K / Q8_0.
#include "hq_internal.h"

namespace hq {

template <int TYPE>
__device__ __forceinline__ void dequant4(const uint8_t* __restrict__ w, uint64_t e, float out[4]) {
    if constexpr (TYPE == HQ_Q4_K) {
        const uint8_t* blk = w + (e >> 8) * Q4K_BYTES;
        const uint32_t ib = (uint32_t)e & 255u;      // element inside the block
        const uint32_t c = ib >> 6;                  // 64-element chunk
        const uint32_t hi = (ib >> 5) & 1u;          // high nibble half
        const uint32_t l = ib & 31u;                 // byte inside the chunk (multiple of 4)
        const uint4 hdr = *reinterpret_cast<const uint4*>(blk);
        const float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
        uint32_t sc0, sc1, m0, m1;
        q4k_scales(hdr.y, hdr.z, hdr.w, (int)c, sc0, sc1, m0, m1);
        const float ds = d * (float)(hi ? sc1 : sc0);
        const float dm = dmin * (float)(hi ? m1 : m0);
        uint32_t q = *reinterpret_cast<const uint32_t*>(blk + 16 + 32 * c + l);
        q = (q >> (4 * hi)) & 0x0f0f0f0fu;
        out[0] = ds * ubyte0(q) - dm;
        out[1] = ds * ubyte1(q) - dm;
        out[2] = ds * ubyte2(q) - dm;
        out[3] = ds * ubyte3(q) - dm;
    } else if constexpr (TYPE == HQ_Q6_K) {
        const uint8_t* blk = w + (e >> 8) * Q6K_BYTES;
        const uint32_t ib = (uint32_t)e & 255u;
        const uint32_t h = ib >> 7;           // 128-element half
        const uint32_t r = (ib >> 5) & 3u;    // 32-element run inside the half
        const uint32_t l = ib & 31u;          // multiple of 4
        uint32_t ql, qh;
        __builtin_memcpy(&ql, blk + 64 * h + 32 * (r & 1u) + l, 4);
        __builtin_memcpy(&qh, blk + 128 + 32 * h + l, 4);
        const uint32_t q = ((ql >> (4 * (r >> 1))) & 0x0f0f0f0fu) | (((qh >> (2 * r)) << 4) & 0x30303030u);
        const int sc = (int)(int8_t)blk[192 + 8 * h + 2 * r + (l >> 4)];
        const float ds = f16_bits_to_f32(ld2(blk + 208)) * (float)sc;
        out[0] = ds * (ubyte0(q) - 32.0f);
        out[1] = ds * (ubyte1(q) - 32.0f);
        out[2] = ds * (ubyte2(q) - 32.0f);
        out[3] = ds * (ubyte3(q) - 32.0f);
    } else if constexpr (TYPE == HQ_Q5_K) {  // as Q4_K with a fifth bit: bit (sub-block) of high-bit byte l
        const uint8_t* blk = w + (e >> 8) * Q5K_BYTES;
        const uint32_t ib = (uint32_t)e & 255u;
        const uint32_t c = ib >> 6, hi = (ib >> 5) & 1u, l = ib & 31u;
        const uint4 hdr = *reinterpret_cast<const uint4*>(blk);
        const float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
        uint32_t sc0, sc1, m0, m1;
        q4k_scales(hdr.y, hdr.z, hdr.w, (int)c, sc0, sc1, m0, m1);
        const float ds = d * (float)(hi ? sc1 : sc0);
        const float dm = dmin * (float)(hi ? m1 : m0);
        uint32_t q = *reinterpret_cast<const uint32_t*>(blk + 48 + 32 * c + l);
        const uint32_t h = *reinterpret_cast<const uint32_t*>(blk + 16 + l) >> (2 * c + hi);
        q = ((q >> (4 * hi)) & 0x0f0f0f0fu) | ((h << 4) & 0x10101010u);
        out[0] = ds * ubyte0(q) - dm;
        out[1] = ds * ubyte1(q) - dm;
        out[2] = ds * ubyte2(q) - dm;
        out[3] = ds * ubyte3(q) - dm;
    } else if constexpr (TYPE == HQ_Q4_0) {  // y = d * (q - 8); low nibbles elements 0..15, high nibbles 16..31
        const uint8_t* blk = w + (e >> 5) * Q4_0_BYTES;
        const uint32_t l = (uint32_t)e & 31u;
        const float d = f16_bits_to_f32(ld2(blk));
        uint32_t q;
        __builtin_memcpy(&q, blk + 2 + (l & 15u), 4);
        q = (q >> (l & 16u ? 4 : 0)) & 0x0f0f0f0fu;
        out[0] = d * (ubyte0(q) - 8.0f);
        out[1] = d * (ubyte1(q) - 8.0f);
        out[2] = d * (ubyte2(q) - 8.0f);
        out[3] = d * (ubyte3(q) - 8.0f);
    } else {
        const uint8_t* blk = w + (e >> 5) * Q8_0_BYTES;
        const uint32_t l = (uint32_t)e & 31u;
        const float d = f16_bits_to_f32(ld2(blk));
        uint32_t q;
        __builtin_memcpy(&q, blk + 2 + l, 4);
        out[0] = d * sbyte(q, 0);
        out[1] = d * sbyte(q, 1);
        out[2] = d * sbyte(q, 2);
        out[3] = d * sbyte(q, 3);
    }
}

template <int TYPE, int OUT>  // OUT: hq_act_dtype of the output
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ w, void* __restrict__ out,
                                                      uint64_t n_quads) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n_quads; i += (uint64_t)gridDim.x * 256) {
        float v[4];
        dequant4<TYPE>(w, i * 4, v);
        if constexpr (OUT == HQ_BF16) {
            uint2 o;
            o.x = f32_to_bf16_bits(v[0]) | (f32_to_bf16_bits(v[1]) << 16);
            o.y = f32_to_bf16_bits(v[2]) | (f32_to_bf16_bits(v[3]) << 16);
            reinterpret_cast<uint2*>(out)[i] = o;
        } else if constexpr (OUT == HQ_F16) {  // v_cvt_f16_f32: round to nearest even, overflow to infinity
            // (the f32 value is made opaque first: the compiler otherwise folds its last multiplication into the
            // conversion as v_fma_mixlo_f16 x, y, +0, which turns a product of -0.0 into +0.0)
            const auto h = [](float f) {
                asm volatile("" : "+v"(f));
                return (uint32_t)__builtin_bit_cast(unsigned short, (_Float16)f);
            };
            uint2 o;
            o.x = h(v[0]) | (h(v[1]) << 16);
            o.y = h(v[2]) | (h(v[3]) << 16);
            reinterpret_cast<uint2*>(out)[i] = o;
        } else {
            reinterpret_cast<float4*>(out)[i] = make_float4(v[0], v[1], v[2], v[3]);
        }
    }
}

template <int TYPE>
static int launch_t(hipStream_t s, const void* w, void* out, hq_act_dtype odt, uint64_t n_elems) {
    const uint64_t quads = n_elems / 4;
    const uint64_t want = (quads + 255) / 256;
    const unsigned grid = (unsigned)(want < 65536 ? want : 65536);
    const uint8_t* wb = static_cast<const uint8_t*>(w);
    if (odt == HQ_BF16)
        hipLaunchKernelGGL((dequant_kernel<TYPE, HQ_BF16>), dim3(grid), dim3(256), 0, s, wb, out, quads);
    else if (odt == HQ_F16)
        hipLaunchKernelGGL((dequant_kernel<TYPE, HQ_F16>), dim3(grid), dim3(256), 0, s, wb, out, quads);
    else
        hipLaunchKernelGGL((dequant_kernel<TYPE, HQ_F32>), dim3(grid), dim3(256), 0, s, wb, out, quads);
    return check_launch("dequant kernel launch");
}

int launch_dequant(hipStream_t s, const void* w, void* out, hq_act_dtype odt, uint64_t n_elems,
                   hq_ggml_type t) {
    switch (t) {
        case HQ_Q4_K: return launch_t<HQ_Q4_K>(s, w, out, odt, n_elems);
        case HQ_Q6_K: return launch_t<HQ_Q6_K>(s, w, out, odt, n_elems);
        case HQ_Q8_0: return launch_t<HQ_Q8_0>(s, w, out, odt, n_elems);
        case HQ_Q5_K: return launch_t<HQ_Q5_K>(s, w, out, odt, n_elems);
        case HQ_Q4_0: return launch_t<HQ_Q4_0>(s, w, out, odt, n_elems);
    }
    return fail(HQ_ERR_UNSUPPORTED, "dequant: ggml type %d", (int)t);
}

}  // namespace hq

// On-disk envelope of a spilled TurboQuant K or V block ("TQP1" / "TQP2") and the capture / restore
// of a range of cache positions between device memory and such an envelope in host memory.
//
// Wire format (kv_persist/families/tq_packed.rs:37-52, 330-352), little-endian:
//   [ 0.. 4] magic "TQP1" (codec_version 1) or "TQP2" (codec_version 2)
//   [ 4.. 8] codec_version   [ 8..12] bits_per_coord (1..8)   [12..16] head_dim
//   [16..20] n_kv_heads      [20..24] n_tokens               [24..28] flags
//   [28..32] reserved = 0    [32..40] f64 scale
//   [40.. ]  indices, ceil(n_kv_heads * n_tokens * head_dim * bits / 8) bytes, [head][token][dim]
//   v2 only: f32 norms, n_kv_heads * n_tokens * max(1, head_dim / 256) values, [head][token][block]
// Host code only; nothing here launches a kernel.
#include <string.h>

#include "hq_internal.h"

namespace {

constexpr uint32_t MAGIC_V1 = 0x31505154u, MAGIC_V2 = 0x32505154u;

void put_u32(uint8_t* p, uint32_t v) {
    p[0] = (uint8_t)v, p[1] = (uint8_t)(v >> 8), p[2] = (uint8_t)(v >> 16), p[3] = (uint8_t)(v >> 24);
}
uint32_t get_u32(const uint8_t* p) { return p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }

size_t norms_per_pos(uint32_t head_dim) { return head_dim / 256 ? head_dim / 256 : 1; }

}  // namespace

using hq::fail;

extern "C" {

size_t hq_tqp_indices_bytes(const hq_tqp_header* h) {
    if (!h) return 0;
    // four 32-bit factors: at most 2^128 - 2^98, which the 128-bit product holds; a count beyond size_t saturates (no
    // buffer has that length, so hq_tqp_pack / hq_tqp_unpack reject the header)
    const unsigned __int128 bits = (unsigned __int128)h->n_kv_heads * h->n_tokens * h->head_dim * h->bits_per_coord;
    const unsigned __int128 bytes = (bits + 7) / 8;
    return bytes > (unsigned __int128)SIZE_MAX ? SIZE_MAX : (size_t)bytes;
}

size_t hq_tqp_norms_bytes(const hq_tqp_header* h) {
    if (!h || h->codec_version != 2) return 0;
    const unsigned __int128 bytes = (unsigned __int128)h->n_kv_heads * h->n_tokens * norms_per_pos(h->head_dim) * 4;
    return bytes > (unsigned __int128)SIZE_MAX ? SIZE_MAX : (size_t)bytes;
}

size_t hq_tqp_total_bytes(const hq_tqp_header* h) {
    if (!h) return 0;
    const size_t a = hq_tqp_indices_bytes(h), b = hq_tqp_norms_bytes(h);
    if (a > SIZE_MAX - HQ_TQP_HEADER_BYTES || b > SIZE_MAX - HQ_TQP_HEADER_BYTES - a) return SIZE_MAX;
    return HQ_TQP_HEADER_BYTES + a + b;
}

int hq_tqp_pack(const hq_tqp_header* h, const void* indices, size_t indices_len, const void* norms_le, size_t norms_len,
                void* out, size_t out_capacity) {
    const char* fn = "hq_tqp_pack";
    if (!h || !out) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null argument", fn);
    if (h->codec_version != 1 && h->codec_version != 2)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: unsupported codec version %u", fn, h->codec_version);
    if (h->bits_per_coord == 0 || h->bits_per_coord > 8)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: invalid bits_per_coord %u", fn, h->bits_per_coord);
    const size_t want_i = hq_tqp_indices_bytes(h), want_n = hq_tqp_norms_bytes(h);
    if (indices_len != want_i)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: payload size mismatch: %zu index bytes expected, got %zu", fn, want_i, indices_len);
    if (norms_len != want_n)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: payload size mismatch: %zu norm bytes expected, got %zu", fn, want_n, norms_len);
    if ((want_i && !indices) || (want_n && !norms_le)) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null body", fn);
    if (out_capacity < HQ_TQP_HEADER_BYTES + want_i + want_n)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: output holds %zu bytes, %zu needed", fn, out_capacity,
                    HQ_TQP_HEADER_BYTES + want_i + want_n);
    uint8_t* o = static_cast<uint8_t*>(out);
    put_u32(o, h->codec_version == 1 ? MAGIC_V1 : MAGIC_V2);
    put_u32(o + 4, h->codec_version);
    put_u32(o + 8, h->bits_per_coord);
    put_u32(o + 12, h->head_dim);
    put_u32(o + 16, h->n_kv_heads);
    put_u32(o + 20, h->n_tokens);
    put_u32(o + 24, h->flags);
    put_u32(o + 28, 0);
    uint64_t sbits;
    memcpy(&sbits, &h->scale, 8);
    put_u32(o + 32, (uint32_t)sbits);
    put_u32(o + 36, (uint32_t)(sbits >> 32));
    if (want_i) memcpy(o + HQ_TQP_HEADER_BYTES, indices, want_i);
    if (want_n) memcpy(o + HQ_TQP_HEADER_BYTES + want_i, norms_le, want_n);
    return HQ_OK;
}

int hq_tqp_unpack(const void* payload, size_t len, hq_tqp_header* h, size_t* indices_offset, size_t* norms_offset) {
    const char* fn = "hq_tqp_unpack";
    if (!payload || !h) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null argument", fn);
    if (len < HQ_TQP_HEADER_BYTES) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: truncated: %zu bytes", fn, len);
    const uint8_t* p = static_cast<const uint8_t*>(payload);
    const uint32_t magic = get_u32(p);
    if (magic != MAGIC_V1 && magic != MAGIC_V2) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: bad magic 0x%08x", fn, magic);
    const uint32_t version = get_u32(p + 4);
    if (version != (magic == MAGIC_V1 ? 1u : 2u))
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: unsupported codec version %u", fn, version);
    const uint32_t bits = get_u32(p + 8);
    if (bits == 0 || bits > 8) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: invalid bits_per_coord %u", fn, bits);
    const uint32_t reserved = get_u32(p + 28);
    if (reserved != 0) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: reserved field is 0x%08x, not zero", fn, reserved);
    hq_tqp_header t;
    t.codec_version = version;
    t.bits_per_coord = bits;
    t.head_dim = get_u32(p + 12);
    t.n_kv_heads = get_u32(p + 16);
    t.n_tokens = get_u32(p + 20);
    t.flags = get_u32(p + 24);
    const uint64_t sbits = get_u32(p + 32) | ((uint64_t)get_u32(p + 36) << 32);
    memcpy(&t.scale, &sbits, 8);
    const size_t want = hq_tqp_indices_bytes(&t) + hq_tqp_norms_bytes(&t);
    if (len - HQ_TQP_HEADER_BYTES != want)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: payload size mismatch: %zu body bytes expected, got %zu", fn, want,
                    len - HQ_TQP_HEADER_BYTES);
    *h = t;
    if (indices_offset) *indices_offset = HQ_TQP_HEADER_BYTES;
    if (norms_offset) *norms_offset = HQ_TQP_HEADER_BYTES + hq_tqp_indices_bytes(&t);
    return HQ_OK;
}

size_t hq_tq_kv_capture_bytes(uint32_t n_kv_heads, uint32_t head_dim, uint32_t n_tokens) {
    hq_tqp_header h{2, 8, head_dim, n_kv_heads, n_tokens, 0, 1.0};
    return hq_tqp_total_bytes(&h);
}

int hq_tq_kv_capture(void* stream, const uint8_t* codes, const float* norms, uint32_t n_kv_heads, uint32_t head_dim,
                     uint32_t capacity, uint32_t start_pos, uint32_t n_tokens, void* payload, size_t payload_capacity) {
    const char* fn = "hq_tq_kv_capture";
    if (head_dim != 256 && head_dim != 512) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: head_dim %u (256 or 512)", fn, head_dim);
    if ((uint64_t)start_pos + n_tokens > capacity)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: positions %u..%llu past the capacity %u", fn, start_pos,
                    (unsigned long long)start_pos + n_tokens, capacity);
    if (!codes || !norms || !payload) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    hq_tqp_header h{2, 8, head_dim, n_kv_heads, n_tokens, HQ_TQP_FLAG_HADAMARD_ROTATED, 1.0};
    const size_t ib = hq_tqp_indices_bytes(&h), nb = hq_tqp_norms_bytes(&h);
    if (payload_capacity < HQ_TQP_HEADER_BYTES + ib + nb)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: payload holds %zu bytes, %zu needed", fn, payload_capacity,
                    HQ_TQP_HEADER_BYTES + ib + nb);
    uint8_t* o = static_cast<uint8_t*>(payload);
    // header first (no body yet: the sizes are checked against zero-length streams by hand)
    put_u32(o, MAGIC_V2), put_u32(o + 4, 2), put_u32(o + 8, 8), put_u32(o + 12, head_dim), put_u32(o + 16, n_kv_heads);
    put_u32(o + 20, n_tokens), put_u32(o + 24, h.flags), put_u32(o + 28, 0);
    uint64_t sbits;
    memcpy(&sbits, &h.scale, 8);
    put_u32(o + 32, (uint32_t)sbits), put_u32(o + 36, (uint32_t)(sbits >> 32));
    if (n_kv_heads == 0 || n_tokens == 0) return HQ_OK;
    hipStream_t s = (hipStream_t)stream;
    const size_t npp = norms_per_pos(head_dim);
    const size_t row_c = (size_t)n_tokens * head_dim, row_n = (size_t)n_tokens * npp * 4;
    // one row per kv head: n_tokens consecutive positions are contiguous inside a head
    if (int rc = hq::check_hip(hipMemcpy2DAsync(o + HQ_TQP_HEADER_BYTES, row_c, codes + (size_t)start_pos * head_dim,
                                                (size_t)capacity * head_dim, row_c, n_kv_heads, hipMemcpyDeviceToHost, s),
                               "capture: codes copy"))
        return rc;
    if (int rc = hq::check_hip(hipMemcpy2DAsync(o + HQ_TQP_HEADER_BYTES + ib, row_n,
                                                reinterpret_cast<const uint8_t*>(norms) + (size_t)start_pos * npp * 4,
                                                (size_t)capacity * npp * 4, row_n, n_kv_heads, hipMemcpyDeviceToHost, s),
                               "capture: norms copy"))
        return rc;
    return hq::check_hip(hipStreamSynchronize(s), "capture: synchronize");
}

int hq_tq_kv_restore(void* stream, const void* payload, size_t len, uint8_t* codes, float* norms, uint32_t n_kv_heads,
                     uint32_t head_dim, uint32_t capacity, uint32_t start_pos) {
    const char* fn = "hq_tq_kv_restore";
    hq_tqp_header h;
    size_t io = 0, no = 0;
    if (int rc = hq_tqp_unpack(payload, len, &h, &io, &no)) return rc;
    if (h.codec_version != 2) return fail(HQ_ERR_UNSUPPORTED, "%s: a version-1 envelope carries no norms", fn);
    if (h.bits_per_coord != 8) return fail(HQ_ERR_UNSUPPORTED, "%s: %u bits per coordinate (the cache holds one byte per code)", fn, h.bits_per_coord);
    if (h.head_dim != head_dim || h.n_kv_heads != n_kv_heads)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: envelope is %u heads x %u, cache is %u x %u", fn, h.n_kv_heads, h.head_dim,
                    n_kv_heads, head_dim);
    if (head_dim != 256 && head_dim != 512) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: head_dim %u (256 or 512)", fn, head_dim);
    if ((uint64_t)start_pos + h.n_tokens > capacity)
        return fail(HQ_ERR_INVALID_ARGUMENT, "%s: positions %u..%llu past the capacity %u", fn, start_pos,
                    (unsigned long long)start_pos + h.n_tokens, capacity);
    if (!codes || !norms) return fail(HQ_ERR_INVALID_ARGUMENT, "%s: null buffer", fn);
    if (n_kv_heads == 0 || h.n_tokens == 0) return HQ_OK;
    hipStream_t s = (hipStream_t)stream;
    const uint8_t* p = static_cast<const uint8_t*>(payload);
    const size_t npp = norms_per_pos(head_dim);
    const size_t row_c = (size_t)h.n_tokens * head_dim, row_n = (size_t)h.n_tokens * npp * 4;
    if (int rc = hq::check_hip(hipMemcpy2DAsync(codes + (size_t)start_pos * head_dim, (size_t)capacity * head_dim, p + io, row_c,
                                                row_c, n_kv_heads, hipMemcpyHostToDevice, s),
                               "restore: codes copy"))
        return rc;
    if (int rc = hq::check_hip(hipMemcpy2DAsync(reinterpret_cast<uint8_t*>(norms) + (size_t)start_pos * npp * 4,
                                                (size_t)capacity * npp * 4, p + no, row_n, row_n, n_kv_heads,
                                                hipMemcpyHostToDevice, s),
                               "restore: norms copy"))
        return rc;
    return hq::check_hip(hipStreamSynchronize(s), "restore: synchronize");
}

}  // extern "C"

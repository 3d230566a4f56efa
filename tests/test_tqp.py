"""TurboQuant block envelope ("TQP1" / "TQP2"): the library's packer / parser against the oracle
restatement and against the reference's own known answers (kv_persist/families/tq_packed.rs tests
:1625-1852 and :2139-2200).  Host code only: runs without a GPU."""
import ctypes
import struct

import numpy as np
import pytest

from hf2q_amd import lib, ops
from oracle import tqp


def _hdr(version, bits, n_kv, n_tok, hd, flags=1, scale=0.5):
    return (ops.TqPackedHeader(version, bits, hd, n_kv, n_tok, flags, scale),
            tqp.Header(version, bits, hd, n_kv, n_tok, flags, scale))


def test_known_answers_of_the_reference():
    # tq_packed_v1_magic_is_frozen / v2: "TQP1" = 0x31505154, "TQP2" = 0x32505154; header is 40 bytes
    for version, magic, tag in ((1, 0x31505154, b"TQP1"), (2, 0x32505154, b"TQP2")):
        h, o = _hdr(version, 8, 1, 0, 256)
        p = ops.pack_tq_payload(h, b"")
        assert len(p) == 40 and p[:4] == tag and struct.unpack_from("<I", p)[0] == magic
        assert struct.unpack_from("<I", p, 4)[0] == version
        assert p == tqp.pack(o, b"")
    # tq_packed_v1_indices_bytes_len_formula
    assert _hdr(1, 8, 4, 100, 256)[0].indices_bytes_len() == 4 * 100 * 256
    assert _hdr(1, 4, 4, 100, 256)[0].indices_bytes_len() == 4 * 100 * 256 // 2
    assert _hdr(1, 2, 4, 100, 256)[0].indices_bytes_len() == 4 * 100 * 256 // 4
    assert _hdr(1, 3, 1, 1, 5)[0].indices_bytes_len() == 2
    # norms_per_pos: 1 up to head_dim 256, 2 at 512 (tq_packed.rs:420-440); none at version 1
    assert _hdr(2, 8, 8, 64, 256)[0].norms_bytes_len() == 8 * 64 * 4
    assert _hdr(2, 8, 8, 64, 512)[0].norms_bytes_len() == 8 * 64 * 2 * 4
    assert _hdr(2, 8, 8, 64, 128)[0].norms_bytes_len() == 8 * 64 * 4
    assert _hdr(1, 8, 8, 64, 512)[0].norms_bytes_len() == 0


@pytest.mark.parametrize("version,bits,n_kv,n_tok,hd", [(1, 4, 8, 256, 256), (1, 8, 2, 64, 256), (2, 8, 2, 33, 512),
                                                      (2, 3, 1, 7, 5), (2, 8, 4, 1, 256)])
def test_round_trip_byte_exact(version, bits, n_kv, n_tok, hd):
    """tq_packed_v1_round_trip_byte_exact: pack -> unpack -> pack returns the same bytes."""
    rng = np.random.default_rng(bits * n_tok)
    h, o = _hdr(version, bits, n_kv, n_tok, hd, flags=3, scale=1.0 / 3.0)
    idx = rng.integers(0, 256, o.indices_bytes_len(), dtype=np.uint8).tobytes()
    nrm = rng.standard_normal(o.norms_bytes_len() // 4).astype("<f4").tobytes()
    a = ops.pack_tq_payload(h, idx, nrm)
    assert a == tqp.pack(o, idx, nrm) and len(a) == h.total_bytes() == o.total_bytes()
    h2, i2, n2 = ops.unpack_tq_payload(a)
    assert h2 == h and i2 == idx and n2 == nrm
    assert ops.pack_tq_payload(h2, i2, n2) == a
    oh, oi, on = tqp.unpack(a)
    assert (oh, oi, on) == (o, idx, nrm)


def test_rejections():
    h, o = _hdr(1, 4, 2, 16, 64)
    idx = bytes(o.indices_bytes_len())
    good = ops.pack_tq_payload(h, idx)

    def bad(payload, kind, needle):
        with pytest.raises(tqp.TqEnvelopeError) as e:
            tqp.unpack(payload)
        assert e.value.kind == kind
        with pytest.raises(ops.HqError) as e:
            ops.unpack_tq_payload(payload)
        assert e.value.status == 1 and needle in str(e.value)

    bad(b"XXXX" + bytes(36), "BadMagic", "bad magic")                                      # …_rejects_bad_magic
    bad(good[:4] + struct.pack("<I", 7) + good[8:], "UnsupportedCodecVersion", "codec version 7")
    bad(good[:8] + struct.pack("<I", 0) + good[12:], "InvalidBitsPerCoord", "bits_per_coord 0")
    bad(good[:8] + struct.pack("<I", 9) + good[12:], "InvalidBitsPerCoord", "bits_per_coord 9")
    bad(bytes(16), "Truncated", "truncated")                                               # …_rejects_truncated_header
    bad(good[:28] + struct.pack("<I", 0xDEADBEEF) + good[32:], "ReservedNonZero", "deadbeef")
    bad(good[:-1], "PayloadSizeMismatch", "size mismatch")
    bad(good + b"\0", "PayloadSizeMismatch", "size mismatch")
    with pytest.raises(ops.HqError) as e:                                                  # …_pack_rejects_short_indices
        ops.pack_tq_payload(h, idx[:-1])
    assert e.value.status == 1 and "size mismatch" in str(e.value)
    with pytest.raises(tqp.TqEnvelopeError):
        tqp.pack(o, idx[:-1])
    h2, _ = _hdr(2, 8, 2, 16, 256)
    with pytest.raises(ops.HqError):                                                       # version 2 needs its norms
        ops.pack_tq_payload(h2, bytes(h2.indices_bytes_len()), b"")


def test_stream_lengths_do_not_wrap():
    """Header fields are 32 bits each: the largest products exceed size_t and must not come back truncated."""
    L = lib.load()
    h = lib.TqpHeader()
    h.codec_version, h.bits_per_coord, h.head_dim, h.n_kv_heads, h.n_tokens = 2, 8, 0xFFFFFF00, 0xFFFFFFFF, 0xFFFFFFFF
    size_max = ctypes.c_size_t(-1).value
    assert L.hq_tqp_indices_bytes(ctypes.byref(h)) == size_max
    assert L.hq_tqp_norms_bytes(ctypes.byref(h)) == size_max
    assert L.hq_tqp_total_bytes(ctypes.byref(h)) == size_max
    h.head_dim, h.n_kv_heads, h.n_tokens = 256, 2, 5
    assert L.hq_tqp_indices_bytes(ctypes.byref(h)) == 2 * 5 * 256 and L.hq_tqp_norms_bytes(ctypes.byref(h)) == 2 * 5 * 4

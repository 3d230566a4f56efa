"""CPU restatement of the reference's TurboQuant block envelope codec ("TQP1" / "TQP2").

Test infrastructure only: the tests compare the library's packer / parser with it.  Follows
src/serve/kv_persist/families/tq_packed.rs: header layout :37-52 and :330-352, indices_bytes_len
:167-178, norms_bytes_len :433-438, pack :199-226 / :459-489, unpack :243-311 / :491-566 (error
order: Truncated, BadMagic, UnsupportedCodecVersion, InvalidBitsPerCoord, ReservedNonZero,
PayloadSizeMismatch).  Pinned by the reference's own known answers (tq_packed.rs:1784-1852): magic
0x31505154 = b"TQP1" and 0x32505154 = b"TQP2", 40-byte header, the four indices_bytes_len cases.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass

HEADER_BYTES = 40
MAGIC = {1: 0x31505154, 2: 0x32505154}


class TqEnvelopeError(ValueError):
    def __init__(self, kind: str, detail=None):
        super().__init__(f"{kind}: {detail}")
        self.kind = kind
        self.detail = detail


@dataclass
class Header:
    codec_version: int
    bits_per_coord: int
    head_dim: int
    n_kv_heads: int
    n_tokens: int
    flags: int
    scale: float

    def indices_bytes_len(self) -> int:
        return -(-(self.n_kv_heads * self.n_tokens * self.head_dim * self.bits_per_coord) // 8)

    def norms_bytes_len(self) -> int:
        if self.codec_version != 2:
            return 0
        return self.n_kv_heads * self.n_tokens * max(1, self.head_dim // 256) * 4

    def total_bytes(self) -> int:
        return HEADER_BYTES + self.indices_bytes_len() + self.norms_bytes_len()


def pack(h: Header, indices: bytes, norms_le: bytes = b"") -> bytes:
    if len(indices) != h.indices_bytes_len():
        raise TqEnvelopeError("PayloadSizeMismatch", (h.indices_bytes_len(), len(indices)))
    if len(norms_le) != h.norms_bytes_len():
        raise TqEnvelopeError("PayloadSizeMismatch", (h.norms_bytes_len(), len(norms_le)))
    head = struct.pack("<8Id", MAGIC[h.codec_version], h.codec_version, h.bits_per_coord, h.head_dim, h.n_kv_heads,
                       h.n_tokens, h.flags, 0, h.scale)
    return head + bytes(indices) + bytes(norms_le)


def unpack(payload: bytes):
    if len(payload) < HEADER_BYTES:
        raise TqEnvelopeError("Truncated", len(payload))
    magic, version, bits, head_dim, n_kv, n_tok, flags, reserved, scale = struct.unpack_from("<8Id", payload, 0)
    if magic not in MAGIC.values():
        raise TqEnvelopeError("BadMagic", magic)
    if MAGIC.get(version) != magic:
        raise TqEnvelopeError("UnsupportedCodecVersion", version)
    if bits == 0 or bits > 8:
        raise TqEnvelopeError("InvalidBitsPerCoord", bits)
    if reserved != 0:
        raise TqEnvelopeError("ReservedNonZero", reserved)
    h = Header(version, bits, head_dim, n_kv, n_tok, flags, scale)
    body = len(payload) - HEADER_BYTES
    if body != h.indices_bytes_len() + h.norms_bytes_len():
        raise TqEnvelopeError("PayloadSizeMismatch", (h.indices_bytes_len() + h.norms_bytes_len(), body))
    i_end = HEADER_BYTES + h.indices_bytes_len()
    return h, payload[HEADER_BYTES:i_end], payload[i_end:]

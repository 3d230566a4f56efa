"""GGUF reader (CPU part): the writer restatement against the reference writer's own known answers, then
the C reader against files made by it."""
import struct

import numpy as np
import pytest

from hf2q_amd import lib, ops
from oracle import gguf as W


def test_writer_known_answers_of_the_reference():
    # writer.rs:625-638: no tensors, no metadata -> 24-byte header padded to 32
    data, _ = W.build([], [])
    assert len(data) == 32 and data[:4] == b"GGUF" and struct.unpack("<I", data[4:8])[0] == 3
    assert data[24:] == b"\0" * 8
    # writer.rs:603-623: two Q4_0 rows of 18 bytes -> offsets 0 and 32
    data, offs = W.build([], [("a.weight", [32], 2, bytes(range(18))), ("b.weight", [32], 2, bytes(range(100, 118)))])
    assert offs == [0, 32]
    # writer.rs:424-445: counts sit at bytes 8..24
    data, _ = W.build([("general.name", W.STRING, "tiny")], [("t", [32], 2, bytes(18))])
    assert struct.unpack("<QQ", data[8:24]) == (1, 1)
    # types.rs:96-101: a string is a u64 length and the bytes
    assert W.metadata_kv("k", W.U32, 7) == b"\x01\0\0\0\0\0\0\0k" + struct.pack("<II", 4, 7)


@pytest.fixture()
def tiny(tmp_path):
    rng = np.random.default_rng(3)
    tensors = [
        ("blk.0.ffn_gate.weight", [256, 4], 12, rng.integers(0, 256, 4 * 144, dtype=np.uint8).tobytes()),
        ("blk.0.ffn_down_exps.weight", [512, 3, 2], 14, rng.integers(0, 256, 2 * 3 * 2 * 210, dtype=np.uint8).tobytes()),
        ("output_norm.weight", [8], 0, np.arange(8, dtype=np.float32).tobytes()),
        ("blk.0.attn_q.weight", [64, 2], 8, rng.integers(0, 256, 4 * 34, dtype=np.uint8).tobytes()),
    ]
    meta = [("general.architecture", W.STRING, "qwen35moe"), ("qwen35moe.block_count", W.U32, 40),
            ("qwen35moe.rope.freq_base", W.F32, 1.0e7), ("tokenizer.ggml.tokens", W.ARRAY, ["a", "bc", ""], W.STRING),
            ("qwen35moe.expert_count", W.U64, 256), ("some.flag", W.BOOL, 1), ("some.ints", W.ARRAY, [1, 2, 3], W.I32),
            ("neg", W.I32, -5)]
    path = tmp_path / "tiny.gguf"
    offs = W.write(str(path), meta, tensors)
    return str(path), meta, tensors, offs


def test_reader_directory_metadata_and_bytes(tiny):
    path, meta, tensors, offs = tiny
    with ops.GgufFile.open(path) as g:
        assert g.tensor_count() == 4 and g.metadata_count() == len(meta)
        assert g.tensor_names() == [t[0] for t in tensors]
        assert g.metadata_keys() == [m[0] for m in meta]
        assert g.metadata_string("general.architecture") == "qwen35moe"
        assert g.metadata_u64("qwen35moe.block_count") == 40 and g.metadata_u64("qwen35moe.expert_count") == 256
        assert g.metadata_u64("some.flag") == 1
        assert g.metadata_f64("qwen35moe.rope.freq_base") == 1.0e7
        with pytest.raises(lib.HqError):
            g.metadata_u64("neg")
        with pytest.raises(lib.HqError):
            g.metadata_u64("general.architecture")
        with pytest.raises(lib.HqError):
            g.metadata_string("missing.key")
        for (name, dims, t, payload) in tensors:
            info = g.tensor_info(name)
            assert info.ggml_dtype == t and info.shape == tuple(dims) and info.byte_len == len(payload)
            assert info.cols == dims[0] and info.rows == int(np.prod(dims[1:])) if len(dims) > 1 else True
            assert g.tensor_bytes(name) == payload
        # an expert stack is one contiguous tensor: stride = byte_len / experts (forward_mlx.rs:2438-2460)
        ex = g.tensor_info("blk.0.ffn_down_exps.weight")
        assert ex.byte_len // ex.shape[2] == 3 * 2 * 210
        with pytest.raises(lib.HqError):
            g.tensor_info("nope")
    # data offsets are absolute and aligned
    L = lib.load()
    import ctypes
    h = ctypes.c_void_p()
    lib.check(L.hq_gguf_open(path.encode(), ctypes.byref(h)))
    ti = lib.GgufTensorInfo()
    lib.check(L.hq_gguf_tensor_info_by_name(h, b"blk.0.attn_q.weight", ctypes.byref(ti)))
    raw = open(path, "rb").read()
    assert ti.data_offset % 32 == 0 and raw[ti.data_offset:ti.data_offset + ti.byte_len] == tensors[3][3]
    assert L.hq_gguf_alignment(h) == 32
    L.hq_gguf_close(h)


def test_reader_rejects_malformed_files(tmp_path, tiny):
    path, _, _, _ = tiny
    raw = open(path, "rb").read()

    def opens(data):
        p = tmp_path / "bad.gguf"
        p.write_bytes(data)
        try:
            ops.GgufFile.open(str(p)).close()
            return True
        except lib.HqError:
            return False

    assert opens(raw)
    assert not opens(b"GGML" + raw[4:])                       # magic
    assert not opens(raw[:4] + struct.pack("<I", 1) + raw[8:])  # version
    assert not opens(raw[:40])                                # truncated metadata
    assert not opens(raw[:len(raw) - 64])                     # last tensor reaches past the end
    assert not opens(b"")                                     # empty file
    with pytest.raises(lib.HqError):
        ops.GgufFile.open(str(tmp_path / "does-not-exist.gguf"))
    # row length that is not a multiple of the block size (quantizer.rs:57-71)
    data, _ = W.build([], [("t", [100], 12, bytes(144))])
    assert not opens(data)
    # unknown ggml type
    data, _ = W.build([], [("t", [32], 99, bytes(32))])
    assert not opens(data)
    # an element count whose byte length does not fit 64 bits (F32 = type 0: 2^62 + 8 elements would wrap to 32 bytes)
    data, _ = W.build([], [("t", [(1 << 62) + 8], 0, bytes(32))])
    assert not opens(data)
    data, _ = W.build([], [("t", [1 << 62], 0, bytes(32))])
    assert not opens(data)
    # general.alignment is honoured
    data, offs = W.build([("general.alignment", W.U32, 64)], [("a", [32], 8, bytes(34)), ("b", [32], 8, bytes(range(34)))], 64)
    p = tmp_path / "a64.gguf"
    p.write_bytes(data)
    with ops.GgufFile.open(str(p)) as g:
        assert offs == [0, 64] and g.tensor_bytes("b") == bytes(range(34))

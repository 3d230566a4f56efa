"""CPU oracle for the hf2q quantized-matmul hot path.

TEST INFRASTRUCTURE ONLY.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package; the shipped
library (``hf2q_amd``) never does.  The arithmetic lives in ``hf2q_oracle.c``
(plain C, scalar, one function per reference function, each citing the
reference file:line it restates); this module is a ctypes/numpy front end.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libhf2q_oracle.so")

Q4_0, Q8_0, Q4_K, Q5_K, Q6_K = 2, 8, 12, 13, 14  # ggml_type.rs:18-53
BLOCK_ELEMS = {Q4_0: 32, Q8_0: 32, Q4_K: 256, Q5_K: 256, Q6_K: 256}
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, Q4_K: 144, Q5_K: 176, Q6_K: 210}

# kv_cache.rs:3871-3876 (same 32 bytes as in hf2q_oracle.c; kept here so tests
# can build the explicit sign vector independently of the C code).
TBQ_SIGNS_256 = bytes.fromhex(
    "a73b91f46dc2580eb37f24d68945ea1c63afd852970be13d76c419fe4a852cdb"
)


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (idempotent unless ``force``)."""
    src = os.path.join(_HERE, "hf2q_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libhf2q_oracle.so"])
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        c = ctypes
        vp, i64, i32, f32 = c.c_void_p, c.c_int64, c.c_int, c.c_float
        L.hq_oracle_quantize.argtypes = [vp, i64, i64, i32, vp, vp, i32]
        L.hq_oracle_quantize.restype = i32
        L.hq_oracle_dequantize.argtypes = [vp, i64, i32, vp, i32]
        L.hq_oracle_dequantize.restype = i32
        L.hq_oracle_matmul_a_by_bt.argtypes = [vp, vp, i64, i64, i64, vp, i32]
        L.hq_oracle_matmul_a_by_bt.restype = None
        L.hq_oracle_qmatmul_f64.argtypes = [vp, i32, vp, i64, i64, i64, i32, vp, i32]
        L.hq_oracle_qmatmul_f64.restype = i32
        L.hq_oracle_qmatmul_id_f64.argtypes = [vp, i32, vp, vp, i64, i64, i64, i64, i64, i64, i32, vp, i32]
        L.hq_oracle_qmatmul_id_f64.restype = i32
        L.hq_oracle_softmax_topk_renorm.argtypes = [vp, i64, i64, i64, vp, vp]
        L.hq_oracle_softmax_topk_renorm.restype = None
        L.hq_oracle_moe_ffn.argtypes = [vp, i64, i64, i64, i64, i64, i64] + [vp] * 9
        L.hq_oracle_moe_ffn.restype = None
        L.hq_oracle_fwht_sign_premult.argtypes = [vp, i32, i32]
        L.hq_oracle_fwht_sign_undo.argtypes = [vp, i32, i32]
        L.hq_oracle_tq_encode_int8.argtypes = [vp, i32, i32, i32, i32, vp, vp]
        L.hq_oracle_tq_attention.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, f32,
                                             i32, i32, f32, i32, f32, vp]
        L.hq_oracle_tq_attention.restype = i32
        L.hq_oracle_tq_dequantize.argtypes = [vp, vp, vp, i32, i32, i32, i32, i32, f32, vp]
        L.hq_oracle_tq_dequantize.restype = i32
        L.hq_oracle_nearest_int.argtypes = [f32]
        L.hq_oracle_nearest_int.restype = i32
        L.hq_oracle_f32_to_f16.argtypes = [f32]
        L.hq_oracle_f32_to_f16.restype = c.c_uint16
        L.hq_oracle_f16_to_f32.argtypes = [c.c_uint16]
        L.hq_oracle_f16_to_f32.restype = f32
        L.hq_oracle_silu.argtypes = [f32]
        L.hq_oracle_silu.restype = f32
        _lib = L
    return _lib


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dt) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dt)


def n_threads_default() -> int:
    return max(1, min(16, os.cpu_count() or 1))


def quantize(src, n_per_row: int, ggml_type: int, imatrix=None, threads: int = 1) -> np.ndarray:
    """quantizer.rs:51-102 — f32 rows -> packed GGML blocks (uint8)."""
    src = _c(src, np.float32).reshape(-1)
    be, bb = BLOCK_ELEMS[ggml_type], BLOCK_BYTES[ggml_type]
    if n_per_row % be or src.size % n_per_row:
        raise ValueError(f"n_per_row {n_per_row} / len {src.size} not aligned to block {be}")
    im = None
    if imatrix is not None:
        im = _c(imatrix, np.float32)
        if im.size != n_per_row:
            raise ValueError("imatrix length must equal n_per_row")
    out = np.empty(src.size // be * bb, dtype=np.uint8)
    rc = lib().hq_oracle_quantize(_p(src), src.size, n_per_row, ggml_type, _p(im), _p(out), threads)
    if rc:
        raise ValueError(f"hq_oracle_quantize rc={rc}")
    return out


def dequantize(blocks, ggml_type: int, threads: int = 1) -> np.ndarray:
    blocks = _c(blocks, np.uint8).reshape(-1)
    be, bb = BLOCK_ELEMS[ggml_type], BLOCK_BYTES[ggml_type]
    if blocks.size % bb:
        raise ValueError("byte length is not a whole number of blocks")
    n = blocks.size // bb * be
    out = np.empty(n, dtype=np.float32)
    rc = lib().hq_oracle_dequantize(_p(blocks), n, ggml_type, _p(out), threads)
    if rc:
        raise ValueError(f"hq_oracle_dequantize rc={rc}")
    return out


def matmul_a_by_bt(lhs, rhs, m: int, k: int, n: int, threads: int = 1) -> np.ndarray:
    """ffn.rs:38-50 — scalar f32 out[m,n] = lhs[m,k] . rhs[n,k]^T."""
    lhs, rhs = _c(lhs, np.float32), _c(rhs, np.float32)
    out = np.empty((m, n), dtype=np.float32)
    lib().hq_oracle_matmul_a_by_bt(_p(lhs), _p(rhs), m, k, n, _p(out), threads)
    return out


def _xdt(x: np.ndarray):
    if x.dtype == np.float32:
        return 0
    if x.dtype == np.uint16:  # bf16 bit patterns
        return 1
    raise TypeError("x must be float32 or uint16 (bf16 bits)")


def qmatmul_f64(x, blocks, m: int, n: int, k: int, ggml_type: int, threads: int | None = None) -> np.ndarray:
    """float64 y[m,n] = x[m,k] . dequant(W)[n,k]^T; x is f32 or bf16 bits (uint16)."""
    x = np.ascontiguousarray(x)
    blocks = _c(blocks, np.uint8)
    y = np.empty((m, n), dtype=np.float64)
    rc = lib().hq_oracle_qmatmul_f64(_p(x), _xdt(x), _p(blocks), m, n, k, ggml_type, _p(y),
                                     threads or n_threads_default())
    if rc:
        raise ValueError(f"hq_oracle_qmatmul_f64 rc={rc}")
    return y


def qmatmul_id_f64(x, stack, ids, n_tokens, top_k, n, k, n_experts, expert_stride, ggml_type,
                   threads: int | None = None) -> np.ndarray:
    x = np.ascontiguousarray(x)
    stack = _c(stack, np.uint8)
    ids = _c(ids, np.uint32)
    y = np.empty((n_tokens * top_k, n), dtype=np.float64)
    rc = lib().hq_oracle_qmatmul_id_f64(_p(x), _xdt(x), _p(stack), _p(ids), n_tokens, top_k, n, k,
                                        n_experts, expert_stride, ggml_type, _p(y),
                                        threads or n_threads_default())
    if rc:
        raise ValueError(f"hq_oracle_qmatmul_id_f64 rc={rc}")
    return y


def softmax_topk_renorm(logits, seq_len: int, n_experts: int, topk: int):
    logits = _c(logits, np.float32)
    idx = np.empty(seq_len * topk, dtype=np.uint32)
    w = np.empty(seq_len * topk, dtype=np.float32)
    lib().hq_oracle_softmax_topk_renorm(_p(logits), seq_len, n_experts, topk, _p(idx), _p(w))
    return idx, w


def moe_ffn(x, h, ne, topk, m_moe, m_sh, router, eg, eu, ed, sgl, sg, su, sd) -> np.ndarray:
    """ffn.rs:179-336 moe_ffn_cpu_ref (all f32)."""
    arrs = [_c(a, np.float32) for a in (x, router, eg, eu, ed, sgl, sg, su, sd)]
    seq = arrs[0].size // h
    out = np.empty((seq, h), dtype=np.float32)
    lib().hq_oracle_moe_ffn(_p(arrs[0]), seq, h, ne, topk, m_moe, m_sh, *[_p(a) for a in arrs[1:]],
                            _p(out))
    return out


def fwht_sign_premult(buf, n_heads: int, head_dim: int) -> np.ndarray:
    b = _c(buf, np.float32).copy()
    lib().hq_oracle_fwht_sign_premult(_p(b), n_heads, head_dim)
    return b


def fwht_sign_undo(buf, n_heads: int, head_dim: int) -> np.ndarray:
    b = _c(buf, np.float32).copy()
    lib().hq_oracle_fwht_sign_undo(_p(b), n_heads, head_dim)
    return b


def tq_encode_int8(kv, n_kv_heads, head_dim, capacity, pos, codes, norms) -> None:
    """Encode one position (kv: [n_kv_heads, head_dim] f32) in place into codes/norms."""
    kv = _c(kv, np.float32)
    assert codes.dtype == np.uint8 and norms.dtype == np.float32
    lib().hq_oracle_tq_encode_int8(_p(kv), n_kv_heads, head_dim, capacity, pos, _p(codes), _p(norms))


def tq_dequantize(codes, norms, lut, n_kv_heads, head_dim, capacity, start_pos, n_tokens,
                  scale_factor_d512=1.0, unrotate=False) -> np.ndarray:
    """kv_cache.rs:431-495 (rotated domain) and :497-583 (followed by fwht_sign_undo over every
    (head, token) chunk): f32 [n_kv_heads, n_tokens, head_dim]."""
    lutc = None if lut is None else _c(lut, np.float32)
    out = np.empty((n_kv_heads, n_tokens, head_dim), dtype=np.float32)
    rc = lib().hq_oracle_tq_dequantize(_p(codes), _p(norms), _p(lutc), n_kv_heads, head_dim, capacity, start_pos,
                                       n_tokens, scale_factor_d512, _p(out))
    if rc:
        raise ValueError(f"hq_oracle_tq_dequantize rc={rc}")
    if unrotate:
        out = fwht_sign_undo(out.reshape(-1, head_dim), n_kv_heads * n_tokens, head_dim).reshape(out.shape)
    return out


def tq_attention(q, k_codes, k_norms, v_codes, v_norms, lut, num_heads, num_kv_heads, head_dim,
                 kv_seq_len, kv_capacity, scale, mask_type=0, sliding_window=0, softcap=0.0,
                 ring_start=0, scale_factor_d512=1.0) -> np.ndarray:
    q = _c(q, np.float32)
    lutc = None if lut is None else _c(lut, np.float32)
    out = np.empty((num_heads, head_dim), dtype=np.float64)
    rc = lib().hq_oracle_tq_attention(_p(q), _p(k_codes), _p(k_norms), _p(v_codes), _p(v_norms),
                                      _p(lutc), num_heads, num_kv_heads, head_dim, kv_seq_len,
                                      kv_capacity, scale, mask_type, sliding_window, softcap,
                                      ring_start, scale_factor_d512, _p(out))
    if rc:
        raise ValueError(f"hq_oracle_tq_attention rc={rc}")
    return out


def f32_to_bf16_bits(x) -> np.ndarray:
    """Round-to-nearest-even f32 -> bf16 bit patterns (uint16)."""
    u = _c(x, np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + 0x7FFF
    return ((u + r) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def mulberry32_imatrix(n: int, seed: int) -> np.ndarray:
    """q4_k.rs:371-384 make_imatrix: mulberry32 -> |2u-1| + 1e-3."""
    out = np.empty(n, dtype=np.float32)
    state = seed & 0xFFFFFFFF
    M = 0xFFFFFFFF
    for i in range(n):
        state = (state + 0x6D2B79F5) & M
        t = state
        t = ((t ^ (t >> 15)) * (t | 1)) & M
        t ^= (t + (((t ^ (t >> 7)) * (t | 61)) & M)) & M
        u = t ^ (t >> 14)
        v = np.float32(np.float32(u) / np.float32(M)) * np.float32(2.0) - np.float32(1.0)
        out[i] = np.float32(abs(v)) + np.float32(1e-3)
    return out

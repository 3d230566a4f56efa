"""Pins the CPU oracle against the reference's own golden vectors and against
mathematics it cannot fake (exact rational arithmetic, closed forms).  CPU only."""
import os
from fractions import Fraction

import numpy as np
import pytest

from _util import GOLDEN

Q4_0, Q8_0, Q4_K, Q5_K, Q6_K = 2, 8, 12, 13, 14
CASES = [("q4_k_512", Q4_K, 512), ("q6_k_512", Q6_K, 512), ("q8_0_64", Q8_0, 64), ("q5_k_512", Q5_K, 512),
         ("q4_0_64", Q4_0, 64)]


def _load(name):
    return np.fromfile(os.path.join(GOLDEN, "ggml_quants", name), dtype=np.uint8)


@pytest.mark.parametrize("name,t,npr", CASES)
@pytest.mark.parametrize("variant", ["noim", "im"])
def test_quantizer_byte_equal_to_reference_fixture(oracle, name, t, npr, variant):
    # q4_k.rs:386-403, q6_k.rs:272-289, q8_0.rs:106-125, q5_k.rs:395-428, q4_0.rs:196-217: assert byte equality.
    x = _load(f"{name}_{variant}_input.bin").view(np.float32)
    expected = _load(f"{name}_{variant}_expected.bin")
    im = None
    if variant == "im":
        # Q8_0's test passes a vector of ones, the K-quants mulberry32 seed 2.
        im = np.ones(npr, np.float32) if t == Q8_0 else oracle.mulberry32_imatrix(npr, 2)
    got = oracle.quantize(x, npr, t, im)
    assert got.size == expected.size
    assert np.array_equal(got, expected)


def test_fixture_shapes():
    assert _load("q4_k_512_noim_expected.bin").size == 4 * 144
    assert _load("q6_k_512_noim_expected.bin").size == 4 * 210
    assert _load("q8_0_64_noim_expected.bin").size == 4 * 34
    assert _load("q5_k_512_noim_expected.bin").size == 4 * 176
    assert _load("q4_0_64_noim_expected.bin").size == 4 * 18
    assert np.array_equal(_load("q4_k_512_noim_input.bin"), _load("q4_k_512_im_input.bin"))


def test_nearest_int_table(oracle):
    # common.rs:525-539
    L = oracle.lib()
    table = {0.0: 0, 1.0: 1, -1.0: -1, 1.4: 1, 1.6: 2, -1.4: -1, -1.6: -2, 0.5: 0, 1.5: 2, 2.5: 2, 3.5: 4}
    for v, e in table.items():
        assert L.hq_oracle_nearest_int(v) == e


def test_f16_roundtrip_all_bit_patterns(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    for b in range(0, 65536, 97):
        f = L.hq_oracle_f16_to_f32(b)
        if np.isnan(ref[b]):
            assert np.isnan(f)
        else:
            assert f == ref[b]
            assert L.hq_oracle_f32_to_f16(f) == b
    # rounding: ties to even and subnormal/overflow behaviour agree with numpy
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(2000).astype(np.float32) * s for s in (1e-8, 1e-5, 1e-3, 1, 1e3, 7e4)])
    xs = np.concatenate([xs, np.float32([0.0, -0.0, 65504.0, 65520.0, 65519.99, 5.9604645e-8, 2.9802322e-8, 2.98e-8])])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.hq_oracle_f32_to_f16(float(v)) for v in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---- dequantisation: exact rational evaluation of the block formulas -----------------

def _f16(b0, b1):
    return Fraction(float(np.array([int(b0) | (int(b1) << 8)], dtype=np.uint16).view(np.float16)[0]))


def _round_f32(fr: Fraction) -> np.float32:
    # Fraction -> nearest f32 (ties to even) through exact integer arithmetic
    if fr == 0:
        return np.float32(0.0)
    return np.float32(float(fr))  # float(Fraction) is correctly rounded to f64; values here have
    # <= 31 significant bits so f64 holds them exactly and the f32 cast rounds once.


def _ref_dequant_q4k(block):
    d, dmin = _f16(block[0], block[1]), _f16(block[2], block[3])
    q = block[4:16]
    out = []
    for j in range(8):
        if j < 4:
            sc, m = int(q[j]) & 63, int(q[j + 4]) & 63
        else:
            sc = (int(q[j + 4]) & 0xF) | ((int(q[j - 4]) >> 6) << 4)
            m = (int(q[j + 4]) >> 4) | ((int(q[j]) >> 6) << 4)
        qs = block[16 + 32 * (j // 2): 16 + 32 * (j // 2) + 32]
        for l in range(32):
            nib = (int(qs[l]) >> (4 * (j & 1))) & 0xF
            out.append(_round_f32(d * int(sc) * nib - dmin * int(m)))
    return np.array(out, dtype=np.float32)


def _ref_dequant_q6k(block):
    d = _f16(block[208], block[209])
    ql, qh, sc = block[0:128], block[128:192], block[192:208].view(np.int8)
    out = [None] * 256
    for h in range(2):
        for l in range(32):
            for r in range(4):
                lo = int(ql[64 * h + 32 * (r & 1) + l])
                nib = (lo >> 4) if r >= 2 else (lo & 0xF)
                hi = (int(qh[32 * h + l]) >> (2 * r)) & 3
                q = (nib | (hi << 4)) - 32
                s = int(sc[8 * h + 2 * r + l // 16])
                out[128 * h + 32 * r + l] = _round_f32(d * s * q)
    return np.array(out, dtype=np.float32)


def _ref_dequant_q5k(block):
    d, dmin = _f16(block[0], block[1]), _f16(block[2], block[3])
    q = block[4:16]
    qh, ql = block[16:48], block[48:176]
    out = []
    for j in range(8):
        if j < 4:
            sc, m = int(q[j]) & 63, int(q[j + 4]) & 63
        else:
            sc = (int(q[j + 4]) & 0xF) | ((int(q[j - 4]) >> 6) << 4)
            m = (int(q[j + 4]) >> 4) | ((int(q[j]) >> 6) << 4)
        for l in range(32):
            nib = (int(ql[32 * (j // 2) + l]) >> (4 * (j & 1))) & 0xF
            hi = (int(qh[l]) >> j) & 1  # bit j of qh[l] belongs to sub-block j
            out.append(_round_f32(d * int(sc) * (nib + 16 * hi) - dmin * int(m)))
    return np.array(out, dtype=np.float32)


def _ref_dequant_q4_0(block):
    d = _f16(block[0], block[1])
    lo = [_round_f32(d * ((int(v) & 0xF) - 8)) for v in block[2:18]]
    hi = [_round_f32(d * ((int(v) >> 4) - 8)) for v in block[2:18]]
    return np.array(lo + hi, dtype=np.float32)


def _ref_dequant_q8_0(block):
    d = _f16(block[0], block[1])
    return np.array([_round_f32(d * int(v)) for v in block[2:34].view(np.int8)], dtype=np.float32)


@pytest.mark.parametrize("name,t,npr", CASES)
def test_dequant_equals_exact_rational_formula(oracle, name, t, npr):
    rng = np.random.default_rng(3)
    blocks = [_load(f"{name}_noim_expected.bin"), _load(f"{name}_im_expected.bin")]
    # plus quantized gaussian data and adversarial raw bytes (all scale/min/nibble patterns)
    x = (rng.standard_normal(8 * 256) * 0.02).astype(np.float32)
    blocks.append(oracle.quantize(x, 256, t))
    bb = oracle.BLOCK_BYTES[t]
    raw = rng.integers(0, 256, size=6 * bb, dtype=np.uint8)
    for i in range(6):  # keep the f16 scale fields finite
        for off in ([1, 3] if t in (Q4_K, Q5_K) else [209] if t == Q6_K else [1]):
            raw[i * bb + off] &= 0x3F
    blocks.append(raw)
    data = np.concatenate(blocks)
    got = oracle.dequantize(data, t)
    fn = {Q4_K: _ref_dequant_q4k, Q6_K: _ref_dequant_q6k, Q8_0: _ref_dequant_q8_0, Q5_K: _ref_dequant_q5k,
          Q4_0: _ref_dequant_q4_0}[t]
    want = np.concatenate([fn(data[i * bb:(i + 1) * bb]) for i in range(data.size // bb)])
    # exact rationals carry no sign of zero: compare zeros by value, everything else by bits
    nz = want != 0
    assert np.array_equal(got[~nz], want[~nz])
    assert np.array_equal(got[nz].view(np.uint32), want[nz].view(np.uint32))


def test_dequant_rmse_known_answers(oracle):
    # RMSE of the reference's golden blocks against their own inputs (uniform[-1,1]).
    for (name, t, _), want in zip(CASES[:3], (0.03162, 0.00790, 0.00223)):
        x = _load(f"{name}_noim_input.bin").view(np.float32)
        y = oracle.dequantize(_load(f"{name}_noim_expected.bin"), t)
        assert abs(float(np.sqrt(np.mean((x - y) ** 2))) - want) < 2e-5


def test_q8_0_roundtrip_error_bound(oracle):
    # in_memory_loader.rs:199-229: |x - dq(q(x))| <= d/2 (+ f16 rounding of d)
    rng = np.random.default_rng(5)
    x = rng.standard_normal(64 * 32).astype(np.float32)
    b = oracle.quantize(x, 32, Q8_0)
    y = oracle.dequantize(b, Q8_0)
    d = b.reshape(-1, 34)[:, :2].copy().view(np.float16).astype(np.float32).repeat(32)
    assert np.all(np.abs(x - y) <= d * 0.5 + np.abs(x) * 2e-3)


def test_dequant_rmse_of_the_added_types(oracle):
    """Round-trip error of the golden blocks against their uniform[-1, 1] inputs: Q5_K has twice the levels of
    Q4_K (half its error), Q4_0 one scale per 32 with 16 levels: step d = amax / 8, error about d / sqrt(12)."""
    rm = {}
    for name, t, _ in CASES:
        x = _load(f"{name}_noim_input.bin").view(np.float32)
        rm[t] = float(np.sqrt(np.mean((x - oracle.dequantize(_load(f"{name}_noim_expected.bin"), t)) ** 2)))
    assert 0.45 < rm[Q5_K] / rm[Q4_K] < 0.55
    assert 0.030 < rm[Q4_0] < 0.042  # amax ~ 0.97: d ~ 0.121, d / sqrt(12) ~ 0.035


@pytest.mark.parametrize("t", [Q4_K, Q6_K, Q8_0])
def test_requantize_is_idempotent(oracle, t):
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(16 * 256) * 0.02).astype(np.float32)
    b1 = oracle.quantize(x, 256, t)
    y1 = oracle.dequantize(b1, t)
    y2 = oracle.dequantize(oracle.quantize(y1, 256, t), t)
    # a second pass may move scales slightly but must stay within one quantisation step
    step = {Q4_K: 0.02 * 6 / 15, Q6_K: 0.02 * 8 / 63, Q8_0: 0.02 * 8 / 127}[t]
    assert np.abs(y1 - y2).max() <= step


def test_zero_blocks(oracle):
    # common.rs:562-618: all-zero input quantises to all-zero payloads and dequantises to 0.
    for t in (Q4_K, Q6_K, Q8_0):
        b = oracle.quantize(np.zeros(512, np.float32), 256, t)
        assert not b.any()
        assert not oracle.dequantize(b, t).any()


def test_shape_validation(oracle):
    # quantizer.rs:217-235
    with pytest.raises(ValueError):
        oracle.quantize(np.zeros(300, np.float32), 300, Q4_K)
    with pytest.raises(ValueError):
        oracle.quantize(np.zeros(512 + 256, np.float32), 512, Q4_K)
    with pytest.raises(ValueError):
        oracle.quantize(np.zeros(512, np.float32), 512, Q4_K, imatrix=np.ones(256, np.float32))


# ---- matmul oracles -------------------------------------------------------------------

def test_matmul_oracles_match_numpy(oracle):
    rng = np.random.default_rng(11)
    m, n, k = 3, 37, 512
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    got = oracle.matmul_a_by_bt(x, w, m, k, n)
    assert np.allclose(got, x.astype(np.float64) @ w.astype(np.float64).T, rtol=1e-4, atol=1e-5)
    for t in (Q4_K, Q6_K, Q8_0):
        b = oracle.quantize(w, k, t)
        wd = oracle.dequantize(b, t).reshape(n, k).astype(np.float64)
        y = oracle.qmatmul_f64(x, b, m, n, k, t)
        assert np.allclose(y, x.astype(np.float64) @ wd.T, rtol=1e-12, atol=1e-12)
        xb = oracle.f32_to_bf16_bits(x)
        yb = oracle.qmatmul_f64(xb, b, m, n, k, t)
        assert np.allclose(yb, oracle.bf16_bits_to_f32(xb).astype(np.float64) @ wd.T, rtol=1e-12, atol=1e-12)


def test_bf16_rounding_matches_torch(oracle):
    import torch

    x = np.random.default_rng(2).standard_normal(4096).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16_bits(x), want)


def test_qmatmul_id_is_per_pair_gemv(oracle):
    rng = np.random.default_rng(13)
    E, n, k, T, K = 5, 16, 256, 3, 2
    w = (rng.standard_normal((E * n, k)) * 0.02).astype(np.float32)
    stack = oracle.quantize(w, k, Q4_K)
    stride = n * 144
    ids = rng.integers(0, E, size=T * K).astype(np.uint32)
    x = rng.standard_normal((T, k)).astype(np.float32)
    y = oracle.qmatmul_id_f64(x, stack, ids, T, K, n, k, E, stride, Q4_K)
    for t in range(T):
        for s in range(K):
            e = int(ids[t * K + s])
            ref = oracle.qmatmul_f64(x[t:t + 1], stack[e * stride:(e + 1) * stride], 1, n, k, Q4_K)
            assert np.array_equal(y[t * K + s], ref[0])
    # the "down" calling convention (n_tokens = T*K, top_k = 1) over repeated rows is the same thing
    xr = np.repeat(x, K, axis=0)
    y2 = oracle.qmatmul_id_f64(xr, stack, ids, T * K, 1, n, k, E, stride, Q4_K)
    assert np.array_equal(y, y2)


def test_softmax_topk_renorm_known_answers(oracle):
    # gpu_ffn.rs:3577-3593 style case: logits [1,2,3,4] top-2 -> experts 3,2 with renormalised weights
    idx, w = oracle.softmax_topk_renorm(np.float32([1, 2, 3, 4]), 1, 4, 2)
    assert idx.tolist() == [3, 2]
    e = np.exp(np.float64([3, 4]) - 4)
    assert np.allclose(w, (e / e.sum())[::-1], rtol=1e-6)
    assert abs(float(w.sum()) - 1) < 1e-6
    # ties keep ascending expert order (stable sort), as Rust's sort_by does
    idx, w = oracle.softmax_topk_renorm(np.float32([0, 5, 5, 5, 1]), 1, 5, 2)
    assert idx.tolist() == [1, 2]
    assert np.allclose(w, [0.5, 0.5])


def test_silu_known_values(oracle):
    # gpu_ffn.rs:3558-3574
    L = oracle.lib()
    assert L.hq_oracle_silu(0.0) == 0.0
    assert abs(L.hq_oracle_silu(1.0) - 0.7310586) < 1e-6
    assert abs(L.hq_oracle_silu(-1.0) + 0.26894143) < 1e-6


def test_moe_ffn_matches_numpy_and_shared_gate_linearity(oracle):
    rng = np.random.default_rng(17)
    h, ne, topk, mm, ms, seq = 32, 4, 2, 64, 48, 3
    g = lambda *s: (rng.standard_normal(s) * 0.2).astype(np.float32)
    x, router = g(seq, h), g(ne, h)
    eg, eu, ed = g(ne * mm, h), g(ne * mm, h), g(ne * h, mm)
    sgl, sg, su, sd = g(h), g(ms, h), g(ms, h), g(h, ms)
    got = oracle.moe_ffn(x, h, ne, topk, mm, ms, router, eg, eu, ed, sgl, sg, su, sd)

    def silu(v):
        return v / (1 + np.exp(-v))

    want = np.zeros((seq, h))
    X = x.astype(np.float64)
    for t in range(seq):
        p = np.exp(router.astype(np.float64) @ X[t])
        p /= p.sum()
        top = np.argsort(-p, kind="stable")[:topk]
        wts = p[top] / p[top].sum()
        for e, wt in zip(top, wts):
            a = silu(eg[e * mm:(e + 1) * mm].astype(np.float64) @ X[t]) * (eu[e * mm:(e + 1) * mm].astype(np.float64) @ X[t])
            want[t] += wt * (ed[e * h:(e + 1) * h].astype(np.float64) @ a)
        a = silu(sg.astype(np.float64) @ X[t]) * (su.astype(np.float64) @ X[t])
        want[t] += (1 / (1 + np.exp(-(sgl.astype(np.float64) @ X[t])))) * (sd.astype(np.float64) @ a)
    assert np.allclose(got, want, rtol=2e-4, atol=2e-5)
    # gpu_ffn.rs:3493-3551: with a zero gate-logit vector the shared expert enters with weight 1/2,
    # so doubling shared_down changes the output by exactly the shared contribution at weight 1/2.
    z = np.zeros_like(sgl)
    a0 = oracle.moe_ffn(x, h, ne, topk, mm, ms, router, eg, eu, ed, z, sg, su, 0 * sd)
    a1 = oracle.moe_ffn(x, h, ne, topk, mm, ms, router, eg, eu, ed, z, sg, su, sd)
    a2 = oracle.moe_ffn(x, h, ne, topk, mm, ms, router, eg, eu, ed, z, sg, su, 2 * sd)
    assert np.allclose(a2 - a1, a1 - a0, rtol=1e-3, atol=1e-5)


# ---- rotation and 8-bit KV cache ------------------------------------------------------

def _hadamard(n):
    H = np.array([[1.0]])
    while H.shape[0] < n:
        H = np.block([[H, H], [H, -H]])
    return H / np.sqrt(n)


def _signs(oracle):
    t = oracle.TBQ_SIGNS_256
    return np.array([-1.0 if (t[j >> 3] >> (j & 7)) & 1 else 1.0 for j in range(256)])


def test_rotation_is_sign_then_sylvester_hadamard(oracle):
    rng = np.random.default_rng(19)
    x = rng.standard_normal((3, 256)).astype(np.float32)
    H, s = _hadamard(256), _signs(oracle)
    got = oracle.fwht_sign_premult(x, 3, 256)
    assert np.allclose(got, (x * s) @ H.T, atol=1e-5)
    back = oracle.fwht_sign_undo(got, 3, 256)
    assert np.allclose(back, x, atol=1e-5)          # FWHT is self-inverse, signs square to 1
    assert s[:8].tolist() == [-1, -1, -1, 1, 1, -1, 1, -1]  # 0xa7 = 1010 0111, LSB first
    # dot products are preserved: (H s q).(H s k) = q.k
    q, k = x[0], x[1]
    assert abs(float(got[0] @ got[1]) - float(q @ k)) < 1e-3
    # head_dim 512 = two independent 256-blocks
    y = rng.standard_normal((1, 512)).astype(np.float32)
    g2 = oracle.fwht_sign_premult(y, 1, 512)
    assert np.allclose(g2[0, :256], (y[0, :256] * s) @ H.T, atol=1e-5)
    assert np.allclose(g2[0, 256:], (y[0, 256:] * s) @ H.T, atol=1e-5)


def test_sign_table_is_the_reference_table_byte_for_byte(oracle):
    # kv_cache.rs:3871-3876 (TBQ_SIGNS_256); its first eight bytes are ggml's TBQ_SIGNS_64 (docs/ADR-007...:624)
    want = bytes.fromhex("a73b91f46dc2580e b37f24d68945ea1c 63afd852970be13d 76c419fe4a852cdb".replace(" ", ""))
    assert bytes(int(b) for b in oracle.TBQ_SIGNS_256) == want and len(want) == 32
    # and the rotation really uses all of them: flipping the sign of element j alone flips the table's bit j
    x = np.ones((1, 256), np.float32)
    H = _hadamard(256)
    got = oracle.fwht_sign_premult(x, 1, 256)[0]
    s = np.array([-1.0 if (want[j >> 3] >> (j & 7)) & 1 else 1.0 for j in range(256)])
    assert np.allclose(got, s @ H.T, atol=1e-5)
    assert np.allclose(oracle.fwht_sign_undo(got.reshape(1, 256).copy(), 1, 256)[0], 1.0, atol=1e-5)


def test_tq_encode_int8_is_amax_over_127_and_round_half_away(oracle):
    """The linear int8 map of the benchmark configuration, restated in numpy on the ROTATED vector: norm = amax / 127 (an
    f32 division), code = round-half-away-from-zero(x * (1 / norm)) as int8, an all-zero vector gives norm 0 and codes 0.
    A truncating cast, round-half-even, a division instead of the reciprocal multiply or amax / 128 each change bytes here."""
    rng = np.random.default_rng(41)
    d, cap = 256, 4
    for trial in range(6):
        if trial == 0:
            rot = np.zeros(d, np.float32)
        elif trial == 1:  # exact ties: amax 127 => norm 1, values k + 0.5 must round away from zero
            rot = (rng.integers(-126, 126, d) + 0.5).astype(np.float32)
            rot[0] = 127.0
        elif trial == 2:  # a scale whose reciprocal is not exact: x * (1 / d) and x / d differ in the last bit for some x
            rot = (rng.standard_normal(d) * 3.0).astype(np.float32)
            rot[5] = 7.3
        else:
            rot = (rng.standard_normal(d) * 10.0 ** rng.integers(-6, 6)).astype(np.float32)
        # the oracle encodes un-rotated input: hand it the inverse rotation of `rot` so that its rotation gives `rot` back
        # bit for bit only where the FWHT is exact; take what its own rotation yields as the vector that was quantised
        x = oracle.fwht_sign_undo(rot.reshape(1, d).copy(), 1, d).astype(np.float32)
        r = oracle.fwht_sign_premult(x.copy(), 1, d)[0].astype(np.float32)
        codes = np.zeros((1, cap, d), np.uint8)
        norms = np.zeros((1, cap, 1), np.float32)
        oracle.tq_encode_int8(x, 1, d, cap, 2, codes, norms)
        amax = np.float32(np.abs(r).max())
        norm = np.float32(amax / np.float32(127.0))
        assert norms[0, 2, 0] == norm
        inv = np.float32(1.0) / norm if norm != 0 else np.float32(0.0)
        prod = (r * inv).astype(np.float32)
        want = (np.sign(prod) * np.floor(np.abs(prod) + np.float32(0.5))).astype(np.int32)  # half away from zero
        assert np.abs(want).max() <= 127
        assert np.array_equal(codes[0, 2].view(np.int8).astype(np.int32), want), f"trial {trial}"
        assert not codes[0, [0, 1, 3]].any() and not norms[0, [0, 1, 3]].any()  # only the addressed slot is written
    # ties really occurred and went away from zero in trial 1
    rot = np.array([127.0, 0.5, -0.5, 1.5, -2.5] + [0.0] * 251, np.float32)
    x = oracle.fwht_sign_undo(rot.reshape(1, d).copy(), 1, d).astype(np.float32)
    r = oracle.fwht_sign_premult(x.copy(), 1, d)[0]
    if np.array_equal(r[:5], rot[:5]):  # (the rotation reproduces these small dyadic values exactly)
        codes = np.zeros((1, 1, d), np.uint8)
        norms = np.zeros((1, 1, 1), np.float32)
        oracle.tq_encode_int8(x, 1, d, 1, 0, codes, norms)
        assert codes[0, 0, :5].view(np.int8).tolist() == [127, 1, -1, 2, -3]


def _encode_cache(oracle, kv, n_kv, d, cap):
    codes = np.zeros((n_kv, cap, d), np.uint8)
    norms = np.zeros((n_kv, cap, max(1, d // 256)), np.float32)
    for pos in range(kv.shape[0]):
        oracle.tq_encode_int8(kv[pos], n_kv, d, cap, pos, codes, norms)
    return codes, norms


def test_tq_cache_byte_count_matches_reference_pin():
    # docs/ADR-027...:44-47: 34,078,720 bytes per slot at 32K, 2 KV heads, d=256
    n_kv, cap, d = 2, 32768, 256
    assert 2 * (n_kv * cap * d) + 2 * (n_kv * cap * 4) == 34_078_720


def test_tq_attention_single_position_closed_form(oracle):
    # kv_cache.rs:3959-4117 litmus: kv_seq_len = 1 => out[h] = V[h / heads_per_kv]
    rng = np.random.default_rng(23)
    nh, nkv, d, cap = 16, 2, 256, 8
    k = rng.standard_normal((1, nkv, d)).astype(np.float32)
    v = rng.standard_normal((1, nkv, d)).astype(np.float32)
    kc, kn = _encode_cache(oracle, k, nkv, d, cap)
    vc, vn = _encode_cache(oracle, v, nkv, d, cap)
    q = oracle.fwht_sign_premult(rng.standard_normal((nh, d)).astype(np.float32), nh, d)
    out = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, 1, cap, 1 / 16)
    out = oracle.fwht_sign_undo(out.astype(np.float32), nh, d)
    want = np.repeat(v[0], nh // nkv, axis=0)
    nrmse = np.sqrt(((out - want) ** 2).sum() / (want ** 2).sum())
    assert nrmse < 0.15          # the reference's gate
    assert nrmse < 0.02          # int8 codes do far better


def test_tq_attention_matches_numpy_softmax(oracle):
    rng = np.random.default_rng(29)
    nh, nkv, d, cap, n = 4, 2, 256, 40, 33
    k = rng.standard_normal((n, nkv, d)).astype(np.float32)
    v = rng.standard_normal((n, nkv, d)).astype(np.float32)
    kc, kn = _encode_cache(oracle, k, nkv, d, cap)
    vc, vn = _encode_cache(oracle, v, nkv, d, cap)
    q = rng.standard_normal((nh, d)).astype(np.float32)
    scale = 1 / 16
    K = kc.view(np.int8).astype(np.float64) * kn.astype(np.float64)
    V = vc.view(np.int8).astype(np.float64) * vn.astype(np.float64)

    def ref(first, last, softcap=0.0):
        out = np.zeros((nh, d))
        for h in range(nh):
            s = (K[h // 2, first:last] @ q[h].astype(np.float64)) * scale
            if softcap:
                s = softcap * np.tanh(s / softcap)
            p = np.exp(s - s.max())
            p /= p.sum()
            out[h] = p @ V[h // 2, first:last]
        return out

    got = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, n, cap, scale)
    assert np.allclose(got, ref(0, n), rtol=1e-10, atol=1e-12)
    got = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, n, cap, scale, mask_type=2, sliding_window=10)
    assert np.allclose(got, ref(n - 10, n), rtol=1e-10, atol=1e-12)
    got = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, n, cap, scale, softcap=5.0)
    assert np.allclose(got, ref(0, n, 5.0), rtol=1e-10, atol=1e-12)
    # LUT form with the identity-linear table reproduces the linear form
    lut = (np.arange(256, dtype=np.uint8).view(np.int8).astype(np.float32)) * 16.0
    got = oracle.tq_attention(q, kc, kn, vc, vn, lut, nh, nkv, d, n, cap, scale)
    assert np.allclose(got, ref(0, n), rtol=1e-6, atol=1e-8)
    # attention with rotated K/V and rotated q approximates un-quantised attention
    qr = oracle.fwht_sign_premult(q, nh, d)
    o = oracle.fwht_sign_undo(oracle.tq_attention(qr, kc, kn, vc, vn, None, nh, nkv, d, n, cap, scale).astype(np.float32), nh, d)
    exact = np.zeros((nh, d))
    for h in range(nh):
        s = (k[:, h // 2].astype(np.float64) @ q[h].astype(np.float64)) * scale
        p = np.exp(s - s.max()); p /= p.sum()
        exact[h] = p @ v[:, h // 2].astype(np.float64)
    assert np.sqrt(((o - exact) ** 2).sum() / (exact ** 2).sum()) < 0.02


def _np_attention(q, K, V, scale, group):
    """Textbook softmax attention in float64 over explicit K, V [n_kv, n, d]."""
    out = np.zeros((q.shape[0], q.shape[1]))
    for h in range(q.shape[0]):
        s = (K[h // group] @ q[h].astype(np.float64)) * scale
        p = np.exp(s - s.max())
        p /= p.sum()
        out[h] = p @ V[h // group]
    return out


def test_tq_dequantize_is_code_times_norm(oracle):
    """hq_oracle_tq_dequantize against codes.view(int8) * norms in numpy: a window that does not start at 0, and
    head_dim 512 with a norm of its own per 256-block (kv_cache.rs:2010-2012)."""
    rng = np.random.default_rng(41)
    for d in (256, 512):
        nkv, cap, start, n = 3, 50, 17, 21
        codes = rng.integers(0, 256, (nkv, cap, d), dtype=np.uint8)
        norms = rng.uniform(0.01, 2.0, (nkv, cap, d // 256)).astype(np.float32)
        got = oracle.tq_dequantize(codes, norms, None, nkv, d, cap, start, n)
        want = (codes.view(np.int8).astype(np.float64).reshape(nkv, cap, d // 256, 256)
                * norms.astype(np.float64)[..., None]).reshape(nkv, cap, d)[:, start:start + n]
        assert got.shape == (nkv, n, d)
        assert np.array_equal(got, want.astype(np.float32))  # int8 * f32 has at most 31 significant bits: one rounding
        assert not np.array_equal(got[:, 0], want[:, 1].astype(np.float32))  # the window really starts at `start`
        # table form: lut[code] * norm / 16 / scale_factor (scale_factor only at head_dim 512)
        lut = rng.standard_normal(256).astype(np.float32)
        sf = 1.7
        got = oracle.tq_dequantize(codes, norms, lut, nkv, d, cap, start, n, scale_factor_d512=sf)
        div = 16.0 * (np.float64(np.float32(sf)) if d == 512 else 1.0)
        want = (lut.astype(np.float64)[codes].reshape(nkv, cap, d // 256, 256) * norms.astype(np.float64)[..., None]
                / div).reshape(nkv, cap, d)[:, start:start + n]
        assert np.allclose(got, want, rtol=1e-6, atol=0)
    with pytest.raises(ValueError):   # kv_cache.rs:427-428: the window may not run past the capacity
        oracle.tq_dequantize(codes, norms, None, 3, 512, 50, 40, 11)


def test_tq_attention_ring_buffer_matches_rolled_cache(oracle):
    """ring_start != 0: logical position i sits in slot (ring_start + i) % capacity, the inverse of
    forward_mlx.rs:7299 (logical = (k_pos - ring_start + cap) % cap).  Checked against numpy attention over the
    cache rolled back explicitly, for a wrapped window, with and without a sliding window."""
    rng = np.random.default_rng(43)
    nh, nkv, d, cap, n, ring = 4, 2, 256, 24, 20, 9   # slots 9..23, 0..4
    kc = rng.integers(0, 256, (nkv, cap, d), dtype=np.uint8)
    vc = rng.integers(0, 256, (nkv, cap, d), dtype=np.uint8)
    kn = rng.uniform(0.001, 0.02, (nkv, cap, 1)).astype(np.float32)
    vn = rng.uniform(0.001, 0.02, (nkv, cap, 1)).astype(np.float32)
    q = rng.standard_normal((nh, d)).astype(np.float32)
    order = [(ring + i) % cap for i in range(n)]      # physical slot of logical position i
    K = (kc.view(np.int8).astype(np.float64) * kn.astype(np.float64))[:, order]
    V = (vc.view(np.int8).astype(np.float64) * vn.astype(np.float64))[:, order]
    got = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, n, cap, 0.0625, ring_start=ring)
    assert np.allclose(got, _np_attention(q, K, V, 0.0625, 2), rtol=1e-10, atol=1e-13)
    # the unrolled reading (ring_start ignored) is a different answer, so the check above can fail
    assert not np.allclose(got, oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, n, cap, 0.0625), rtol=1e-3)
    got = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, n, cap, 0.0625, mask_type=2, sliding_window=7,
                              ring_start=ring)
    assert np.allclose(got, _np_attention(q, K[:, n - 7:], V[:, n - 7:], 0.0625, 2), rtol=1e-10, atol=1e-13)
    # mask types 0 and 1 see the same positions for the single query at the end of the sequence
    a = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, n, cap, 0.0625, mask_type=1, ring_start=ring)
    b = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, n, cap, 0.0625, mask_type=0, ring_start=ring)
    assert np.array_equal(a, b)


def test_tq_attention_head_dim_512_two_norms_and_table_scale(oracle):
    """head_dim 512: every row carries two norms, one per 256-block (kv_cache.rs:2010-2012), and the table form
    divides by scale_factor_d512.  Against numpy over the explicitly dequantised cache; rows whose two norms differ
    by orders of magnitude make a swapped or shared norm visible."""
    rng = np.random.default_rng(47)
    nh, nkv, d, cap, n = 4, 2, 512, 16, 13
    kc = rng.integers(0, 256, (nkv, cap, d), dtype=np.uint8)
    vc = rng.integers(0, 256, (nkv, cap, d), dtype=np.uint8)
    kn = (rng.uniform(0.5, 1.5, (nkv, cap, 2)) * np.array([1e-3, 3e-2])).astype(np.float32)
    vn = (rng.uniform(0.5, 1.5, (nkv, cap, 2)) * np.array([4e-2, 2e-3])).astype(np.float32)
    q = rng.standard_normal((nh, d)).astype(np.float32)

    def deq(c, nrm, lut=None, sf=1.0):
        vals = c.view(np.int8).astype(np.float64) if lut is None else lut.astype(np.float64)[c] / 16.0 / sf
        return (vals.reshape(nkv, cap, 2, 256) * nrm.astype(np.float64)[..., None]).reshape(nkv, cap, d)[:, :n]

    got = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, d, n, cap, 0.046875)
    assert np.allclose(got, _np_attention(q, deq(kc, kn), deq(vc, vn), 0.046875, 2), rtol=1e-10, atol=1e-13)
    swapped = _np_attention(q, deq(kc, kn[..., ::-1]), deq(vc, vn), 0.046875, 2)
    assert not np.allclose(got, swapped, rtol=1e-3)
    lut = (rng.standard_normal(256) * 40).astype(np.float32)
    for sf in (1.0, 2.5):
        got = oracle.tq_attention(q, kc, kn, vc, vn, lut, nh, nkv, d, n, cap, 0.046875, scale_factor_d512=sf)
        want = _np_attention(q, deq(kc, kn, lut, np.float64(np.float32(sf))), deq(vc, vn, lut, np.float64(np.float32(sf))),
                             0.046875, 2)
        assert np.allclose(got, want, rtol=1e-9, atol=1e-13)
    # at head_dim 256 the scale factor is not applied
    q256 = q[:, :256].copy()
    a = oracle.tq_attention(q256, kc[..., :256].copy(), kn[..., :1].copy(), vc[..., :256].copy(), vn[..., :1].copy(), lut,
                            nh, nkv, 256, n, cap, 0.046875, scale_factor_d512=2.5)
    b = oracle.tq_attention(q256, kc[..., :256].copy(), kn[..., :1].copy(), vc[..., :256].copy(), vn[..., :1].copy(), lut,
                            nh, nkv, 256, n, cap, 0.046875, scale_factor_d512=1.0)
    assert np.array_equal(a, b)


def test_tq_attention_rejects_bad_shapes(oracle):
    z8, zf = np.zeros((1, 4, 256), np.uint8), np.zeros((1, 4, 1), np.float32)
    q = np.zeros((2, 256), np.float32)
    with pytest.raises(ValueError):   # kv_cache.rs:3816 rejects_kv_seq_len_zero
        oracle.tq_attention(q, z8, zf, z8, zf, None, 2, 1, 256, 0, 4, 1.0)
    with pytest.raises(ValueError):   # kv_cache.rs:331-333 capacity < seq_len
        oracle.tq_attention(q, z8, zf, z8, zf, None, 2, 1, 256, 5, 4, 1.0)
    with pytest.raises(ValueError):   # head_dim must be 256 or 512
        oracle.tq_attention(np.zeros((2, 128), np.float32), z8, zf, z8, zf, None, 2, 1, 128, 1, 4, 1.0)

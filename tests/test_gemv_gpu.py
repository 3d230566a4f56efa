"""GPU parity of the dequantiser and the dequant-fused GEMV / mul_mat_id kernels
against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from _util import acts, assert_matmul_close, weights
from _util import assert_matmul_close_f16_tile
from hf2q_amd import ops
from hf2q_amd.ops import (HQ_Q4_0, HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, GgmlQuantizedMatmulIdParams,
                          GgmlQuantizedMatmulParams)

pytestmark = pytest.mark.gpu
TYPES = [HQ_Q4_K, HQ_Q6_K, HQ_Q8_0]
# dequantiser and GEMV / mul_mat_id also take the next two types of the reference's production models
# (quantised on the host; the device quantizer and the tile GEMMs cover TYPES)
ALL_TYPES = TYPES + [HQ_Q5_K, HQ_Q4_0]


def _adversarial_blocks(oracle, t, nblocks, seed):
    """Raw random bytes (every nibble / 6-bit scale / sign pattern) with finite f16 scales."""
    bb = oracle.BLOCK_BYTES[t]
    raw = np.random.default_rng(seed).integers(0, 256, size=nblocks * bb, dtype=np.uint8)
    for off in ([1, 3] if t in (HQ_Q4_K, HQ_Q5_K) else [209] if t == HQ_Q6_K else [1]):
        raw[off::bb] &= 0x3F
    return raw


@pytest.mark.parametrize("t", ALL_TYPES)
def test_dequant_bit_exact(oracle, dev, t):
    be = oracle.BLOCK_ELEMS[t]
    w = weights(100 + t, 64, 1024)
    blocks = np.concatenate([oracle.quantize(w, 1024, t), _adversarial_blocks(oracle, t, 4096 // be * 8, t)])
    n = blocks.size // oracle.BLOCK_BYTES[t] * be
    want = oracle.dequantize(blocks, t)
    wd = torch.from_numpy(blocks).to(dev)
    got = ops.dequantize_ggml(wd, n, t).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    got16 = ops.dequantize_ggml(wd, n, t, torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got16, oracle.f32_to_bf16_bits(want))
    # the f16 shadow of materialize_f16_shadow (forward_mlx.rs:9426-9440): the f32 value rounded to nearest even
    goth = ops.dequantize_ggml(wd, n, t, torch.float16).view(torch.int16).cpu().numpy().view(np.uint16)
    with np.errstate(over="ignore", invalid="ignore"):
        wanth = want.astype(np.float16)
    nan = np.isnan(wanth)  # (adversarial raw blocks hold NaN scales: any NaN payload will do)
    assert np.array_equal(np.isnan(goth.view(np.float16)), nan)
    assert np.array_equal(goth[~nan], wanth.view(np.uint16)[~nan])


@pytest.mark.parametrize("t", ALL_TYPES)
def test_dequant_golden_blocks(oracle, dev, t):
    import os
    from _util import GOLDEN
    name = {HQ_Q4_K: "q4_k_512", HQ_Q6_K: "q6_k_512", HQ_Q8_0: "q8_0_64", HQ_Q5_K: "q5_k_512", HQ_Q4_0: "q4_0_64"}[t]
    blocks = np.fromfile(os.path.join(GOLDEN, "ggml_quants", f"{name}_noim_expected.bin"), dtype=np.uint8)
    n = blocks.size // oracle.BLOCK_BYTES[t] * oracle.BLOCK_ELEMS[t]
    # Q6_K / Q8_0 blocks need only 2-byte alignment: also run from an odd-word offset
    pad = torch.zeros(blocks.size + 16, dtype=torch.uint8, device=dev)
    for off in ([0] if t in (HQ_Q4_K, HQ_Q5_K) else [0, 2, 6]):
        pad[off:off + blocks.size] = torch.from_numpy(blocks).to(dev)
        got = ops.dequantize_ggml(pad[off:], n, t).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), oracle.dequantize(blocks, t).view(np.uint32))


SHAPES = [  # (m, n, k)
    (1, 512, 4096), (1, 1000, 2048), (1, 64, 256), (1, 37, 512), (1, 130, 768), (1, 96, 1024),
    (1, 257, 12288), (3, 200, 4096), (8, 128, 2048), (1, 4, 8192),
]


@pytest.mark.parametrize("t", ALL_TYPES)
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemv_matches_f64_oracle(oracle, dev, t, xdt, m, n, k):
    w = weights(7 * n + k + t, n, k)
    blocks = oracle.quantize(w, k, t, threads=8)
    x = acts(n + k, m, k)
    if xdt == "bf16":
        xb = oracle.f32_to_bf16_bits(x)
        xd = torch.from_numpy(xb.view(np.int16)).to(dev).view(torch.bfloat16).reshape(m, k)
        ref = oracle.qmatmul_f64(xb, blocks, m, n, k, t)
    else:
        xd = torch.from_numpy(x).to(dev)
        ref = oracle.qmatmul_f64(x, blocks, m, n, k, t)
    y = torch.full((m, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd, torch.from_numpy(blocks).to(dev), y, GgmlQuantizedMatmulParams(m, n, k, t))
    assert_matmul_close(y.cpu().numpy(), ref, f"gemv t={t} {xdt} {m}x{n}x{k}")


@pytest.mark.parametrize("t", ALL_TYPES)
def test_gemv_adversarial_blocks(oracle, dev, t):
    """Every scale / min / sign bit pattern, not just what the quantizer emits."""
    n, k = 96, 1024
    blocks = _adversarial_blocks(oracle, t, n * k // oracle.BLOCK_ELEMS[t], 5)
    x = acts(1, 1, k)
    for xv, xd in ((x, torch.from_numpy(x).to(dev)),
                   (oracle.f32_to_bf16_bits(x), torch.from_numpy(x).to(dev).to(torch.bfloat16))):
        ref = oracle.qmatmul_f64(xv, blocks, 1, n, k, t)
        y = torch.empty((1, n), device=dev)
        ops.quantized_matmul_ggml(xd, torch.from_numpy(blocks).to(dev), y, GgmlQuantizedMatmulParams(1, n, k, t))
        assert_matmul_close(y.cpu().numpy(), ref, f"adversarial t={t}")


@pytest.mark.parametrize("t", ALL_TYPES)
def test_gemv_zero_weights_give_zero(oracle, dev, t):
    # gpu_ffn.rs:3323-3351
    n, k = 64, 512
    blocks = oracle.quantize(np.zeros((n, k), np.float32), k, t)
    y = torch.full((1, n), 7.0, device=dev)
    ops.quantized_matmul_ggml(torch.randn(1, k, device=dev), torch.from_numpy(blocks).to(dev), y,
                              GgmlQuantizedMatmulParams(1, n, k, t))
    assert not y.cpu().numpy().any()


@pytest.mark.parametrize("t", ALL_TYPES)
def test_gemv_unaligned_weight_base(oracle, dev, t):
    if t in (HQ_Q4_K, HQ_Q5_K):
        pytest.skip("Q4_K / Q5_K require 16-byte aligned blocks (144 = 9*16, 176 = 11*16)")
    n, k = 48, 512
    blocks = oracle.quantize(weights(3, n, k), k, t)
    x = acts(4, 1, k)
    ref = oracle.qmatmul_f64(x, blocks, 1, n, k, t)
    buf = torch.zeros(blocks.size + 16, dtype=torch.uint8, device=dev)
    buf[2:2 + blocks.size] = torch.from_numpy(blocks).to(dev)
    y = torch.empty((1, n), device=dev)
    ops.quantized_matmul_ggml(torch.from_numpy(x).to(dev), buf[2:], y, GgmlQuantizedMatmulParams(1, n, k, t))
    assert_matmul_close(y.cpu().numpy(), ref, "unaligned base")


ID_CASES = [  # (E, n, k, T, K); k = 768, 2816, 1280: rows whose pieces no sixteen lanes divide (a ragged last step under bf16 rows)
    (8, 64, 512, 1, 2), (16, 512, 2048, 1, 8), (16, 2048, 512, 8, 1), (256, 128, 256, 8, 8), (4, 33, 768, 5, 3),
    (8, 48, 2816, 3, 2), (4, 40, 1280, 2, 4),
]


@pytest.mark.parametrize("t", ALL_TYPES)
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("E,n,k,T,K", ID_CASES)
def test_mul_mat_id_matches_oracle(oracle, dev, t, xdt, E, n, k, T, K):
    rng = np.random.default_rng(E * n + k)
    # quantise a few distinct experts and tile them: cheap to build, ids still select real data
    base = min(E, 4)
    blocks = oracle.quantize(weights(E + n, base * n, k), k, t, threads=8)
    stride = n * ops.ggml_row_bytes(t, k)
    stack = np.concatenate([blocks[(e % base) * stride:(e % base + 1) * stride] for e in range(E)])
    ids = rng.integers(0, E, size=T * K).astype(np.uint32)
    x = acts(k, T, k)
    xv = oracle.f32_to_bf16_bits(x) if xdt == "bf16" else x
    xd = torch.from_numpy(x).to(dev)
    xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
    ref = oracle.qmatmul_id_f64(xv, stack, ids, T, K, n, k, E, stride, t)
    y = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_ggml(xd, torch.from_numpy(stack).to(dev), torch.from_numpy(ids.view(np.int32)).to(dev), y,
                                 GgmlQuantizedMatmulIdParams(T, K, n, k, E, stride, t))
    assert_matmul_close(y.cpu().numpy(), ref, f"mul_mat_id t={t} {xdt}")


def test_mul_mat_id_invariants(oracle, dev):
    """Permuting ids permutes output rows; the down-projection calling form equals the grouped form;
    an out-of-range id poisons only its own rows."""
    t, E, n, k, T, K = HQ_Q4_K, 8, 64, 512, 4, 2
    stride = n * ops.ggml_row_bytes(t, k)
    stack = torch.from_numpy(oracle.quantize(weights(1, E * n, k), k, t)).to(dev)
    x = torch.from_numpy(acts(2, T, k)).to(dev)
    ids = torch.tensor([3, 1, 0, 7, 2, 2, 5, 4], dtype=torch.int32, device=dev)
    p = GgmlQuantizedMatmulIdParams(T, K, n, k, E, stride, t)
    y = torch.empty((T * K, n), device=dev)
    ops.quantized_matmul_id_ggml(x, stack, ids, y, p)
    swap = ids.view(T, K).flip(1).contiguous().view(-1)
    y2 = torch.empty_like(y)
    ops.quantized_matmul_id_ggml(x, stack, swap, y2, p)
    assert torch.equal(y.view(T, K, n).flip(1), y2.view(T, K, n))
    y3 = torch.empty_like(y)
    ops.quantized_matmul_id_ggml(x.repeat_interleave(K, 0).contiguous(), stack, ids, y3,
                                 GgmlQuantizedMatmulIdParams(T * K, 1, n, k, E, stride, t))
    assert torch.equal(y, y3)
    bad = ids.clone()
    bad[3] = E
    y4 = torch.empty_like(y)
    ops.quantized_matmul_id_ggml(x, stack, bad, y4, p)
    assert torch.isnan(y4[3]).all() and torch.equal(y4[[0, 1, 2, 4, 5, 6, 7]], y[[0, 1, 2, 4, 5, 6, 7]])


# ---- device-side quantizer ------------------------------------------------------------

@pytest.mark.parametrize("t", ALL_TYPES)
def test_quantizer_matches_reference_golden_bytes(oracle, dev, t):
    """The reference's own byte-equality fixtures (q4_k.rs:386-393, q6_k.rs:272-279, q8_0.rs:106-113, and the
    q5_k / q4_0 files beside them)."""
    import os
    from _util import GOLDEN
    name, npr = {HQ_Q4_K: ("q4_k_512", 512), HQ_Q6_K: ("q6_k_512", 512), HQ_Q8_0: ("q8_0_64", 64),
                 HQ_Q5_K: ("q5_k_512", 512), HQ_Q4_0: ("q4_0_64", 64)}[t]
    x = np.fromfile(os.path.join(GOLDEN, "ggml_quants", f"{name}_noim_input.bin"), dtype=np.float32)
    want = np.fromfile(os.path.join(GOLDEN, "ggml_quants", f"{name}_noim_expected.bin"), dtype=np.uint8)
    got = ops.quantize_ggml(torch.from_numpy(x).to(dev), npr, t).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_quantizer_byte_equal_to_oracle(oracle, dev, t):
    rng = np.random.default_rng(40 + t)
    parts = [
        (rng.standard_normal(300 * 256) * 0.02).astype(np.float32),          # the benchmark's weight distribution
        rng.uniform(-1, 1, 40 * 256).astype(np.float32),
        (rng.standard_normal(40 * 256) ** 3).astype(np.float32),              # heavy tails
        np.zeros(2 * 256, np.float32),                                       # zero blocks
        np.full(256, 0.37, np.float32), np.full(256, -1e-3, np.float32),     # constant blocks
        (rng.standard_normal(8 * 256) * 1e-18).astype(np.float32),           # below GROUP_MAX_EPS
        (rng.standard_normal(8 * 256) * 3e4).astype(np.float32),             # near the f16 range of d
        np.abs(rng.standard_normal(8 * 256)).astype(np.float32),             # all positive (min clamps to 0)
        np.where(rng.random(8 * 256) < 0.9, 0, rng.standard_normal(8 * 256)).astype(np.float32),  # sparse
    ]
    x = np.concatenate(parts)
    want = oracle.quantize(x, 256, t, threads=8)
    got = ops.quantize_ggml(torch.from_numpy(x).to(dev), 256, t).cpu().numpy()
    bb = oracle.BLOCK_BYTES[t]
    bad = np.nonzero((got.reshape(-1, bb) != want.reshape(-1, bb)).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} blocks differ, first {bad[:5]}"


@pytest.mark.parametrize("t", ALL_TYPES)
def test_imatrix_quantizer_matches_reference_golden_bytes(oracle, dev, t):
    """The reference's importance-matrix fixtures (q4_k.rs:395-403, q6_k.rs:281-289, q8_0.rs:115-125, q5_k.rs, q4_0.rs): the
    same inputs, the mulberry32 weights of the reference's tests (ones for Q8_0), byte equality with the `_im_` files."""
    import os
    from _util import GOLDEN
    name, npr = {HQ_Q4_K: ("q4_k_512", 512), HQ_Q6_K: ("q6_k_512", 512), HQ_Q8_0: ("q8_0_64", 64),
                 HQ_Q5_K: ("q5_k_512", 512), HQ_Q4_0: ("q4_0_64", 64)}[t]
    x = np.fromfile(os.path.join(GOLDEN, "ggml_quants", f"{name}_im_input.bin"), dtype=np.float32)
    want = np.fromfile(os.path.join(GOLDEN, "ggml_quants", f"{name}_im_expected.bin"), dtype=np.uint8)
    im = np.ones(npr, np.float32) if t == HQ_Q8_0 else oracle.mulberry32_imatrix(npr, 2)
    got = ops.quantize_ggml(torch.from_numpy(x).to(dev), npr, t, imatrix=torch.from_numpy(im).to(dev)).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("t", ALL_TYPES)
def test_imatrix_quantizer_byte_equal_to_oracle(oracle, dev, t):
    """Rows of several blocks (the weights of a column depend on its place in the row), the distributions of the plain
    quantizer's test, importance weights over four decades with some zeros; Q4_0's weights also depend on the whole row."""
    rng = np.random.default_rng(140 + t)
    npr = 1024
    parts = [
        (rng.standard_normal(96 * npr) * 0.02).astype(np.float32),
        rng.uniform(-1, 1, 12 * npr).astype(np.float32),
        (rng.standard_normal(12 * npr) ** 3).astype(np.float32),
        np.zeros(npr, np.float32), np.full(npr, 0.37, np.float32), np.full(npr, -1e-3, np.float32),
        (rng.standard_normal(2 * npr) * 1e-18).astype(np.float32),
        (rng.standard_normal(2 * npr) * 3e4).astype(np.float32),
        np.abs(rng.standard_normal(2 * npr)).astype(np.float32),
        np.where(rng.random(2 * npr) < 0.9, 0, rng.standard_normal(2 * npr)).astype(np.float32),
    ]
    x = np.concatenate(parts)
    for im in (oracle.mulberry32_imatrix(npr, 7),
               (10.0 ** rng.uniform(-2, 2, npr) * (rng.random(npr) > 0.05)).astype(np.float32)):
        want = oracle.quantize(x, npr, t, im, threads=8)
        got = ops.quantize_ggml(torch.from_numpy(x).to(dev), npr, t, imatrix=torch.from_numpy(im).to(dev)).cpu().numpy()
        bb = oracle.BLOCK_BYTES[t]
        bad = np.nonzero((got.reshape(-1, bb) != want.reshape(-1, bb)).any(axis=1))[0]
        assert bad.size == 0, f"{bad.size} blocks differ, first {bad[:5]}"
    if t != HQ_Q8_0:  # the importance matrix matters: not the bytes of the plain quantizer
        assert not np.array_equal(got, ops.quantize_ggml(torch.from_numpy(x).to(dev), npr, t).cpu().numpy())


def test_imatrix_quantizer_rejects_bad_arguments(dev):
    x = torch.zeros(1024, device=dev)
    with pytest.raises(ValueError):
        ops.quantize_ggml(x, 512, HQ_Q4_K, imatrix=torch.ones(256, device=dev))  # ImatrixLenMismatch (quantizer.rs:72-80)
    import ctypes
    from hf2q_amd import lib
    L = lib.load()
    out = torch.empty(1024 // 32 * 18, dtype=torch.uint8, device=dev)
    im = torch.ones(512, device=dev)
    assert L.hq_quantize_ggml_imatrix_scratch_bytes(1024, 512, HQ_Q4_0) == 8
    assert L.hq_quantize_ggml_imatrix_scratch_bytes(1024, 512, HQ_Q4_K) == 0
    rc = L.hq_quantize_ggml_imatrix(None, x.data_ptr(), 1024, 512, HQ_Q4_0, im.data_ptr(), out.data_ptr(), None, 0)
    assert rc == lib.HQ_ERR_INVALID_ARGUMENT  # Q4_0 needs its row scratch
    rc = L.hq_quantize_ggml_imatrix(None, x.data_ptr(), 1024, 512, HQ_Q4_K, None, out.data_ptr(), None, 0)
    assert rc == lib.HQ_ERR_INVALID_ARGUMENT  # no imatrix


def test_quantizer_rejects_bad_shapes(dev):
    # quantizer.rs:217-235
    x = torch.zeros(768, device=dev)
    with pytest.raises(ops.HqError):
        ops.quantize_ggml(x, 300, HQ_Q4_K)
    with pytest.raises(ops.HqError):
        ops.quantize_ggml(x, 512, HQ_Q4_K)


def test_mul_mat_id_many_rows(oracle, dev):
    """Prefill-sized routing (n_tokens * top_k in the hundreds) goes through the same per-row kernel."""
    t, E, n, k, T, K = HQ_Q4_K, 8, 64, 256, 96, 4
    stride = n * ops.ggml_row_bytes(t, k)
    stack = oracle.quantize(weights(11, E * n, k), k, t, threads=8)
    ids = np.random.default_rng(1).integers(0, E, size=T * K).astype(np.uint32)
    x = acts(12, T, k)
    ref = oracle.qmatmul_id_f64(x, stack, ids, T, K, n, k, E, stride, t)
    y = torch.empty(T * K, n, device=dev)
    ops.quantized_matmul_id_ggml(torch.from_numpy(x).to(dev), torch.from_numpy(stack).to(dev),
                                 torch.from_numpy(ids.view(np.int32)).to(dev), y,
                                 GgmlQuantizedMatmulIdParams(T, K, n, k, E, stride, t))
    assert_matmul_close(y.cpu().numpy(), ref, "mul_mat_id 384 rows")


# ---- grouped (expert-sorted) tile GEMM for prefill-sized mul_mat_id -------------------

GROUPED_CASES = [  # (E, n, k, T, K): at least 3 routed rows per expert and 256 rows
    (8, 128, 512, 64, 4),      # 32 rows per expert: one partly filled tile each
    (4, 160, 256, 400, 3),     # 300 rows per expert: two tiles each, n not a multiple of the tile
    (16, 64, 1024, 300, 1),    # the down-projection calling form
    (3, 256, 512, 700, 2),     # several full tiles
    (6, 200, 768, 150, 5),     # about 125 rows per expert: tiles of 128 rows, two for the experts above that
]


def _grouped_setup(oracle, dev, t, E, n, k, T, K, xdt, seed=0, skew=False):
    rng = np.random.default_rng(seed + E * n + k + T)
    base = min(E, 4)
    blocks = oracle.quantize(weights(E + n + seed, base * n, k), k, t, threads=8)
    stride = n * ops.ggml_row_bytes(t, k)
    stack = np.concatenate([blocks[(e % base) * stride:(e % base + 1) * stride] for e in range(E)])
    if skew:  # most rows to one expert, some experts unused
        ids = np.where(rng.random(T * K) < 0.7, 1, rng.integers(0, max(1, E // 2), size=T * K)).astype(np.uint32)
    else:
        ids = rng.integers(0, E, size=T * K).astype(np.uint32)
    x = acts(k + seed, T, k)
    xv = oracle.f32_to_bf16_bits(x) if xdt == "bf16" else x
    xd = torch.from_numpy(x).to(dev)
    xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
    p = GgmlQuantizedMatmulIdParams(T, K, n, k, E, stride, t)
    return stack, ids, xv, xd, p


@pytest.mark.parametrize("t", ALL_TYPES)
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("E,n,k,T,K", GROUPED_CASES)
def test_mul_mat_id_grouped_matches_oracle(oracle, dev, t, xdt, E, n, k, T, K):
    if t in (HQ_Q8_0, HQ_Q4_0) and k % 128:
        pytest.skip("Q8_0 / Q4_0 tile kernel needs k % 128 == 0")
    stack, ids, xv, xd, p = _grouped_setup(oracle, dev, t, E, n, k, T, K, xdt)
    need = ops.quantized_matmul_id_workspace_bytes(p)
    assert need > 0, "this shape must take the grouped route"
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    ref = oracle.qmatmul_id_f64(xv, stack, ids, T, K, n, k, E, p.expert_stride, t)
    y = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_ggml(xd, torch.from_numpy(stack).to(dev), torch.from_numpy(ids.view(np.int32)).to(dev), y, p,
                                 scratch=scratch)
    # the tile GEMM rounds every dequantised weight (and f32 activations) once to f16: its own gate
    assert_matmul_close_f16_tile(y.cpu().numpy(), ref, f"grouped mul_mat_id t={t} {xdt}")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q5_K, HQ_Q6_K])
def test_mul_mat_id_grouped_sparse_experts_skewed(oracle, dev, t):
    """40 routed rows per expert on average (the smallest tiles: 64 rows for Q4_K / Q5_K) with most rows on one expert,
    which then takes several of those tiles, and experts without rows."""
    E, n, k, T, K = 16, 160, 512, 160, 4
    stack, ids, xv, xd, p = _grouped_setup(oracle, dev, t, E, n, k, T, K, "bf16", seed=9, skew=True)
    assert np.bincount(ids, minlength=E).max() > 300
    need = ops.quantized_matmul_id_workspace_bytes(p)
    assert need > 0
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    ref = oracle.qmatmul_id_f64(xv, stack, ids, T, K, n, k, E, p.expert_stride, t)
    y = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_ggml(xd, torch.from_numpy(stack).to(dev), torch.from_numpy(ids.view(np.int32)).to(dev), y, p,
                                 scratch=scratch)
    assert_matmul_close_f16_tile(y.cpu().numpy(), ref, f"grouped, sparse + skewed, t={t}")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q6_K, HQ_Q8_0])
@pytest.mark.parametrize("E,n,k,T,K", [(8, 128, 512, 64, 4), (4, 160, 256, 400, 3), (16, 64, 1024, 300, 1)])
def test_mul_mat_id_grouped_with_prepared_weight_row_scales(oracle, dev, t, E, n, k, T, K):
    """The stack's weight-row scales computed once and handed to the call: the bits of the call that works them out."""
    if t == HQ_Q8_0 and k % 128:
        pytest.skip("Q8_0 tile kernel needs k % 128 == 0")
    stack, ids, xv, xd, p = _grouped_setup(oracle, dev, t, E, n, k, T, K, "bf16", seed=3)
    need = ops.quantized_matmul_id_workspace_bytes(p)
    assert need > 0
    sd = torch.from_numpy(stack).to(dev)
    idd = torch.from_numpy(ids.view(np.int32)).to(dev)
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    y0 = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_ggml(xd, sd, idd, y0, p, scratch=scratch)
    scales = ops.weight_row_scales_ggml(sd, E * n, k, t)
    scratch.fill_(0xFF)
    y1 = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_ggml(xd, sd, idd, y1, p, scratch=scratch, w_row_scales=scales)
    assert torch.equal(y0, y1)
    with pytest.raises(ValueError):
        ops.quantized_matmul_id_ggml(xd, sd, idd, y1, p, scratch=scratch, w_row_scales=scales[: E * n - 1])


def test_mul_mat_id_grouped_many_rows_and_unaligned_ids(oracle, dev):
    """More routed rows than the expert sort stages in LDS (its permutation then goes straight to memory, and the ids
    are walked in several batches), and ids that start 4 bytes past a 16-byte boundary (single loads instead of
    16-byte ones): the same products."""
    t, E, n, k, T, K = HQ_Q4_K, 8, 128, 256, 5200, 4
    stack, ids, xv, xd, p = _grouped_setup(oracle, dev, t, E, n, k, T, K, "bf16", seed=11)
    assert T * K > 16384
    need = ops.quantized_matmul_id_workspace_bytes(p)
    assert need > 0
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    sd = torch.from_numpy(stack).to(dev)
    ref = oracle.qmatmul_id_f64(xv, stack, ids, T, K, n, k, E, p.expert_stride, t)
    y = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_ggml(xd, sd, torch.from_numpy(ids.view(np.int32)).to(dev), y, p, scratch=scratch)
    assert_matmul_close_f16_tile(y.cpu().numpy(), ref, "grouped, 20800 routed rows")
    # a shorter call over ids that are not 16-byte aligned
    T2 = 300
    p2 = GgmlQuantizedMatmulIdParams(T2, K, n, k, E, p.expert_stride, t)
    holder = torch.zeros(T2 * K + 1, dtype=torch.int32, device=dev)
    holder[1:] = torch.from_numpy(ids[:T2 * K].view(np.int32)).to(dev)
    off = holder[1:]
    assert off.data_ptr() % 16 == 4
    y2 = torch.full((T2 * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_ggml(xd[:T2].contiguous(), sd, off, y2, p2, scratch=scratch)
    assert torch.equal(y2, y[:T2 * K])


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q5_K])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("E,n,k,T,K", [(8, 128, 512, 64, 4), (6, 200, 768, 150, 5), (4, 160, 256, 400, 3)])
def test_mul_mat_id_swiglu_grouped(oracle, dev, t, xdt, E, n, k, T, K):
    """Gate, up and SwiGLU of a MoE block as one grouped product: the bits of two grouped calls followed by silu_mul
    (also with the stacks' row scales computed beforehand), and silu(gate) * up of the f64 oracle's two products."""
    gate, ids, xv, xd, p = _grouped_setup(oracle, dev, t, E, n, k, T, K, xdt, seed=1)
    up, _, _, _, _ = _grouped_setup(oracle, dev, t, E, n, k, T, K, xdt, seed=2)
    assert not np.array_equal(gate, up)
    need = ops.quantized_matmul_id_swiglu_workspace_bytes(p)
    assert need >= ops.quantized_matmul_id_workspace_bytes(p) > 0
    gd, ud = torch.from_numpy(gate).to(dev), torch.from_numpy(up).to(dev)
    idd = torch.from_numpy(ids.view(np.int32)).to(dev)
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    yg, yu = torch.empty(T * K, n, device=dev), torch.empty(T * K, n, device=dev)
    ops.quantized_matmul_id_ggml(xd, gd, idd, yg, p, scratch=scratch)
    ops.quantized_matmul_id_ggml(xd, ud, idd, yu, p, scratch=scratch)
    sep = torch.empty_like(yg)
    ops.dispatch_silu_mul(yg, yu, sep)
    scratch.fill_(0xFF)
    y = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_swiglu_ggml(xd, gd, ud, idd, y, p, scratch)
    assert torch.equal(y, sep)
    scratch.fill_(0xFF)
    y2 = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_swiglu_ggml(xd, gd, ud, idd, y2, p, scratch, ops.weight_row_scales_ggml(gd, E * n, k, t),
                                        ops.weight_row_scales_ggml(ud, E * n, k, t))
    assert torch.equal(y2, sep)
    rg = oracle.qmatmul_id_f64(xv, gate, ids, T, K, n, k, E, p.expert_stride, t)
    ru = oracle.qmatmul_id_f64(xv, up, ids, T, K, n, k, E, p.expert_stride, t)
    ref = rg / (1.0 + np.exp(-rg)) * ru
    got = y.cpu().numpy().astype(np.float64)
    # silu(g) * u moves by at most |u| (1.1 dg) + |silu(g)| du for errors dg, du of the two products (|silu'| <= 1.1)
    tg = 1e-3 * np.abs(rg) + 3e-3 * np.sqrt(np.mean(rg * rg))
    tu = 1e-3 * np.abs(ru) + 3e-3 * np.sqrt(np.mean(ru * ru))
    bound = 1.1 * np.abs(ru) * tg + np.abs(rg) * tu + tg * tu + 1e-6 * np.abs(ref)
    assert (np.abs(got - ref) <= bound).all()
    assert np.sqrt(np.mean((got - ref) ** 2)) <= 1.5e-3 * np.sqrt(np.mean(ref * ref))


def test_mul_mat_id_swiglu_has_no_form_for_other_types_and_small_calls(dev):
    p = GgmlQuantizedMatmulIdParams(64, 4, 128, 512, 8, 128 * ops.ggml_row_bytes(HQ_Q6_K, 512), HQ_Q6_K)
    assert ops.quantized_matmul_id_workspace_bytes(p) > 0 and ops.quantized_matmul_id_swiglu_workspace_bytes(p) == 0
    small = GgmlQuantizedMatmulIdParams(8, 2, 128, 512, 8, 128 * ops.ggml_row_bytes(HQ_Q4_K, 512), HQ_Q4_K)
    assert ops.quantized_matmul_id_swiglu_workspace_bytes(small) == 0
    x = torch.zeros(8, 512, device=dev)
    w = torch.zeros(8 * small.expert_stride, dtype=torch.uint8, device=dev)
    with pytest.raises(ops.HqError) as e:
        ops.quantized_matmul_id_swiglu_ggml(x, w, w, torch.zeros(16, dtype=torch.int32, device=dev), torch.empty(16, 128, device=dev),
                                            small, torch.empty(256, dtype=torch.uint8, device=dev))
    assert e.value.status == 2 and "hq_silu_mul" in str(e.value)


def test_mul_mat_id_grouped_routing_properties(oracle, dev):
    """Skewed routing with unused experts, an id that is no expert (NaN rows, the others untouched), agreement with
    the per-row GEMV form, a scratch that is too small, and a strided stack (which keeps the GEMV form)."""
    t, E, n, k, T, K = HQ_Q4_K, 8, 128, 512, 200, 2
    stack, ids, xv, xd, p = _grouped_setup(oracle, dev, t, E, n, k, T, K, "bf16", seed=5, skew=True)
    need = ops.quantized_matmul_id_workspace_bytes(p)
    assert need > 0
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    sd = torch.from_numpy(stack).to(dev)
    idd = torch.from_numpy(ids.view(np.int32)).to(dev)
    ref = oracle.qmatmul_id_f64(xv, stack, ids, T, K, n, k, E, p.expert_stride, t)
    y = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_ggml(xd, sd, idd, y, p, scratch=scratch)
    assert_matmul_close_f16_tile(y.cpu().numpy(), ref, "grouped, skewed routing")
    y_gemv = torch.empty_like(y)
    ops.quantized_matmul_id_ggml(xd, sd, idd, y_gemv, p)  # no scratch: one GEMV per row
    assert_matmul_close(y_gemv.cpu().numpy(), ref, "gemv form")
    assert np.abs(y.cpu().numpy() - y_gemv.cpu().numpy()).max() <= 1e-3 * np.abs(ref).max()
    bad = idd.clone()
    bad[[7, 150]] = E + 3
    y_bad = torch.zeros_like(y)
    ops.quantized_matmul_id_ggml(xd, sd, bad, y_bad, p, scratch=scratch)
    keep = np.setdiff1d(np.arange(T * K), [7, 150])
    assert torch.isnan(y_bad[[7, 150]]).all() and torch.equal(y_bad[keep], y[keep])
    with pytest.raises(ops.HqError) as e:
        ops.quantized_matmul_id_ggml(xd, sd, idd, y, p, scratch=scratch[:need - 256])
    assert e.value.status == 1
    padded = GgmlQuantizedMatmulIdParams(T, K, n, k, E, p.expert_stride + 16, t)
    assert ops.quantized_matmul_id_workspace_bytes(padded) == 0
    small = GgmlQuantizedMatmulIdParams(8, 2, n, k, E, p.expert_stride, t)
    assert ops.quantized_matmul_id_workspace_bytes(small) == 0


# ---- 4..8 activation rows sharing one pass over the weights (small-batch decode) ------

ROWS_SHAPES = [(3, 80, 2048), (4, 64, 1024), (4, 200, 4096), (4, 16, 2048), (5, 33, 1024), (6, 130, 3072), (7, 250, 2048), (8, 96, 12288)]


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q6_K, HQ_Q5_K])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k", ROWS_SHAPES)
def test_small_batch_rows_match_f64_oracle(oracle, dev, t, xdt, m, n, k):
    """Q4_K / Q5_K (3 <= m <= 8) and Q6_K (4 <= m <= 8) with k % 1024 == 0 take the kernel that fetches every weight once for all rows."""
    blocks = oracle.quantize(weights(3 * n + k + m, n, k), k, t, threads=8)
    x = acts(n + k + m, m, k)
    xv = oracle.f32_to_bf16_bits(x) if xdt == "bf16" else x
    xd = torch.from_numpy(x).to(dev)
    xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
    ref = oracle.qmatmul_f64(xv, blocks, m, n, k, t)
    y = torch.full((m, n), float("nan"), device=dev)
    wd = torch.from_numpy(blocks).to(dev)
    ops.quantized_matmul_ggml(xd, wd, y, GgmlQuantizedMatmulParams(m, n, k, t))
    assert_matmul_close(y.cpu().numpy(), ref, f"rows t={t} {xdt} {m}x{n}x{k}")
    # every row equals the one-row product of the same activations (the GEMV kernel) to accumulation noise
    y1 = torch.empty((1, n), device=dev)
    for r in range(m):
        ops.quantized_matmul_ggml(xd[r:r + 1].contiguous(), wd, y1, GgmlQuantizedMatmulParams(1, n, k, t))
        assert np.abs(y1.cpu().numpy()[0] - y.cpu().numpy()[r]).max() <= 1e-4 * np.abs(ref).max()


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q6_K])
@pytest.mark.parametrize("m,k", [(3, 24576), (4, 24576), (4, 20480), (7, 24576)])
def test_small_batch_rows_of_very_wide_matrices(oracle, dev, t, m, k):
    """bf16 rows over k = 20480 / 24576: three or four staged activation rows would not fit a workgroup's LDS (4 x 24576 x
    2.25 bytes = 221 KB), so the rows go in passes of as many as do fit; each row equals its one-row product."""
    n = 2048  # enough rows for the streaming form at 256 CUs x 16 waves
    blocks = oracle.quantize(weights(k + m + t, n, k), k, t, threads=8)
    x = acts(k + m, m, k)
    ref = oracle.qmatmul_f64(oracle.f32_to_bf16_bits(x), blocks, m, n, k, t)
    xd = torch.from_numpy(x).to(dev).to(torch.bfloat16)
    wd = torch.from_numpy(blocks).to(dev)
    y = torch.full((m, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd, wd, y, GgmlQuantizedMatmulParams(m, n, k, t))
    assert_matmul_close(y.cpu().numpy(), ref, f"wide rows t={t} {m}x{n}x{k}")
    y1 = torch.empty((1, n), device=dev)
    for r in range(m):
        ops.quantized_matmul_ggml(xd[r:r + 1].contiguous(), wd, y1, GgmlQuantizedMatmulParams(1, n, k, t))
        assert np.abs(y1.cpu().numpy()[0] - y.cpu().numpy()[r]).max() <= 1e-4 * np.abs(ref).max()


ROWS32_SHAPES = [  # (m, n, k): Q8_0 / Q4_0; k is walked in chunks of 2048 (64 blocks, one per lane)
    (2, 80, 2048), (3, 64, 1024), (4, 200, 4096), (4, 5, 32), (5, 33, 320), (6, 130, 3104), (7, 250, 2048), (8, 96, 12288),
    (8, 4100, 256),   # more rows than one pass of 16 waves x 256 workgroups covers on a small device share
]


@pytest.mark.parametrize("t", [HQ_Q8_0, HQ_Q4_0])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k", ROWS32_SHAPES)
def test_small_batch_rows_of_32_weight_blocks_match_f64_oracle(oracle, dev, t, xdt, m, n, k):
    """Q8_0 / Q4_0 with 2 <= m <= 8 take the kernel that fetches every weight once for all rows: exact products, so the
    GEMV's tolerance; a short last chunk (k % 2048 != 0), fewer rows than waves, ragged n; the same bits on every call
    (later chunks are added to y by the row's one writer, in chunk order)."""
    blocks = oracle.quantize(weights(3 * n + k + m + t, n, k), k, t, threads=8)
    x = acts(n + k + m, m, k)
    xv = oracle.f32_to_bf16_bits(x) if xdt == "bf16" else x
    xd = torch.from_numpy(x).to(dev)
    xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
    ref = oracle.qmatmul_f64(xv, blocks, m, n, k, t)
    y = torch.full((m, n), float("nan"), device=dev)
    wd = torch.from_numpy(blocks).to(dev)
    ops.quantized_matmul_ggml(xd, wd, y, GgmlQuantizedMatmulParams(m, n, k, t))
    assert_matmul_close(y.cpu().numpy(), ref, f"rows32 t={t} {xdt} {m}x{n}x{k}")
    y2 = torch.full((m, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd, wd, y2, GgmlQuantizedMatmulParams(m, n, k, t))
    assert torch.equal(y, y2)
    y1 = torch.empty((1, n), device=dev)
    for r in range(m):
        ops.quantized_matmul_ggml(xd[r:r + 1].contiguous(), wd, y1, GgmlQuantizedMatmulParams(1, n, k, t))
        assert np.abs(y1.cpu().numpy()[0] - y.cpu().numpy()[r]).max() <= 1e-4 * max(np.abs(ref).max(), 1e-30)


@pytest.mark.parametrize("t", [HQ_Q8_0, HQ_Q4_0])
def test_small_batch_rows_of_32_weight_blocks_adversarial_and_scaling(oracle, dev, t):
    """Every byte pattern of the blocks (finite scales); scaling the activations by a power of two scales the result
    exactly; rows past m of the staged activations do not leak into the output (m = 3 runs the 4-row instantiation)."""
    m, n, k = 3, 48, 2048 + 64
    bb = oracle.BLOCK_BYTES[t]
    raw = np.random.default_rng(11).integers(0, 256, size=n * k // 32 * bb, dtype=np.uint8)
    raw[1::bb] &= 0x3F  # f16 scale: finite, modest magnitude
    x = acts(4, m, k)
    wd = torch.from_numpy(raw).to(dev)
    for xv, xd in ((x, torch.from_numpy(x).to(dev)),
                   (oracle.f32_to_bf16_bits(x), torch.from_numpy(x).to(dev).to(torch.bfloat16))):
        ref = oracle.qmatmul_f64(xv, raw, m, n, k, t)
        y = torch.full((m + 1, n), 7.0, device=dev)
        ops.quantized_matmul_ggml(xd, wd, y[:m], GgmlQuantizedMatmulParams(m, n, k, t))
        assert_matmul_close(y[:m].cpu().numpy(), ref, "rows32, adversarial blocks")
        assert (y[m] == 7.0).all()
        y4 = torch.empty((m, n), device=dev)
        ops.quantized_matmul_ggml(xd * 4.0, wd, y4, GgmlQuantizedMatmulParams(m, n, k, t))
        assert torch.equal(y4, y[:m] * 4.0)


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q6_K, HQ_Q5_K])
@pytest.mark.parametrize("xdt,m", [("bf16", 8), ("f32", 5)])
def test_small_batch_rows_tall_matrix(oracle, dev, t, xdt, m):
    """From 49152 weight rows on a workgroup takes 64 rows instead of 16; the last workgroup here is ragged (n % 64 = 40,
    so one of its waves has 8 rows and one none).  Weights: a quantized 1024-row tile repeated, rotated per repeat."""
    n, k, tile = 49152 + 40, 2048, 1024
    tile_blocks = oracle.quantize(weights(77, tile, k), k, t, threads=8).reshape(tile, -1)
    reps = -(-n // tile)
    blocks = np.concatenate([np.roll(tile_blocks, 37 * i, axis=0) for i in range(reps)])[:n].copy().reshape(-1)
    x = acts(78, m, k)
    xv = oracle.f32_to_bf16_bits(x) if xdt == "bf16" else x
    xd = torch.from_numpy(x).to(dev)
    xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
    ref = oracle.qmatmul_f64(xv, blocks, m, n, k, t)
    y = torch.full((m, n + 64), float("nan"), device=dev)[:, :n].contiguous()
    ops.quantized_matmul_ggml(xd, torch.from_numpy(blocks).to(dev), y, GgmlQuantizedMatmulParams(m, n, k, t))
    assert_matmul_close(y.cpu().numpy(), ref, f"rows, tall matrix t={t} {xdt} m={m}")


@pytest.mark.parametrize("t,m,k", [(HQ_Q4_K, 9, 2048), (HQ_Q4_K, 16, 1024), (HQ_Q5_K, 16, 1024), (HQ_Q6_K, 12, 768),
                                   (HQ_Q6_K, 16, 1280), (HQ_Q5_K, 13, 256), (HQ_Q4_K, 15, 768)])
def test_a_few_rows_past_eight_run_in_chunks_of_eight(oracle, dev, t, m, k):
    """Up to 16 rows of Q4_K / Q5_K (whose tiles of 64 token rows take over beyond that), and up to 16 rows of a K-quant
    whose k has no small-batch kernel (k % 1024 != 0), do not take a tile kernel: chunks of eight through the
    small-batch kernel, the remainder through it or the GEMV.  Every product is exact on this route, so the GEMV's
    tolerance holds, and no scratch is asked for."""
    n = 136
    blocks = oracle.quantize(weights(m + k + t, n, k), k, t, threads=8)
    x = acts(m + t, m, k)
    ref = oracle.qmatmul_f64(oracle.f32_to_bf16_bits(x), blocks, m, n, k, t)
    y = torch.full((m, n), float("nan"), device=dev)
    p = GgmlQuantizedMatmulParams(m, n, k, t)
    assert ops.quantized_matmul_workspace_bytes(p, torch.bfloat16) == 0
    ops.quantized_matmul_ggml(torch.from_numpy(x).to(dev).to(torch.bfloat16), torch.from_numpy(blocks).to(dev), y, p)
    assert_matmul_close(y.cpu().numpy(), ref, f"chunked rows t={t} m={m} k={k}")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q6_K, HQ_Q5_K])
def test_small_batch_rows_adversarial_blocks_and_scaling(oracle, dev, t):
    """Every scale / min / nibble pattern; and scaling the activations by a power of two scales the result exactly."""
    m, n, k = 8, 48, 2048
    blocks = _adversarial_blocks(oracle, t, n * k // 256, 9)
    x = acts(2, m, k)
    wd = torch.from_numpy(blocks).to(dev)
    for xv, xd in ((x, torch.from_numpy(x).to(dev)),
                   (oracle.f32_to_bf16_bits(x), torch.from_numpy(x).to(dev).to(torch.bfloat16))):
        ref = oracle.qmatmul_f64(xv, blocks, m, n, k, t)
        y = torch.empty((m, n), device=dev)
        ops.quantized_matmul_ggml(xd, wd, y, GgmlQuantizedMatmulParams(m, n, k, t))
        assert_matmul_close(y.cpu().numpy(), ref, "rows, adversarial blocks")
        y2 = torch.empty_like(y)
        ops.quantized_matmul_ggml(xd * 1024, wd, y2, GgmlQuantizedMatmulParams(m, n, k, t))
        assert torch.equal(y2, y * 1024)


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q6_K])
def test_decode_gemvs_replay_from_a_hip_graph(oracle, dev, t):
    """The streaming GEMV form (one workgroup per CU, results kept in lanes and stored 64 rows at a time) as a decode
    loop runs it: a single matrix and the two-matrix launch recorded into a HIP graph, three replays with the
    activations rewritten, every replay equal to the eager calls and within the GEMV bound of the f64 product."""
    n, k = 8192, 4096  # enough rows for two per wave of the device: the streaming route
    w0 = oracle.quantize(weights(201, n, k), k, t, threads=8)
    w1 = oracle.quantize(weights(202, n, k), k, t, threads=8)
    dq0 = oracle.dequantize(w0, t, threads=8).reshape(n, k).astype(np.float64)
    wd0, wd1 = torch.from_numpy(w0).to(dev), torch.from_numpy(w1).to(dev)
    x = torch.zeros(1, k, device=dev, dtype=torch.bfloat16)
    y, ya, yb = (torch.empty(1, n, device=dev) for _ in range(3))
    p = GgmlQuantizedMatmulParams(1, n, k, t)

    def step(o, oa, ob):
        ops.quantized_matmul_ggml(x, wd0, o, p)
        ops.quantized_matmul_batch_ggml([ops.QmatmulJob(x, wd0, oa, 1, n, k), ops.QmatmulJob(x, wd1, ob, 1, n, k)], t)

    step(y, ya, yb)  # warm-up outside the capture (kernel attributes are set here)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            step(y, ya, yb)
    torch.cuda.synchronize()
    for rep in range(3):
        xa = acts(210 + rep, 1, k)
        x.copy_(torch.from_numpy(xa).to(dev).to(torch.bfloat16))
        for o in (y, ya, yb):
            o.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in (y, ya, yb)]
        want = [torch.empty(1, n, device=dev) for _ in range(3)]
        step(*want)
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), f"replay {rep}"
        assert torch.equal(got[0], got[1])  # the same matrix through the one-matrix and the two-matrix launch
        xb = x.float().cpu().numpy().astype(np.float64)
        assert_matmul_close(got[0].cpu().numpy(), xb @ dq0.T, f"replay {rep}")


def test_stream_read_probe_reads_and_writes_nothing(dev):
    """hq_stream_read_probe only reads: any size that is whole 16-byte pieces (ragged against the 8 KiB runs), the buffer and
    the sink unchanged; odd sizes and alignments are rejected."""
    buf = torch.arange(0, (3 << 20) + 4, dtype=torch.int32, device=dev)  # 12 MiB + 16 bytes
    keep = buf.clone()
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    ops.stream_read_probe(buf, sink)
    ops.stream_read_probe(buf[:4], sink)
    torch.cuda.synchronize()
    assert torch.equal(buf, keep) and sink.item() == 0
    with pytest.raises(ops.HqError):
        ops.stream_read_probe(buf[:3], sink)   # 12 bytes
    with pytest.raises(ops.HqError):
        ops.stream_read_probe(buf[1:5], sink)  # not 16-byte aligned

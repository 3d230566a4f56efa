"""GPU parity of the batched-prefill MFMA GEMM (m > 8) against the f64 oracle."""
import numpy as np
import pytest
import torch

from _util import acts, assert_matmul_close, weights
from hf2q_amd import ops
from hf2q_amd.ops import HQ_Q4_K, HQ_Q6_K, HQ_Q8_0, GgmlQuantizedMatmulParams

pytestmark = pytest.mark.gpu

SHAPES = [  # (m, n, k): tile edges in every dimension (tile is 256 x 128 x 64)
    (9, 128, 256), (33, 200, 512), (256, 128, 1024), (300, 257, 768), (64, 96, 4096), (513, 384, 256),
]


def _run(oracle, dev, t, xdt, m, n, k, blocks=None, seed=0):
    if blocks is None:
        blocks = oracle.quantize(weights(31 * n + k + t + seed, n, k), k, t, threads=8)
    x = acts(n + k + m + seed, m, k)
    if xdt == "bf16":
        xv = oracle.f32_to_bf16_bits(x)
        xd = torch.from_numpy(xv.view(np.int16)).to(dev).view(torch.bfloat16).reshape(m, k)
    else:
        xv = x
        xd = torch.from_numpy(x).to(dev)
    ref = oracle.qmatmul_f64(xv, blocks, m, n, k, t)
    y = torch.full((m, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd, torch.from_numpy(blocks).to(dev), y, GgmlQuantizedMatmulParams(m, n, k, t))
    return y.cpu().numpy(), ref


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0, HQ_Q6_K])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_matches_f64_oracle(oracle, dev, t, xdt, m, n, k):
    y, ref = _run(oracle, dev, t, xdt, m, n, k)
    assert_matmul_close(y, ref, f"gemm t={t} {xdt} {m}x{n}x{k}")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0])
def test_gemm_adversarial_blocks(oracle, dev, t):
    """Every scale / min / nibble bit pattern (raw random bytes with finite f16 fields)."""
    m, n, k = 40, 128, 512
    bb = oracle.BLOCK_BYTES[t]
    raw = np.random.default_rng(9).integers(0, 256, size=n * k // oracle.BLOCK_ELEMS[t] * bb, dtype=np.uint8)
    for off in ([1, 3] if t == HQ_Q4_K else [1]):
        raw[off::bb] &= 0x3F
    for xdt in ("bf16", "f32"):
        y, ref = _run(oracle, dev, t, xdt, m, n, k, blocks=raw)
        assert_matmul_close(y, ref, f"gemm adversarial t={t} {xdt}")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0])
def test_gemm_rows_equal_gemv_rows(oracle, dev, t):
    """Row i of the m>8 result agrees with the m=1 GEMV of activation row i (both within 1e-3 of f64,
    and with each other far tighter)."""
    m, n, k = 24, 256, 1024
    blocks = oracle.quantize(weights(5, n, k), k, t, threads=8)
    wd = torch.from_numpy(blocks).to(dev)
    x = torch.from_numpy(acts(6, m, k)).to(dev).to(torch.bfloat16)
    y = torch.empty(m, n, device=dev)
    ops.quantized_matmul_ggml(x, wd, y, GgmlQuantizedMatmulParams(m, n, k, t))
    y1 = torch.empty(1, n, device=dev)
    for i in (0, 7, 23):
        ops.quantized_matmul_ggml(x[i:i + 1].contiguous(), wd, y1, GgmlQuantizedMatmulParams(1, n, k, t))
        scale = y1.abs().max().item()
        assert (y[i] - y1[0]).abs().max().item() <= 2e-5 * scale


def test_gemm_zero_weights_give_zero(oracle, dev):
    m, n, k = 32, 128, 512
    blocks = oracle.quantize(np.zeros((n, k), np.float32), k, HQ_Q4_K)
    y = torch.full((m, n), 3.0, device=dev)
    ops.quantized_matmul_ggml(torch.randn(m, k, device=dev).to(torch.bfloat16), torch.from_numpy(blocks).to(dev), y,
                              GgmlQuantizedMatmulParams(m, n, k, HQ_Q4_K))
    assert not y.cpu().numpy().any()

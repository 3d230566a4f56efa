"""The benchmark configurations at their full sizes.

The other GPU tests compare whole outputs with the oracle at sizes it finishes in seconds.  Here every
configuration runs at the shape its throughput is quoted on, and is checked (a) against the oracle on a sample
of output rows that the oracle can afford (its inputs are slices of the same device-quantized weights, and the
device quantizer is byte-equal to the oracle's by test_gemv_gpu.py), and (b) through properties that hold at
any size: linearity in the activations, exact scaling by powers of two, a known closed form."""
import numpy as np
import pytest
import torch

from _util import acts, assert_matmul_close, assert_matmul_close_f16_tile
from hf2q_amd import ops
from hf2q_amd.ops import (HQ_Q4_0, HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, FlashAttnVecTqHbParams,
                          GgmlQuantizedMatmulParams)

pytestmark = pytest.mark.gpu


def _quantized(dev, n, k, t, seed):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    return ops.quantize_ggml(torch.randn(n * k, generator=g, device=dev).mul_(0.02), k, t)


def _rows_of(blocks, rows, k, t, oracle):
    """The packed rows `rows` of a device weight matrix, as one small host matrix."""
    rb = k // oracle.BLOCK_ELEMS[t] * oracle.BLOCK_BYTES[t]
    m = blocks.view(-1, rb)
    return m[torch.as_tensor(rows, device=blocks.device)].contiguous().view(-1).cpu().numpy()


# decode GEMV: gate / up 12288 x 4096 and down 4096 x 12288 in Q4_K, the output head 151936 x 4096 in Q6_K
DECODE_SHAPES = [(12288, 4096, HQ_Q4_K), (4096, 12288, HQ_Q4_K), (151936, 4096, HQ_Q6_K)]


@pytest.mark.parametrize("n,k,t", DECODE_SHAPES)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 7, 8])
def test_decode_gemv_full_size(oracle, dev, n, k, t, m):
    """m = 1: the GEMV kernels of the decode step; m = 2 .. 4: their multi-row forms (one pass over the weights);
    m = 7: a four-row and a three-row pass (Q6_K) or the small-batch kernel (Q4_K); m = 8: the small-batch kernels."""
    w = _quantized(dev, n, k, t, 7 + n)
    rng = np.random.default_rng(n + m)
    # multiples of 1/8 below 4 in magnitude: exact in bf16, and so are the sums of two of them
    xa = (rng.integers(-12, 13, (m, k)) / 8.0).astype(np.float32)
    xb = (rng.integers(-12, 13, (m, k)) / 8.0).astype(np.float32)
    p = GgmlQuantizedMatmulParams(m, n, k, t)

    def run(x):
        y = torch.full((m, n), float("nan"), device=dev)
        ops.quantized_matmul_ggml(torch.from_numpy(x).to(dev).to(torch.bfloat16), w, y, p)
        return y

    ya, yb, yab = run(xa), run(xb), run(xa + xb)
    assert torch.isfinite(yab).all()
    # (a) sampled rows against the f64 oracle
    rows = np.unique(np.concatenate([[0, 1, n - 2, n - 1], rng.integers(0, n, 60)]))
    ref = oracle.qmatmul_f64(oracle.f32_to_bf16_bits(xa), _rows_of(w, rows, k, t, oracle), m, rows.size, k, t)
    assert_matmul_close(ya[:, torch.as_tensor(rows, device=dev)].cpu().numpy(), ref, f"gemv {n}x{k} m={m}, sampled rows")
    # (b) linearity over every output, to f32 accumulation noise of the output's scale
    scale = yab.abs().max().item()
    assert (yab - (ya + yb)).abs().max().item() <= 2e-5 * scale
    # (c) exact scaling by a power of two
    assert torch.equal(run(xa * 4.0), ya * 4.0)


@pytest.mark.parametrize("n", [8192, 65539, 70001, 70002])
def test_q6k_head_rows_copied_through_lds(oracle, dev, n):
    """Q6_K matrices of 4096 columns with 8192 rows or more and one bf16 activation row: a wave copies groups of four
    whole rows through LDS.  Row counts that leave the last group with 4, 3, 1 and 2 rows; every output row against the
    two-row pass over the same activations twice (the kernel whose lanes fetch their own pieces, which gives the same
    bits), sampled rows against the f64 oracle."""
    k, t = 4096, HQ_Q6_K
    w = _quantized(dev, n, k, t, 3 + n)
    rng = np.random.default_rng(n)
    x = (rng.integers(-12, 13, (1, k)) / 8.0).astype(np.float32)
    xd = torch.from_numpy(x).to(dev).to(torch.bfloat16)
    y = torch.full((1, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd, w, y, GgmlQuantizedMatmulParams(1, n, k, t))
    assert torch.isfinite(y).all()
    y2 = torch.full((2, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(torch.cat([xd, xd]), w, y2, GgmlQuantizedMatmulParams(2, n, k, t))
    assert torch.equal(y2[0:1], y) and torch.equal(y2[1:2], y)
    rows = np.unique(np.concatenate([[0, 1, 2, 3, n - 4, n - 3, n - 2, n - 1], rng.integers(0, n, 40)]))
    ref = oracle.qmatmul_f64(oracle.f32_to_bf16_bits(x), _rows_of(w, rows, k, t, oracle), 1, rows.size, k, t)
    assert_matmul_close(y[:, torch.as_tensor(rows, device=dev)].cpu().numpy(), ref, f"q6_k {n}x{k}, sampled rows")


@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("t,n,k", [(HQ_Q6_K, 8192, 4096), (HQ_Q6_K, 65539, 4096), (HQ_Q6_K, 16384, 2048), (HQ_Q6_K, 40001, 2048),
                                   (HQ_Q6_K, 40006, 2048), (HQ_Q4_K, 8192, 4096), (HQ_Q4_K, 12289, 4096), (HQ_Q5_K, 8192, 4096),
                                   (HQ_Q5_K, 20001, 4096)])
def test_weights_copied_through_lds_f32_and_short_rows(oracle, dev, xdt, t, n, k):
    """The forms of the one-row GEMV that copy the weights through LDS, beyond the bf16 head: f32 activations (the dtype of
    the reference's call sites, gpu_full_attn.rs:835) over Q6_K chunks and over Q4_K / Q5_K rows of 4096, and Q6_K rows
    of 2048 elements (two rows per chunk of sixteen blocks; row counts that leave the last chunk with one row and the
    last group with 1 .. 4 chunks).  Every output row against the product over a slice of the matrix small enough for
    the kernels whose lanes fetch their own pieces, sampled rows against the f64 oracle, and the same bits on a second
    call."""
    w = _quantized(dev, n, k, t, 5 + n)
    rng = np.random.default_rng(n + k)
    x = (rng.integers(-12, 13, (1, k)) / 8.0).astype(np.float32)
    xd = torch.from_numpy(x).to(dev)
    xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
    y = torch.full((1, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd, w, y, GgmlQuantizedMatmulParams(1, n, k, t))
    assert torch.isfinite(y).all()
    rows = np.unique(np.concatenate([[0, 1, 2, 3, n - 4, n - 3, n - 2, n - 1], rng.integers(0, n, 40)]))
    xv = oracle.f32_to_bf16_bits(x) if xdt == "bf16" else x
    ref = oracle.qmatmul_f64(xv, _rows_of(w, rows, k, t, oracle), 1, rows.size, k, t)
    assert_matmul_close(y[:, torch.as_tensor(rows, device=dev)].cpu().numpy(), ref, f"type {t} {xdt} {n}x{k}, sampled rows")
    row_bytes = k // oracle.BLOCK_ELEMS[t] * oracle.BLOCK_BYTES[t]
    part = 2048  # rows per slice: below what the chunk-copy form takes
    for r0 in (0, (n - part) // 2, n - part):
        ys = torch.full((1, part), float("nan"), device=dev)
        ops.quantized_matmul_ggml(xd, w[r0 * row_bytes:(r0 + part) * row_bytes].clone(), ys, GgmlQuantizedMatmulParams(1, part, k, t))
        assert (ys - y[:, r0:r0 + part]).abs().max().item() <= 2e-6 * np.abs(ref).max(), (xdt, n, k, r0)
    y2 = torch.full((1, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd, w, y2, GgmlQuantizedMatmulParams(1, n, k, t))
    assert torch.equal(y, y2)


@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("t,n,k", [(HQ_Q6_K, 8192, 4096), (HQ_Q6_K, 4096, 5120), (HQ_Q6_K, 2048, 8192), (HQ_Q8_0, 8192, 4096),
                                   (HQ_Q8_0, 12288, 2816), (HQ_Q4_0, 8192, 4096)])
def test_copy_forms_and_their_fallbacks_give_the_same_bits(dev, xdt, t, n, k):
    """The forms that copy weights through LDS need every copy to start on a 16-byte boundary; a matrix whose base is
    not a multiple of 16 takes the kernels whose lanes fetch their own pieces.  Both compute the same pieces, products and
    sums: the outputs are equal bit for bit (Q6_K chunk copy, the flat walk's copied windows for Q6_K, Q8_0 and Q4_0)."""
    w = _quantized(dev, n, k, t, 21 + n + k)
    g = torch.Generator(device=dev)
    g.manual_seed(n + k)
    x = torch.randn(1, k, generator=g, device=dev)
    x = x.to(torch.bfloat16) if xdt == "bf16" else x
    p = GgmlQuantizedMatmulParams(1, n, k, t)
    y = torch.full((1, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(x, w, y, p)
    assert torch.isfinite(y).all()
    for off in (2, 8):
        holder = torch.zeros(w.numel() + 32, dtype=torch.uint8, device=dev)
        shifted = holder[off:off + w.numel()]
        shifted.copy_(w)
        assert shifted.data_ptr() % 16 == off
        y2 = torch.full((1, n), float("nan"), device=dev)
        ops.quantized_matmul_ggml(x, shifted, y2, p)
        assert torch.equal(y, y2), (t, n, k, xdt, off)


@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("t,n,k", [(HQ_Q6_K, 262144, 2816), (HQ_Q6_K, 151936, 2560), (HQ_Q6_K, 151936, 3072), (HQ_Q6_K, 152064, 3584),
                                   (HQ_Q6_K, 131072, 3840), (HQ_Q6_K, 152064, 5120), (HQ_Q6_K, 65536, 7168), (HQ_Q6_K, 32768, 14336),
                                   (HQ_Q4_K, 262144, 2816), (HQ_Q4_K, 152064, 5120), (HQ_Q4_K, 151936, 3072), (HQ_Q5_K, 262144, 2816),
                                   (HQ_Q5_K, 152064, 3584), (HQ_Q5_K, 65536, 7168), (HQ_Q8_0, 262144, 2816), (HQ_Q4_0, 262144, 2816),
                                   (HQ_Q4_0, 152064, 3584), (HQ_Q8_0, 65536, 7168)])
def test_rows_that_are_not_whole_windows(oracle, dev, xdt, t, n, k):
    """Q8_0 / Q4_0 matrices (windows of 64 block pairs) and K-quant matrices whose rows are not whole windows of sixteen super-blocks (hidden sizes 2560 .. 3840, 5120, 7168; k =
    14336): every wave takes one fixed window of the period after which the row boundaries repeat (11 windows = 16 rows
    for k = 2816, 5 = 8 for 2560, 3 = 4 for 3072, 7 = 8 for 3584, 15 = 16 for 3840, 5 = 4 for 5120, 7 = 4 for 7168, 7 = 2 for
    14336), the rows' parts meet in LDS.  151936 x 3072 leaves a workgroup more periods than its slots hold (two rounds)
    and a ragged share.  Sampled rows against the f64 oracle; Q6_K, Q8_0, Q4_0: the same bits as the flat walk, which a matrix off the
    16-byte grid takes; slices of 2048 rows against the kernels whose lanes fetch their own pieces; two activation rows; the
    same on a second call."""
    w = _quantized(dev, n, k, t, 31 + n + k)
    rng = np.random.default_rng(n + k)
    x = (rng.integers(-12, 13, (2, k)) / 8.0).astype(np.float32)
    xd = torch.from_numpy(x).to(dev)
    xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
    p = GgmlQuantizedMatmulParams(1, n, k, t)
    y = torch.full((1, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd[0:1], w, y, p)
    assert torch.isfinite(y).all()
    rows = np.unique(np.concatenate([np.arange(0, 34), np.arange(n - 34, n), rng.integers(0, n, 60)]))
    xv = oracle.f32_to_bf16_bits(x) if xdt == "bf16" else x
    ref = oracle.qmatmul_f64(xv, _rows_of(w, rows, k, t, oracle), 2, rows.size, k, t)
    sel = torch.as_tensor(rows, device=dev)
    assert_matmul_close(y[:, sel].cpu().numpy(), ref[0:1], f"type {t} {xdt} {n}x{k}, sampled rows")
    if t in (HQ_Q6_K, HQ_Q8_0, HQ_Q4_0):  # (Q4_K / Q5_K matrices must lie on the 16-byte grid)
        holder = torch.zeros(w.numel() + 32, dtype=torch.uint8, device=dev)
        shifted = holder[2:2 + w.numel()]
        shifted.copy_(w)
        ys = torch.full((1, n), float("nan"), device=dev)
        ops.quantized_matmul_ggml(xd[0:1], shifted, ys, p)
        assert torch.equal(y, ys), (t, n, k, xdt)
        del holder, shifted, ys
    # every row against the product over slices of the matrix small enough for the kernels whose lanes fetch their own pieces
    row_bytes = k // oracle.BLOCK_ELEMS[t] * oracle.BLOCK_BYTES[t]
    part = 2048
    for r0 in (0, (n - part) // 2 + 3, n - part):
        ysl = torch.full((1, part), float("nan"), device=dev)
        ops.quantized_matmul_ggml(xd[0:1], w[r0 * row_bytes:(r0 + part) * row_bytes].clone(), ysl, GgmlQuantizedMatmulParams(1, part, k, t))
        assert (ysl - y[:, r0:r0 + part]).abs().max().item() <= 2e-6 * np.abs(ref).max(), (t, xdt, n, k, r0)
    y2 = torch.full((2, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd, w, y2, GgmlQuantizedMatmulParams(2, n, k, t))
    # (two f32 rows: two passes of this kernel; two bf16 rows: the small-batch kernel where the matrix fits its stage-once form)
    assert (y2[0:1] - y).abs().max().item() <= 1e-4 * np.abs(ref).max()
    assert_matmul_close(y2[:, sel].cpu().numpy(), ref, f"type {t} {xdt} {n}x{k}, two rows")
    y3 = torch.full((1, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(xd[0:1], w, y3, p)
    assert torch.equal(y, y3)


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, HQ_Q4_0])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("n,k", [(8200, 4096), (8195, 1024), (40000, 2048), (8203, 2816), (9001, 3584), (8192, 5120), (33000, 2816), (1000, 2816),
                                 (4100, 3584)])
def test_small_batch_rows_staged_once(oracle, dev, t, xdt, n, k):
    """3 .. 8 activation rows over matrices of two groups of 16 rows per CU or more, all of k in LDS: the small-batch form
    that stages the activations once per CU (bf16: weights fetched as 16-byte pieces through LDS; f32: fetched by the
    lanes that use them).  Ragged last group (n % 16 = 8 / 3 / 0 / 11 / 9).  k = 2816, 3584 and 5120 are not whole chunks
    of 1024 activations (the last chunk holds 3, 2 and 1 super-blocks): only this form takes them; 5120 as f32 does not fit
    the LDS and runs a pass per row.  Q8_0 and Q4_0 (eight blocks = a super-block of seventeen / nine pieces, one MFMA per block
    over the bytes / nibbles as bf16) take the form with bf16 rows from two rows on; f32 rows up to four likewise, five to eight as two
    passes on matrices of 32768 rows or more (33000 x 2816), else through the kernel of exact f32 products.  1000 x 2816 and 4100 x 3584: K-quant
    matrices too small for the form at two or three rows (a pass per row), which takes them from four rows on because such k has
    no other kernel that reads the weights once.  Sampled rows against the f64 oracle, every row
    against the one-row product of the same activations, and the same result on a second call."""
    w = _quantized(dev, n, k, t, 11 + n + t)
    rng = np.random.default_rng(n + k + t)
    rows = np.unique(np.concatenate([[0, 1, 15, 16, n - 17, n - 16, n - 2, n - 1], rng.integers(0, n, 50)]))
    wr = _rows_of(w, rows, k, t, oracle)
    for m in (2, 3, 4, 5, 8):  # (up to four f32 rows are staged as hi and lo parts in the space of eight bf16 rows)
        x = acts(m + n, m, k)
        xd = torch.from_numpy(x).to(dev)
        xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
        xv = oracle.f32_to_bf16_bits(x) if xdt == "bf16" else x
        y = torch.full((m, n), float("nan"), device=dev)
        p = GgmlQuantizedMatmulParams(m, n, k, t)
        ops.quantized_matmul_ggml(xd, w, y, p)
        assert torch.isfinite(y).all()
        ref = oracle.qmatmul_f64(xv, wr, m, rows.size, k, t)
        assert_matmul_close(y[:, torch.as_tensor(rows, device=dev)].cpu().numpy(), ref, f"rows staged once t={t} {xdt} {m}x{n}x{k}")
        y1 = torch.empty((1, n), device=dev)
        for r in range(m):
            ops.quantized_matmul_ggml(xd[r:r + 1].contiguous(), w, y1, GgmlQuantizedMatmulParams(1, n, k, t))
            assert (y1[0] - y[r]).abs().max().item() <= 1e-4 * np.abs(ref).max()
        y2 = torch.full((m, n), float("nan"), device=dev)
        ops.quantized_matmul_ggml(xd, w, y2, p)
        assert torch.equal(y, y2)


# The reference's own decode shapes and dtype: f32 activations (gpu_full_attn.rs:835), k = 2816 (Gemma-4 projections, 11
# super-blocks per row: windows of the streaming walk straddle rows) and k = 2048 (Qwen3.6 hidden: two rows per window), and
# the 32-weight-block types; plus k = 4096 with f32 activations.  All of them take the flat streaming GEMV.
# (4096, 5120), (2048, 14336) and (2048, 17408): rows of a window of sixteen super-blocks or more, whole and ragged, which the
# Q6_K walk copies through LDS under bf16 activations.
# (1024, 2816) ... (100, 5632): the projections of a decode step; rows whose super-block count is not a power of two take the flat
# form from sixteen windows on, f32 activations and the 32-weight-block types from half a window per CU.
FLAT_SHAPES = [(12288, 2816), (16384, 2048), (12288, 4096), (4099, 11264), (4096, 2816), (2816, 4096), (1500, 8960), (4096, 5120),
               (2048, 14336), (2048, 17408), (1024, 2816), (256, 2816), (130, 2816), (24, 2816), (1024, 5120), (512, 1024), (100, 5632),
               (300, 4096)]


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, HQ_Q4_0])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("n,k", FLAT_SHAPES)
def test_decode_gemv_any_k_and_dtype(oracle, dev, t, xdt, n, k):
    w = _quantized(dev, n, k, t, 11 + n + k)
    rng = np.random.default_rng(n + k + t)
    m = 2 if (n, k) == (16384, 2048) else 1
    xa = (rng.integers(-12, 13, (m, k)) / 8.0).astype(np.float32)  # exact in bf16
    xb = (rng.integers(-12, 13, (m, k)) / 8.0).astype(np.float32)
    if xdt == "f32":  # values that need all of f32's 24 bits
        xa = (xa + rng.standard_normal((m, k)) * 1e-3).astype(np.float32)
        xb = (xb + rng.standard_normal((m, k)) * 1e-3).astype(np.float32)
    p = GgmlQuantizedMatmulParams(m, n, k, t)

    def run(x):
        y = torch.full((m, n), float("nan"), device=dev)
        xd = torch.from_numpy(x).to(dev)
        ops.quantized_matmul_ggml(xd.to(torch.bfloat16) if xdt == "bf16" else xd, w, y, p)
        return y

    ya, yb, yab = run(xa), run(xb), run((xa + xb).astype(np.float32))
    assert torch.isfinite(yab).all()
    rows = np.unique(np.concatenate([[0, 1, 2, 15, 16, 17, n - 3, n - 2, n - 1], rng.integers(0, n, 80)]))
    xin = oracle.f32_to_bf16_bits(xa) if xdt == "bf16" else xa
    ref = oracle.qmatmul_f64(xin, _rows_of(w, rows, k, t, oracle), m, rows.size, k, t)
    assert_matmul_close(ya[:, torch.as_tensor(rows, device=dev)].cpu().numpy(), ref, f"gemv {n}x{k} t={t} {xdt}, sampled rows")
    scale = yab.abs().max().item()
    assert (yab - (ya + yb)).abs().max().item() <= 2e-5 * scale
    assert torch.equal(run(xa * 4.0), ya * 4.0)


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q6_K, HQ_Q8_0])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("n,k", [(12288, 2816), (6144, 5120)])
def test_gate_and_up_in_one_launch_any_k(oracle, dev, t, xdt, n, k):
    """Two matrices of one shape over the same activations as one batched launch: the bits of the two separate calls."""
    wg, wu = _quantized(dev, n, k, t, 5), _quantized(dev, n, k, t, 6)
    g = torch.Generator(device=dev)
    g.manual_seed(9)
    x = torch.randn(1, k, generator=g, device=dev)
    x = x.to(torch.bfloat16) if xdt == "bf16" else x
    p = GgmlQuantizedMatmulParams(1, n, k, t)
    yg, yu, bg, bu = (torch.full((1, n), float("nan"), device=dev) for _ in range(4))
    ops.quantized_matmul_ggml(x, wg, yg, p)
    ops.quantized_matmul_ggml(x, wu, yu, p)
    ops.quantized_matmul_batch_ggml([ops.QmatmulJob(x, wg, bg, 1, n, k), ops.QmatmulJob(x, wu, bu, 1, n, k)], t)
    assert torch.equal(yg, bg) and torch.equal(yu, bu)
    rows = np.arange(0, n, 397)
    xin = oracle.f32_to_bf16_bits(x.float().cpu().numpy()) if xdt == "bf16" else x.cpu().numpy()
    ref = oracle.qmatmul_f64(xin, _rows_of(wu, rows, k, t, oracle), 1, rows.size, k, t)
    assert_matmul_close(bu[:, torch.as_tensor(rows, device=dev)].cpu().numpy(), ref, "up of the pair")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0])
def test_prefill_gemm_full_size(oracle, dev, t):
    """2048 tokens x K = 4096 x N = 12288, Q4_K and Q8_0 (both variants of BASELINE config 4), bf16 activations: a
    sample of (token, weight row) pairs against the oracle, scaling of a token row by a power of two, and agreement
    of token rows with the m = 1 GEMV."""
    m, k, n = 2048, 4096, 12288
    w = _quantized(dev, n, k, t, 1234)
    g = torch.Generator(device=dev)
    g.manual_seed(5678)
    x = torch.randn(m, k, generator=g, device=dev).to(torch.bfloat16)
    p = GgmlQuantizedMatmulParams(m, n, k, t)
    ws = torch.empty(ops.quantized_matmul_workspace_bytes(p, torch.bfloat16), dtype=torch.uint8, device=dev)
    y = torch.full((m, n), float("nan"), device=dev)
    ops.quantized_matmul_ggml(x, w, y, p, workspace=ws)
    assert torch.isfinite(y).all()
    rng = np.random.default_rng(3)
    toks = np.unique(np.concatenate([[0, 255, 256, m - 1], rng.integers(0, m, 12)]))
    rows = np.unique(np.concatenate([[0, 127, 128, n - 1], rng.integers(0, n, 44)]))
    xs = x[torch.as_tensor(toks, device=dev)].float().cpu().numpy()
    ref = oracle.qmatmul_f64(oracle.f32_to_bf16_bits(xs), _rows_of(w, rows, k, t, oracle), toks.size, rows.size, k, t)
    got = y[torch.as_tensor(toks, device=dev)][:, torch.as_tensor(rows, device=dev)].cpu().numpy()
    assert_matmul_close_f16_tile(got, ref, "prefill gemm, sampled tokens x rows")
    # The distribution of the error, tighter than the gate above (the tile kernels round every dequantised weight once
    # to f16, so they are not held to the GEMV's bound element by element).  Observed at this shape, Q4_K / Q8_0 /
    # Q6_K alike: |err| / rms(ref) median 1.4e-4, 99th percentile 5.3e-4, maximum 7.6e-4 .. 8.4e-4; rms error 2.1e-4
    # of the output rms; 93 % of the elements inside the GEMV's own bound 1e-3 |ref| + 1e-4 rms; every output of at
    # least rms magnitude within 7.5e-4 of its own value.
    e = np.abs(got.astype(np.float64) - ref).reshape(-1)
    r = np.abs(ref).reshape(-1)
    rms = float(np.sqrt(np.mean(r * r)))
    assert np.quantile(e, 0.5) <= 2.5e-4 * rms and np.quantile(e, 0.99) <= 8e-4 * rms and e.max() <= 1.5e-3 * rms
    assert np.mean(e <= 1e-3 * r + 1e-4 * rms) >= 0.9
    big = r >= rms
    assert (e[big] <= 1e-3 * r[big]).all(), "an output of at least rms magnitude is off by more than 1e-3 of its value"
    # a token row scaled by 2^5 gives that output row scaled by 2^5, bit for bit; the others do not move
    x2 = x.clone()
    x2[777] *= 32.0
    y2 = torch.empty_like(y)
    ops.quantized_matmul_ggml(x2, w, y2, p, workspace=ws)
    assert torch.equal(y2[777], y[777] * 32.0)
    assert torch.equal(y2[:777], y[:777]) and torch.equal(y2[778:], y[778:])
    # token rows agree with the GEMV of the same row (exact products there, f16-rounded weights here)
    y1 = torch.empty(1, n, device=dev)
    for i in (0, 1029, m - 1):
        ops.quantized_matmul_ggml(x[i:i + 1].contiguous(), w, y1, GgmlQuantizedMatmulParams(1, n, k, t))
        assert (y[i] - y1[0]).abs().max().item() <= 1e-3 * y1.abs().max().item()


@pytest.mark.parametrize("shape", ["gate_up", "down"])
def test_grouped_mul_mat_id_full_size(oracle, dev, shape):
    """Prefill-sized mul_mat_id of BASELINE config 3's layer: 2048 tokens x top-8 over 256 Q4_K experts, expert
    512 x 2048 with one activation row per token (gate / up) or 2048 x 512 with one per routed row (down).  The
    grouped tile form against the oracle on a sample of routed rows, against the per-row GEMV form (exact products,
    itself checked against the oracle elsewhere) on every output, and with the stack's weight-row scales computed
    once: the same bits."""
    E, K, T = 256, 8, 2048
    n, k = (512, 2048) if shape == "gate_up" else (2048, 512)
    t = HQ_Q4_K
    stack = _quantized(dev, E * n, k, t, 4321 + n)
    stride = n * (k // oracle.BLOCK_ELEMS[t]) * oracle.BLOCK_BYTES[t]
    g = torch.Generator(device=dev)
    g.manual_seed(99)
    rows, top_k = (T, K) if shape == "gate_up" else (T * K, 1)
    x = torch.randn(rows, k, generator=g, device=dev).to(torch.bfloat16)
    ids = torch.randint(0, E, (T * K,), generator=g, device=dev, dtype=torch.int32)
    p = ops.GgmlQuantizedMatmulIdParams(rows, top_k, n, k, E, stride, t)
    need = ops.quantized_matmul_id_workspace_bytes(p)
    assert need > 0, "this shape takes the grouped route"
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    y = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_ggml(x, stack, ids, y, p, scratch=scratch)
    assert torch.isfinite(y).all()
    # (a) sampled routed rows against the f64 oracle
    rng = np.random.default_rng(5)
    ids_h = ids.cpu().numpy()
    for pair in np.unique(np.concatenate([[0, 1, T * K - 1], rng.integers(0, T * K, 13)])):
        e = int(ids_h[pair])
        xs = x[pair // top_k:pair // top_k + 1].float().cpu().numpy()
        wrows = stack[e * stride:(e + 1) * stride].cpu().numpy()
        ref = oracle.qmatmul_f64(oracle.f32_to_bf16_bits(xs), wrows, 1, n, k, t)
        assert_matmul_close_f16_tile(y[pair].cpu().numpy(), ref, f"grouped {shape}, routed row {pair} (expert {e})")
    # (b) every output against the per-row GEMV form
    y_gemv = torch.empty_like(y)
    ops.quantized_matmul_id_ggml(x, stack, ids, y_gemv, p)
    ref = y_gemv.double()
    rms = ref.pow(2).mean().sqrt().item()
    err = (y.double() - ref).abs()
    assert (err <= 1e-3 * ref.abs() + 3e-3 * rms).all()
    assert err.pow(2).mean().sqrt().item() <= 5e-4 * rms
    # (c) the weight-row scales kept from an earlier pass over the stack
    scales = ops.weight_row_scales_ggml(stack, E * n, k, t)
    scratch.fill_(0xFF)
    y2 = torch.full_like(y, float("nan"))
    ops.quantized_matmul_id_ggml(x, stack, ids, y2, p, scratch=scratch, w_row_scales=scales)
    assert torch.equal(y, y2)


def test_grouped_swiglu_full_size(oracle, dev):
    """Gate, up and SwiGLU of BASELINE config 3's layer at prefill size (2048 tokens x top-8 over 256 Q4_K experts of
    512 x 2048) as one grouped product: the bits of the two grouped calls followed by silu_mul, and a sample of routed
    rows against silu(gate) * up of the f64 oracle."""
    E, K, T, n, k, t = 256, 8, 2048, 512, 2048, HQ_Q4_K
    gate, up = _quantized(dev, E * n, k, t, 777), _quantized(dev, E * n, k, t, 778)
    stride = n * (k // oracle.BLOCK_ELEMS[t]) * oracle.BLOCK_BYTES[t]
    g = torch.Generator(device=dev)
    g.manual_seed(42)
    x = torch.randn(T, k, generator=g, device=dev).to(torch.bfloat16)
    ids = torch.randint(0, E, (T * K,), generator=g, device=dev, dtype=torch.int32)
    p = ops.GgmlQuantizedMatmulIdParams(T, K, n, k, E, stride, t)
    need = ops.quantized_matmul_id_swiglu_workspace_bytes(p)
    assert need > 0
    scratch = torch.empty(need, dtype=torch.uint8, device=dev)
    yg, yu, sep = (torch.empty(T * K, n, device=dev) for _ in range(3))
    ops.quantized_matmul_id_ggml(x, gate, ids, yg, p, scratch=scratch)
    ops.quantized_matmul_id_ggml(x, up, ids, yu, p, scratch=scratch)
    ops.dispatch_silu_mul(yg, yu, sep)
    y = torch.full((T * K, n), float("nan"), device=dev)
    ops.quantized_matmul_id_swiglu_ggml(x, gate, up, ids, y, p, scratch)
    assert torch.equal(y, sep)
    rng = np.random.default_rng(6)
    ids_h = ids.cpu().numpy()
    for pair in np.unique(np.concatenate([[0, T * K - 1], rng.integers(0, T * K, 10)])):
        e = int(ids_h[pair])
        xs = oracle.f32_to_bf16_bits(x[pair // K:pair // K + 1].float().cpu().numpy())
        rg = oracle.qmatmul_f64(xs, gate[e * stride:(e + 1) * stride].cpu().numpy(), 1, n, k, t)
        ru = oracle.qmatmul_f64(xs, up[e * stride:(e + 1) * stride].cpu().numpy(), 1, n, k, t)
        ref = (rg / (1.0 + np.exp(-rg)) * ru).reshape(-1)
        got = y[pair].cpu().numpy().astype(np.float64)
        assert np.sqrt(np.mean((got - ref) ** 2)) <= 1.5e-3 * np.sqrt(np.mean(ref * ref)), pair
        assert np.abs(got - ref).max() <= 5e-3 * np.abs(ref).max(), pair


def test_moe_layer_full_size(oracle, dev):
    """hidden 2048, 256 experts x inter 512 (Q4_K), one shared expert, top-8, one token and eight: the block against
    a float64 evaluation over the device-dequantised weights of the experts the router picked.  The reference here is
    the library's own dequantiser (hq_dequant_ggml) and torch float64 on the GPU, not the CPU oracle (150 MB stacks);
    it counts as a reference only because hq_dequant_ggml is held bit-exact to the oracle by test_dequant_bit_exact and
    test_dequant_golden_blocks, and the routing is checked against the CPU specification below."""
    H, E, I, K, t = 2048, 256, 512, 8, HQ_Q4_K
    g = torch.Generator(device=dev)
    g.manual_seed(99)
    rnd = lambda *s: torch.randn(*s, generator=g, device=dev)  # noqa: E731
    w = ops.MoeFfnWeightsGpuQ(
        router=(rnd(E, H) * 0.1).to(torch.bfloat16), expert_gate=_quantized(dev, E * I, H, t, 1),
        expert_up=_quantized(dev, E * I, H, t, 2), expert_down=_quantized(dev, E * H, I, t, 3),
        shared_gate_logit=(rnd(1, H) * 0.1).to(torch.bfloat16), shared_gate=_quantized(dev, I, H, t, 4),
        shared_up=_quantized(dev, I, H, t, 5), shared_down=_quantized(dev, H, I, t, 6),
        n_experts=E, top_k=K, hidden=H, inter=I, shared_inter=I, ggml_type=t)
    deq = lambda b, r, c: ops.dequantize_ggml(b, r * c, t).view(r, c).double()  # noqa: E731
    sg, su, sd = deq(w.shared_gate, I, H), deq(w.shared_up, I, H), deq(w.shared_down, H, I)
    rb_h, rb_i = ops.ggml_row_bytes(t, H), ops.ggml_row_bytes(t, I)
    for T in (1, 8):
        x = rnd(T, H).to(torch.bfloat16)
        s = ops.MoeFfnScratch(w, T, dev)
        out = torch.full((T, H), float("nan"), device=dev)
        ops.build_moe_ffn_layer_gpu_q_into(x, w, s, out)  # default: the one-launch block (hq_moe_ffn_decode)
        assert int(s.fused[4:8].view(torch.int32).item()) == 0
        ops.dense_gemv_bf16_f32(x, w.router, s.logits, T, E, H)  # the router logits, which the one launch keeps to itself
        xd = x.double()
        ids, tw = s.ids.view(T, K).long(), s.topk_w.view(T, K).double()
        # the routing itself: softmax / top-k of the router logits, against the CPU specification
        want_i, want_w = oracle.softmax_topk_renorm(s.logits.cpu().numpy(), T, E, K)
        assert np.array_equal(ids.cpu().numpy().reshape(-1).astype(np.uint32), want_i)
        assert np.allclose(tw.cpu().numpy().reshape(-1), want_w, rtol=1e-5, atol=1e-7)
        assert torch.allclose(s.logits.double(), xd @ w.router.double().T, rtol=1e-4, atol=1e-4)
        ref = torch.zeros(T, H, dtype=torch.float64, device=dev)
        for ti in range(T):
            for kk in range(K):
                e = int(ids[ti, kk])
                eg = deq(w.expert_gate.view(E, -1)[e], I, H)
                eu = deq(w.expert_up.view(E, -1)[e], I, H)
                ed = deq(w.expert_down.view(E, -1)[e], H, I)
                a = torch.nn.functional.silu(eg @ xd[ti]) * (eu @ xd[ti])
                ref[ti] += tw[ti, kk] * (ed @ a)
            gate = torch.sigmoid((w.shared_gate_logit.double() @ xd[ti])[0])
            ref[ti] += gate * (sd @ (torch.nn.functional.silu(sg @ xd[ti]) * (su @ xd[ti])))
        assert rb_h * I * E == w.expert_gate.numel() and rb_i * H * E == w.expert_down.numel()
        err = (out.double() - ref).abs().max().item()
        rms = ref.pow(2).mean().sqrt().item()
        assert err <= 2e-3 * rms, f"T={T}: max err {err} vs rms {rms}"


def test_tq_attention_full_size(oracle, dev):
    """32768 cached tokens, 16 query heads over 2 KV heads, head_dim 256, int8 codes: the whole output against the
    f64 oracle, the fused rotate-attend-rotate call against the three separate calls, and the closed form of a
    cache whose values are all one vector."""
    nh, nkv, hd, n = 16, 2, 256, 32768
    rng = np.random.default_rng(5)
    kc = rng.integers(-127, 128, (nkv, n, hd)).astype(np.int8).view(np.uint8)
    vc = rng.integers(-127, 128, (nkv, n, hd)).astype(np.int8).view(np.uint8)
    kn = rng.uniform(0.5, 2.0, (nkv, n, 1)).astype(np.float32)
    vn = rng.uniform(0.5, 2.0, (nkv, n, 1)).astype(np.float32)
    q = rng.standard_normal((nh, hd)).astype(np.float32)
    qr = oracle.fwht_sign_premult(q.copy(), nh, hd)
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, n, 1.0 / 16.0)
    ref = oracle.tq_attention(qr, kc, kn, vc, vn, None, nh, nkv, hd, n, n, p.scale)
    d = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    kcd, knd, vcd, vnd = d(kc), d(kn), d(vc), d(vn)
    tmp = torch.empty(ops.tq_tmp_buffer_bytes(nh, hd, n) // 4, device=dev)
    out = torch.full((nh, hd), float("nan"), device=dev)
    ops.flash_attn_vec_tq_hb(d(qr), kcd, knd, vcd, vnd, out, tmp, p)
    got = out.cpu().numpy()
    scale = np.abs(ref).max(axis=1, keepdims=True)
    assert np.isfinite(got).all() and (np.abs(got - ref) <= 1e-3 * scale).all()
    assert np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()) < 1e-4
    # one call with both rotations inside = rotate, attend, rotate back
    sep = out.clone()
    ops.dispatch_fwht_sign_undo_f32(sep, nh, hd)
    fused = torch.full((nh, hd), float("nan"), device=dev)
    pf = FlashAttnVecTqHbParams(nh, nkv, hd, n, n, 1.0 / 16.0, fuse_fwht_pre=1)
    ops.flash_attn_vec_tq_hb(d(q), kcd, knd, vcd, vnd, fused, tmp, pf, undo_rotation=True)
    assert torch.equal(fused, sep)
    # every cached value the same vector (per KV head): the output is that vector whatever the scores
    v1 = rng.integers(-127, 128, (nkv, 1, hd)).astype(np.int8)
    vcc = np.broadcast_to(v1, (nkv, n, hd)).copy().view(np.uint8)
    vnc = np.full((nkv, n, 1), 1.25, np.float32)
    ops.flash_attn_vec_tq_hb(d(qr), kcd, knd, d(vcc), d(vnc), out, tmp, p)
    want = np.repeat(oracle.tq_dequantize(vcc, vnc, None, nkv, hd, n, 0, 1)[:, 0, :], nh // nkv, axis=0)
    # (the softmax weights are 22-bit numbers summed over 32768 positions: 2e-5 of the magnitude observed)
    err, mag = float(np.abs(out.cpu().numpy() - want).max()), float(np.abs(want).max())
    assert err <= 1e-4 * mag, f"constant-value cache: {err} vs {mag}"


def test_tq_attention_full_size_over_an_encoded_cache(oracle, dev):
    """BASELINE config 5 as it is stated: K and V ~ N(0, 1), rotated and quantised per (token, head) by hq_tq_encode_kv
    (the cache then has the code and scale statistics of real keys, not uniform codes), 32768 positions, 16 / 2 heads,
    d = 256.  The device encode is byte-equal to the oracle's on sampled positions, the attention over the device-built
    cache matches the f64 oracle over the same bytes, and against exact f32 attention over the un-quantised K / V the
    whole chain stays far inside the reference's NRMSE gate (kv_cache.rs:3959: < 0.15)."""
    nh, nkv, hd, n = 16, 2, 256, 32768
    g = torch.Generator(device=dev)
    g.manual_seed(1234)
    k = torch.randn(n, nkv, hd, generator=g, device=dev)
    v = torch.randn(n, nkv, hd, generator=g, device=dev)
    q = torch.randn(nh, hd, generator=g, device=dev)
    kc, kn = ops.alloc_tq_kv(nkv, n, hd, dev)
    vc, vn = ops.alloc_tq_kv(nkv, n, hd, dev)
    ops.hadamard_quantize_kv(k, kc, kn, 0)
    ops.hadamard_quantize_kv(v, vc, vn, 0)
    kch, knh, vch, vnh = (t.cpu().numpy() for t in (kc, kn, vc, vn))
    # the encode, on sampled positions, against the oracle
    rng = np.random.default_rng(7)
    for pos in np.unique(np.concatenate([[0, 1, n - 1], rng.integers(0, n, 29)])):
        codes = np.zeros((nkv, 1, hd), np.uint8)
        norms = np.zeros((nkv, 1, 1), np.float32)
        oracle.tq_encode_int8(k[pos].cpu().numpy(), nkv, hd, 1, 0, codes, norms)
        assert np.array_equal(codes[:, 0], kch[:, pos]) and np.array_equal(norms[:, 0], knh[:, pos]), pos
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, n, 1.0 / 16.0, fuse_fwht_pre=1)
    tmp = torch.empty(ops.tq_tmp_buffer_bytes(nh, hd, n) // 4, device=dev)
    out = torch.full((nh, hd), float("nan"), device=dev)
    ops.flash_attn_vec_tq_hb(q, kc, kn, vc, vn, out, tmp, p, undo_rotation=True)
    got = out.cpu().numpy()
    qr = oracle.fwht_sign_premult(q.cpu().numpy().copy(), nh, hd)
    ref = oracle.tq_attention(qr, kch, knh, vch, vnh, None, nh, nkv, hd, n, n, p.scale)
    ref = oracle.fwht_sign_undo(ref.astype(np.float32), nh, hd)
    scale = np.abs(ref).max(axis=1, keepdims=True)
    assert np.isfinite(got).all() and (np.abs(got - ref) <= 1e-3 * scale).all()
    assert np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()) < 1e-4
    # against attention over the un-quantised keys and values (float64 on the device)
    qd, kd, vd = q.double(), k.double(), v.double()
    exact = torch.empty(nh, hd, dtype=torch.float64, device=dev)
    for h in range(nh):
        kv = h // (nh // nkv)
        w = torch.softmax((kd[:, kv, :] @ qd[h]) * p.scale, dim=0)
        exact[h] = w @ vd[:, kv, :]
    ex = exact.cpu().numpy()
    nrmse = np.sqrt(((got - ex) ** 2).sum() / (ex ** 2).sum())
    assert nrmse < 0.05, nrmse

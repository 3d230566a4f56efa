"""GPU parity of the batched-prefill MFMA GEMM (m > 8) against the f64 oracle."""
import numpy as np
import pytest
import torch

from _util import acts, assert_matmul_close, assert_matmul_close_f16_tile, weights
from hf2q_amd import ops
from hf2q_amd.ops import HQ_Q4_0, HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, GgmlQuantizedMatmulParams

pytestmark = pytest.mark.gpu

def _f16_tile(t, k):
    return (t in (HQ_Q4_K, HQ_Q5_K, HQ_Q6_K) and k % 256 == 0) or (t in (HQ_Q8_0, HQ_Q4_0) and k % 128 == 0)


def _check(t, k):
    """Q4_K / Q5_K / Q6_K (k % 256 == 0) and Q8_0 / Q4_0 with k % 128 == 0 take the f16 tile kernels; everything else
    keeps every product exact."""
    return assert_matmul_close_f16_tile if _f16_tile(t, k) else assert_matmul_close


SHAPES = [  # (m, n, k): tile edges in every dimension (tile is 256 x 128 x 64); k = 320: exact kernels for Q8_0
    (9, 128, 256), (33, 200, 512), (256, 128, 1024), (300, 257, 768), (64, 96, 4096), (513, 384, 256), (40, 130, 320),
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


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0, HQ_Q6_K, HQ_Q5_K, HQ_Q4_0])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_matches_f64_oracle(oracle, dev, t, xdt, m, n, k):
    if k % oracle.BLOCK_ELEMS[t]:
        pytest.skip("k is not a multiple of the block size")
    y, ref = _run(oracle, dev, t, xdt, m, n, k)
    _check(t, k)(y, ref, f"gemm t={t} {xdt} {m}x{n}x{k}")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, HQ_Q4_0])
@pytest.mark.parametrize("m,n,k", [
    (17, 64, 2048),     # one tile, k in two slices
    (65, 130, 2304),    # ragged weight rows, nine runs of 256 in slices of five and four
    (128, 70, 4352),    # seventeen runs in four slices (5, 5, 5, 2)
    (100, 320, 256),    # a single run: no slices
    (64, 12288, 512),   # more tiles than CUs' worth: no slices
    (40, 200, 1152),    # Q8_0 / Q4_0 only: k % 256 = 128, the last run is half a one (and k is not cut)
    (200, 130, 2304),   # one token tile of 256 rows, two slices
    (256, 64, 4352),    # a full one, four slices
    (64, 1536, 8960),   # 35 runs: slices of five, seven of them (eight of ceil(35 / 8) would leave the last one empty)
    (200, 256, 8448),   # 33 runs
])
def test_small_tiles_and_k_slices_match_f64_oracle(oracle, dev, t, m, n, k):
    """Up to 256 activation rows are one token tile (64, 128 or 256 rows; Q4_K / Q5_K have the 64-row one), with k cut
    into slices (summed in a fixed order by a second launch) where the weight-row tiles alone would leave most CUs idle;
    the same result on every call."""
    if k % oracle.BLOCK_ELEMS[t]:
        pytest.skip("k is not a multiple of the block size")
    y, ref = _run(oracle, dev, t, "bf16", m, n, k)
    assert_matmul_close_f16_tile(y, ref, f"small tiles t={t} {m}x{n}x{k}")
    y2, _ = _run(oracle, dev, t, "bf16", m, n, k)
    assert np.array_equal(y, y2)


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0, HQ_Q6_K, HQ_Q5_K, HQ_Q4_0])
def test_gemm_adversarial_blocks(oracle, dev, t):
    """Every scale / min / nibble bit pattern (raw random bytes with finite f16 fields)."""
    m, n, k = 72, 128, 512  # past every type's chunked range: the tile kernels
    bb = oracle.BLOCK_BYTES[t]
    raw = np.random.default_rng(9).integers(0, 256, size=n * k // oracle.BLOCK_ELEMS[t] * bb, dtype=np.uint8)
    for off in ([1, 3] if t in (HQ_Q4_K, HQ_Q5_K) else [209] if t == HQ_Q6_K else [1]):
        raw[off::bb] &= 0x3F
    for xdt in ("bf16", "f32"):
        y, ref = _run(oracle, dev, t, xdt, m, n, k, blocks=raw)
        _check(t, k)(y, ref, f"gemm adversarial t={t} {xdt}")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0, HQ_Q6_K, HQ_Q5_K, HQ_Q4_0])
def test_gemm_rows_equal_gemv_rows(oracle, dev, t):
    """Row i of the m>8 result agrees with the m=1 GEMV of activation row i; the tile kernels round
    their weights to f16, so the agreement is to 1e-3 of the row's largest output."""
    m, n, k = 72, 256, 1024
    blocks = oracle.quantize(weights(5, n, k), k, t, threads=8)
    wd = torch.from_numpy(blocks).to(dev)
    x = torch.from_numpy(acts(6, m, k)).to(dev).to(torch.bfloat16)
    y = torch.empty(m, n, device=dev)
    ops.quantized_matmul_ggml(x, wd, y, GgmlQuantizedMatmulParams(m, n, k, t))
    y1 = torch.empty(1, n, device=dev)
    for i in (0, 7, 71):
        ops.quantized_matmul_ggml(x[i:i + 1].contiguous(), wd, y1, GgmlQuantizedMatmulParams(1, n, k, t))
        scale = y1.abs().max().item()
        assert (y[i] - y1[0]).abs().max().item() <= 1e-3 * scale


def test_gemm_zero_weights_give_zero(oracle, dev):
    m, n, k = 32, 128, 512
    blocks = oracle.quantize(np.zeros((n, k), np.float32), k, HQ_Q4_K)
    y = torch.full((m, n), 3.0, device=dev)
    ops.quantized_matmul_ggml(torch.randn(m, k, device=dev).to(torch.bfloat16), torch.from_numpy(blocks).to(dev), y,
                              GgmlQuantizedMatmulParams(m, n, k, HQ_Q4_K))
    assert not y.cpu().numpy().any()


def test_q4k_tile_gemm_workspace_variant(oracle, dev):
    """The caller-owned-scratch entry point gives the same bits as the allocating one, says how much it
    needs, and rejects a short buffer."""
    from hf2q_amd import lib

    m, n, k = 48, 160, 512
    blocks = oracle.quantize(weights(11, n, k), k, HQ_Q4_K, threads=8)
    wd = torch.from_numpy(blocks).to(dev)
    x = torch.from_numpy(acts(12, m, k)).to(dev).to(torch.bfloat16)
    p = GgmlQuantizedMatmulParams(m, n, k, HQ_Q4_K)
    need = ops.quantized_matmul_workspace_bytes(p, torch.bfloat16)
    assert need >= m * k * 2 + m * 4
    assert ops.quantized_matmul_workspace_bytes(GgmlQuantizedMatmulParams(1, n, k, HQ_Q4_K), torch.bfloat16) == 0
    assert ops.quantized_matmul_workspace_bytes(GgmlQuantizedMatmulParams(m, n, k, HQ_Q8_0), torch.bfloat16) >= m * k * 2
    assert ops.quantized_matmul_workspace_bytes(GgmlQuantizedMatmulParams(m, n, 320, HQ_Q8_0), torch.bfloat16) == 0
    assert ops.quantized_matmul_workspace_bytes(GgmlQuantizedMatmulParams(m, n, k, HQ_Q6_K), torch.bfloat16) >= m * k * 2
    y0 = torch.empty(m, n, device=dev)
    y1 = torch.empty(m, n, device=dev)
    ops.quantized_matmul_ggml(x, wd, y0, p)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    ops.quantized_matmul_ggml(x, wd, y1, p, workspace=ws)
    assert torch.equal(y0, y1)
    with pytest.raises(lib.HqError):
        ops.quantized_matmul_ggml(x, wd, y1, p, workspace=ws[: need - 256])


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q5_K])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k", [(48, 160, 512), (300, 257, 768), (2048, 512, 2048), (130, 128, 256), (64, 1024, 4096),
                                   (127, 100, 2048)])
def test_dense_swiglu_tile_form(oracle, dev, t, xdt, m, n, k):
    """silu(x . Wg^T) * (x . Wu^T) as one call: the bits of the two tile products followed by silu_mul wherever the
    plain product sums all of k inside one tile (the shapes that also have the gated form; where it cuts k into slices
    the two associate the f32 sums differently and agree to a few units in the last place), the same with the row
    scales of both matrices computed beforehand, and silu(gate) * up of the f64 oracle's products."""
    from hf2q_amd import lib
    gate = oracle.quantize(weights(41 * n + k + t, n, k), k, t, threads=8)
    up = oracle.quantize(weights(43 * n + k + t, n, k), k, t, threads=8)
    x = acts(n + k + m, m, k)
    if xdt == "bf16":
        xv = oracle.f32_to_bf16_bits(x)
        xd = torch.from_numpy(xv.view(np.int16)).to(dev).view(torch.bfloat16).reshape(m, k)
    else:
        xv, xd = x, torch.from_numpy(x).to(dev)
    gd, ud = torch.from_numpy(gate).to(dev), torch.from_numpy(up).to(dev)
    p = GgmlQuantizedMatmulParams(m, n, k, t)
    adt = torch.bfloat16 if xdt == "bf16" else torch.float32
    need = ops.quantized_matmul_swiglu_workspace_bytes(p, adt)
    plain = ops.quantized_matmul_workspace_bytes(p, adt)  # larger than `need` where it holds partial sums of k slices
    assert need > 0 and plain > 0
    ws = torch.empty(max(need, plain), dtype=torch.uint8, device=dev)
    yg, yu, sep = (torch.empty(m, n, device=dev) for _ in range(3))
    ops.quantized_matmul_ggml(xd, gd, yg, p, workspace=ws)
    ops.quantized_matmul_ggml(xd, ud, yu, p, workspace=ws)
    ops.dispatch_silu_mul(yg.view(-1)[: m * n - (m * n) % 4], yu.view(-1)[: m * n - (m * n) % 4], sep.view(-1)[: m * n - (m * n) % 4])
    ws.fill_(0xFF)
    y = torch.full((m, n), float("nan"), device=dev)
    ops.quantized_matmul_swiglu_ggml(xd, gd, ud, y, p, ws)
    cut = m * n - (m * n) % 4
    if ops.quantized_matmul_gated_workspace_bytes(p, adt) > 0:
        assert torch.equal(y.view(-1)[:cut], sep.view(-1)[:cut])
    else:
        assert (k, m) in ((4096, 64), (2048, 127))  # only the sliced shapes may differ
        diff = (y.view(-1)[:cut] - sep.view(-1)[:cut]).abs().max().item()
        assert diff <= 4e-6 * sep.view(-1)[:cut].abs().max().item()
    ws.fill_(0xFF)
    y2 = torch.full((m, n), float("nan"), device=dev)
    ops.quantized_matmul_swiglu_ggml(xd, gd, ud, y2, p, ws, ops.weight_row_scales_ggml(gd, n, k, t), ops.weight_row_scales_ggml(ud, n, k, t))
    assert torch.equal(y2, y)
    rg, ru = oracle.qmatmul_f64(xv, gate, m, n, k, t), oracle.qmatmul_f64(xv, up, m, n, k, t)
    ref = rg / (1.0 + np.exp(-rg)) * ru
    got = y.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all()
    assert np.sqrt(np.mean((got - ref) ** 2)) <= 1.5e-3 * np.sqrt(np.mean(ref * ref))
    assert np.abs(got - ref).max() <= 5e-3 * np.abs(ref).max()
    with pytest.raises(lib.HqError):
        ops.quantized_matmul_swiglu_ggml(xd, gd, ud, y, p, ws[: need - 256])
    if ops.quantized_matmul_gated_workspace_bytes(p, adt) > 0:
        assert need >= plain


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0, HQ_Q6_K, HQ_Q5_K, HQ_Q4_0])
@pytest.mark.parametrize("m,n,k", [(300, 257, 768), (2048, 384, 512), (64, 1024, 256)])
def test_gated_epilogue_equals_product_then_silu_mul(oracle, dev, t, m, n, k):
    """y = silu(gate) * (x . W^T) from the up projection's epilogue: the bits of the product followed by silu_mul, also in
    place over the gate buffer and with the weight's row scales brought by the caller."""
    blocks = oracle.quantize(weights(51 * n + k + t, n, k), k, t, threads=8)
    wd = torch.from_numpy(blocks).to(dev)
    x = torch.from_numpy(acts(n + m, m, k)).to(dev).to(torch.bfloat16)
    gate = torch.from_numpy(acts(n + m + 1, m, n)).to(dev) * 2.0
    p = GgmlQuantizedMatmulParams(m, n, k, t)
    need = ops.quantized_matmul_gated_workspace_bytes(p, torch.bfloat16)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    up = torch.empty(m, n, device=dev)
    ops.quantized_matmul_ggml(x, wd, up, p, workspace=ws)
    want = gate / (1.0 + torch.exp(-gate)) * up  # torch's silu * up: close; the library's own kernel is the bit reference
    cut = m * n - (m * n) % 4
    sep = torch.empty(m, n, device=dev)
    ops.dispatch_silu_mul(gate.view(-1)[:cut], up.view(-1)[:cut], sep.view(-1)[:cut])
    y = torch.full((m, n), float("nan"), device=dev)
    ops.quantized_matmul_gated_ggml(x, wd, gate, y, p, ws)
    assert torch.equal(y.view(-1)[:cut], sep.view(-1)[:cut])
    assert torch.allclose(y, want, rtol=1e-5, atol=1e-6 * float(want.abs().max()))
    g2 = gate.clone()
    ops.quantized_matmul_gated_ggml(x, wd, g2, g2, p, ws, ops.weight_row_scales_ggml(wd, n, k, t))
    assert torch.equal(g2, y)


def test_gated_epilogue_has_no_form_where_k_is_cut_into_slices(dev):
    p = GgmlQuantizedMatmulParams(64, 256, 4096, HQ_Q4_K)  # 64 rows over two column tiles: slices of k
    assert ops.quantized_matmul_workspace_bytes(p, torch.bfloat16) > 0
    assert ops.quantized_matmul_gated_workspace_bytes(p, torch.bfloat16) == 0
    assert ops.quantized_matmul_gated_workspace_bytes(GgmlQuantizedMatmulParams(4, 256, 4096, HQ_Q4_K), torch.bfloat16) == 0


def test_dense_swiglu_has_no_form_for_other_types_and_few_rows(dev):
    assert ops.quantized_matmul_swiglu_workspace_bytes(GgmlQuantizedMatmulParams(64, 128, 512, HQ_Q6_K), torch.bfloat16) == 0
    assert ops.quantized_matmul_swiglu_workspace_bytes(GgmlQuantizedMatmulParams(4, 128, 512, HQ_Q4_K), torch.bfloat16) == 0
    x = torch.zeros(4, 512, device=dev)
    w = torch.zeros(128 * 2 * 144, dtype=torch.uint8, device=dev)
    with pytest.raises(ops.HqError) as e:
        ops.quantized_matmul_swiglu_ggml(x, w, w, torch.empty(4, 128, device=dev), GgmlQuantizedMatmulParams(4, 128, 512, HQ_Q4_K),
                                         torch.empty(256, dtype=torch.uint8, device=dev))
    assert e.value.status == 2


def _row_bounds(blocks, n, k, t):
    """Largest possible |w| of every weight row from its block headers alone, in f64."""
    per, nbytes, d_at = {HQ_Q4_K: (256, 144, 0), HQ_Q5_K: (256, 176, 0), HQ_Q6_K: (256, 210, 208), HQ_Q8_0: (32, 34, 0),
                         HQ_Q4_0: (32, 18, 0)}[t]
    b = blocks.reshape(n, k // per, nbytes)
    d = np.abs(b[:, :, d_at:d_at + 2].copy().view(np.float16).astype(np.float64)[:, :, 0])
    if t in (HQ_Q4_K, HQ_Q5_K):
        dmin = np.abs(b[:, :, 2:4].copy().view(np.float16).astype(np.float64)[:, :, 0])
        return (d * (63 * 15 if t == HQ_Q4_K else 63 * 31) + dmin * 63).max(axis=1)
    return (d * {HQ_Q6_K: 128 * 32, HQ_Q8_0: 128, HQ_Q4_0: 8}[t]).max(axis=1)


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0, HQ_Q6_K, HQ_Q5_K, HQ_Q4_0])
def test_prepared_weight_row_scales(oracle, dev, t):
    """The weight-row scales computed once (powers of two that bring a row's largest possible weight to [2^13, 2^14])
    and handed to the call give the bits of the call that works them out itself, for the large and the small tiles;
    a route without tile kernels ignores them."""
    for m, n, k in ((300, 257, 768), (48, 160, 512), (64, 200, 256)):
        blocks = oracle.quantize(weights(17 * n + k + t, n, k), k, t, threads=8)
        blocks = blocks.copy()
        per_row = blocks.size // n
        blocks[3 * per_row:4 * per_row] = 0  # a row of zero scales: scale 1
        wd = torch.from_numpy(blocks).to(dev)
        scales = ops.weight_row_scales_ggml(wd, n, k, t)
        sc = scales.cpu().numpy().astype(np.float64)
        mant, _ = np.frexp(sc)
        assert (mant == 0.5).all(), "powers of two"
        bound = _row_bounds(blocks, n, k, t)
        live = bound > 0
        assert live.sum() == n - 1 and sc[~live] == 1.0
        scaled = bound[live] * sc[live]
        assert (scaled >= 2.0 ** 13 * (1 - 1e-6)).all() and (scaled <= 2.0 ** 14 * (1 + 1e-6)).all()
        x = torch.from_numpy(acts(m + n, m, k)).to(dev).to(torch.bfloat16)
        p = GgmlQuantizedMatmulParams(m, n, k, t)
        need = ops.quantized_matmul_workspace_bytes(p, torch.bfloat16)
        assert need > 0
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        y0 = torch.empty(m, n, device=dev)
        ops.quantized_matmul_ggml(x, wd, y0, p, workspace=ws)
        ws.fill_(0xFF)  # nothing of the first call's pre-pass is left to lean on
        y1 = torch.full((m, n), float("nan"), device=dev)
        ops.quantized_matmul_ggml(x, wd, y1, p, workspace=ws, w_row_scales=scales)
        assert torch.equal(y0, y1), (m, n, k)
    # one row: the GEMV route, no workspace needed, the scales are not looked at
    p1 = GgmlQuantizedMatmulParams(1, n, k, t)
    ya, yb = torch.empty(1, n, device=dev), torch.empty(1, n, device=dev)
    ops.quantized_matmul_ggml(x[:1], wd, ya, p1)
    ops.quantized_matmul_ggml(x[:1], wd, yb, p1, workspace=ws, w_row_scales=scales)
    assert torch.equal(ya, yb)


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0, HQ_Q6_K, HQ_Q5_K, HQ_Q4_0])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
def test_tile_gemm_scale_equivariance(oracle, dev, xdt, t):
    """Activation rows and weight rows are rescaled by powers of two inside the kernel (f16 has a narrow
    exponent range): scaling an activation row by 2^a scales its output row by exactly 2^a, across 80
    binades, and weights 10^4 times smaller or larger than usual lose no accuracy."""
    m, n, k = 72, 128, 512  # past every type's chunked range: the tile kernels
    x = acts(21, m, k)
    if xdt == "bf16":
        x = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(x)).reshape(m, k)
    exps = np.array([(-40 + 2 * i) for i in range(m)], dtype=np.int32)
    xs = np.ldexp(x, exps[:, None]).astype(np.float32)
    for sigma in (0.02, 2e-6, 2e2):
        blocks = oracle.quantize(weights(22, n, k, sigma), k, t, threads=8)
        wd = torch.from_numpy(blocks).to(dev)
        tdt = torch.bfloat16 if xdt == "bf16" else torch.float32
        y = torch.empty(m, n, device=dev)
        ys = torch.empty(m, n, device=dev)
        p = GgmlQuantizedMatmulParams(m, n, k, t)
        ops.quantized_matmul_ggml(torch.from_numpy(x).to(dev).to(tdt), wd, y, p)
        ops.quantized_matmul_ggml(torch.from_numpy(xs).to(dev).to(tdt), wd, ys, p)
        assert np.array_equal(np.ldexp(y.cpu().numpy(), exps[:, None]).astype(np.float32), ys.cpu().numpy())
        xv = oracle.f32_to_bf16_bits(x) if xdt == "bf16" else x
        assert_matmul_close_f16_tile(y.cpu().numpy(), oracle.qmatmul_f64(xv, blocks, m, n, k, t),
                                     f"tile gemm t={t} sigma={sigma} {xdt}")


def test_shapes_without_a_tile_kernel_run_as_gemv_chunks(oracle, dev):
    """Prefill-sized m with a k no tile kernel takes (Q4_0, k % 128 != 0): the GEMV form, eight activation rows per
    launch (exact f32 accumulation of bf16 x weight)."""
    t = HQ_Q4_0
    m, n, k = 21, 96, 1056
    blocks = oracle.quantize(weights(t, n, k), k, t, threads=8)
    x = acts(5, m, k)
    xb = oracle.f32_to_bf16_bits(x)
    ref = oracle.qmatmul_f64(xb, blocks, m, n, k, t)
    y = torch.full((m, n), float("nan"), device=dev)
    p = GgmlQuantizedMatmulParams(m, n, k, t)
    assert ops.quantized_matmul_workspace_bytes(p, torch.bfloat16) == 0
    ops.quantized_matmul_ggml(torch.from_numpy(x).to(dev).to(torch.bfloat16), torch.from_numpy(blocks).to(dev), y, p)
    assert_matmul_close(y.cpu().numpy(), ref, f"m=21 t={t}")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, HQ_Q4_0])
@pytest.mark.parametrize("m,heads,hd,n", [(64, 4, 256, 96), (300, 8, 128, 160), (5, 2, 256, 64)])
def test_perm021_matches_oracle_and_the_plain_product(oracle, dev, t, m, heads, hd, n):
    """quantized_matmul_mm_tensor_perm021 (forward_prefill_batched.rs:2219-2257): activations stored
    [heads, m, head_dim]; the result is the plain product over the transposed activations, bit for bit."""
    k = heads * hd
    blocks = oracle.quantize(weights(t + m, n, k), k, t, threads=8)
    x = acts(m + hd, m, k)                                   # logical [m, k]
    xb = oracle.f32_to_bf16_bits(x)
    ref = oracle.qmatmul_f64(xb, blocks, m, n, k, t)
    xd = torch.from_numpy(x).to(dev).to(torch.bfloat16)
    x_perm = xd.view(m, heads, hd).permute(1, 0, 2).contiguous()  # [heads, m, head_dim]
    wd = torch.from_numpy(blocks).to(dev)
    y = torch.full((m, n), float("nan"), device=dev)
    ops.quantized_matmul_mm_tensor_perm021(x_perm, wd, y, ops.GgmlQuantizedMatmulPerm021Params(m, n, k, hd, t))
    check = assert_matmul_close_f16_tile if (m > 8 and _f16_tile(t, k)) else assert_matmul_close
    check(y.cpu().numpy(), ref, f"perm021 t={t} m={m}")
    y2 = torch.empty_like(y)
    ops.quantized_matmul_ggml(xd, wd, y2, GgmlQuantizedMatmulParams(m, n, k, t))
    assert torch.equal(y, y2)
    with pytest.raises(ops.HqError):  # head_dim must divide k
        ops.quantized_matmul_mm_tensor_perm021(x_perm, wd, y, ops.GgmlQuantizedMatmulPerm021Params(m, n, k, hd + 8, t))


@pytest.mark.parametrize("k", [1024, 4096])
def test_tile_gemm_with_caller_workspace_replays_from_a_hip_graph(oracle, dev, k):
    """hq_qmatmul_ggml_ws on the f16 tile route allocates nothing, so a prefill step can record it into a HIP graph:
    three replays with the activations rewritten in between, each checked against the eager call.  k = 4096 cuts k
    into four slices here (pre-pass, tiles, ordered sum: three launches, no memset node)."""
    m, n, t = 96, 384, HQ_Q4_K
    w = torch.from_numpy(oracle.quantize(weights(71, n, k), k, t, threads=8)).to(dev)
    p = GgmlQuantizedMatmulParams(m, n, k, t)
    need = ops.quantized_matmul_workspace_bytes(p, torch.bfloat16)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    x = torch.zeros(m, k, device=dev, dtype=torch.bfloat16)
    y = torch.empty(m, n, device=dev)
    ops.quantized_matmul_ggml(x, w, y, p, workspace=ws)  # warm-up outside the capture (kernel attributes are set here)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            ops.quantized_matmul_ggml(x, w, y, p, workspace=ws)
    torch.cuda.synchronize()
    for rep in range(3):
        x.copy_(torch.from_numpy(acts(80 + rep, m, k)).to(dev).to(torch.bfloat16))
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = y.clone()
        eager = torch.empty_like(y)
        ops.quantized_matmul_ggml(x, w, eager, p, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay {rep}"
        assert torch.isfinite(got).all()


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q6_K, HQ_Q8_0])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k", [(9, 64, 256), (72, 130, 1024), (300, 256, 2048), (17, 1000, 520)])
def test_f16_shadow_matmul_matches_f64_oracle(oracle, dev, t, xdt, m, n, k):
    """dispatch_mm_v2_f16's route (forward_mlx.rs:9790-9817): the weight dequantised to f16 once, then a dense product.
    Against float64 over exactly those f16 weights and the f16-rounded activations (what the product consumes), to the
    tile kernels' bound; and against the quantized-weight product of the same call, which differs by the f16 rounding
    of the weights (2^-11 relative per weight)."""
    if k % oracle.BLOCK_ELEMS[t]:
        k = k // 256 * 256
    blocks = oracle.quantize(weights(11 + m, n, k), k, t, threads=8)
    x = acts(12 + n, m, k)
    xd = torch.from_numpy(x).to(dev)
    xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
    wd = torch.from_numpy(blocks).to(dev)
    shadow = ops.dequantize_ggml(wd, n * k, t, dtype=torch.float16)
    assert torch.equal(shadow.float(), ops.dequantize_ggml(wd, n * k, t).half().float())
    ws = torch.empty(ops.matmul_f16_shadow_workspace_bytes(m, n, k), dtype=torch.uint8, device=dev)
    y = torch.full((m, n), float("nan"), device=dev)
    for _ in range(2):  # the second call reuses the remembered plan
        ops.matmul_f16_shadow(xd, shadow, y, m, n, k, ws)
    torch.cuda.synchronize()
    x16 = xd.float().half().double().cpu().numpy()
    ref = x16 @ shadow.double().cpu().numpy().reshape(n, k).T
    assert_matmul_close_f16_tile(y.cpu().numpy(), ref, f"f16 shadow t={t} {xdt} {m}x{n}x{k}")
    yq = torch.empty(m, n, device=dev)
    ops.quantized_matmul_ggml(xd, wd, yq, GgmlQuantizedMatmulParams(m, n, k, t))
    assert (y - yq).abs().max().item() <= 2e-3 * np.abs(ref).max()


def test_f16_shadow_matmul_rejects_bad_arguments(dev):
    m, n, k = 16, 32, 64
    x = torch.zeros(m, k, device=dev)
    w = torch.zeros(n, k, device=dev, dtype=torch.float16)
    y = torch.empty(m, n, device=dev)
    ws = torch.empty(ops.matmul_f16_shadow_workspace_bytes(m, n, k), dtype=torch.uint8, device=dev)
    with pytest.raises(ops.HqError):
        ops.matmul_f16_shadow(x, w, y, m, n, k, ws[:1024])       # workspace too small
    with pytest.raises(ops.HqError):
        ops.matmul_f16_shadow(x, w, y, m, n, 60, ws)             # k % 8
    with pytest.raises(ValueError):
        ops.matmul_f16_shadow(x, w.float(), y, m, n, k, ws)      # not an f16 shadow
    assert ops.matmul_f16_shadow_workspace_bytes(0, n, k) == 0


def test_dispatch_qmatmul_routes_by_rows_and_shadow(oracle, dev):
    """dispatch_qmatmul (forward_mlx.rs:9655-9969): up to 8 rows, or no shadow -> the quantized product (same bits as
    calling it); more rows over a weight with a shadow -> the f16 product (same bits as calling that)."""
    n, k, t = 192, 1024, HQ_Q4_K
    wq = ops.MlxQWeight(torch.from_numpy(oracle.quantize(weights(3, n, k), k, t, threads=8)).to(dev), t, n, k)
    assert wq.matmul_params(5) == GgmlQuantizedMatmulParams(5, n, k, t)
    for m in (1, 8, 40):
        x = torch.from_numpy(acts(m, m, k)).to(dev)
        yq = torch.empty(m, n, device=dev)
        ops.quantized_matmul_ggml(x, wq.buffer, yq, wq.matmul_params(m))
        y = torch.full((m, n), float("nan"), device=dev)
        ops.dispatch_qmatmul(x, wq, y, m)
        assert torch.equal(y, yq)
    wq.populate_f16_shadow()
    assert wq.f16_shadow.dtype == torch.float16 and wq.f16_shadow.numel() == n * k
    for m in (8, 9, 40):
        x = torch.from_numpy(acts(m, m, k)).to(dev)
        want = torch.empty(m, n, device=dev)
        if m > ops.MM_ROUTING_THRESHOLD:
            ws = torch.empty(ops.matmul_f16_shadow_workspace_bytes(m, n, k), dtype=torch.uint8, device=dev)
            ops.matmul_f16_shadow(x, wq.f16_shadow, want, m, n, k, ws)
        else:
            ops.quantized_matmul_ggml(x, wq.buffer, want, wq.matmul_params(m))
        y = torch.full((m, n), float("nan"), device=dev)
        ops.dispatch_qmatmul(x, wq, y, m)
        assert torch.equal(y, want)


@pytest.mark.gpu
@pytest.mark.parametrize("wdt", ["f16", "f32"])
@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k", [
    (1, 128, 2816),     # a router projection (Gemma 4: ffn_gate_inp f32 [2816, 128], forward_mlx.rs:9827-9830)
    (1, 2816, 704),     # an expert down projection kept as f16 (rows of 704 are not whole super-blocks, :9878-9880)
    (1, 1000, 4096),    # an lm_head slice: 512 pieces of a row, eight per lane
    (1, 70, 64),        # eight pieces per row: eight rows per wave step, ragged last step
    (3, 300, 2112),     # a few rows: one pass each
    (8, 33, 8200),      # a row of more pieces than 64 lanes x 8 in flight
    (9, 130, 704),      # one row more: the vendor library's GEMM
    (300, 257, 2112),
])
def test_dense_matmul_over_f16_and_f32_weights(dev, wdt, xdt, m, n, k):
    """dispatch_qmatmul's routes for weights that are not quantized (forward_mlx.rs:9820-9917) against numpy float64 over
    the same values: the row passes widen the weights exactly and accumulate in f32 (1e-5 of the row's magnitude); the
    GEMM over f16 weights rounds the activations to f16 first, like hq_matmul_f16_shadow; over f32 weights the vendor
    library may split f32 operands (1e-3 of the magnitude allowed, 1e-6 observed)."""
    rng = np.random.default_rng(m * 1000 + n + k)
    w32 = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    wd = torch.from_numpy(w32).to(dev)
    wd = wd.half() if wdt == "f16" else wd
    xd = torch.from_numpy(acts(m + n, m, k)).to(dev)
    xd = xd.to(torch.bfloat16) if xdt == "bf16" else xd
    y = torch.full((m, n), float("nan"), device=dev)
    for _ in range(2):
        ops.dense_matmul(xd, wd, y, m, n, k)
    torch.cuda.synchronize()
    rows = m <= 8
    assert (ops.dense_matmul_workspace_bytes(m, n, k, xd.dtype, wd.dtype) == 0) == rows
    xv = xd.float() if rows or wdt == "f32" else xd.float().half()
    ref = xv.double().cpu().numpy() @ wd.double().cpu().numpy().T
    got = y.cpu().numpy()
    assert np.isfinite(got).all()
    scale = np.sqrt((ref ** 2).mean())
    tol = 1e-5 if rows else 1e-3
    assert np.abs(got - ref).max() <= tol * max(scale, np.abs(ref).max()), (np.abs(got - ref).max(), scale)
    # the same through dispatch_qmatmul
    wq = ops.MlxQWeight(wd, ops.GGML_F16 if wdt == "f16" else ops.GGML_F32, n, k)
    y2 = torch.full((m, n), float("nan"), device=dev)
    ops.dispatch_qmatmul(xd, wq, y2, m)
    assert torch.equal(y2, y)


@pytest.mark.gpu
def test_dense_matmul_rejects_bad_arguments(dev):
    x = torch.zeros(2, 64, device=dev)
    w = torch.zeros(16, 64, device=dev)
    y = torch.empty(2, 16, device=dev)
    with pytest.raises(ops.HqError):
        ops.dense_matmul(x, w, y, 2, 16, 60)                      # k % 8
    with pytest.raises(ValueError):
        ops.dense_matmul(x, w.to(torch.bfloat16), y, 2, 16, 64)   # bf16 weights have no route here
    with pytest.raises(TypeError):
        ops.dispatch_qmatmul(x, ops.MlxQWeight(w, ops.GGML_F16, 16, 64), y, 2)  # an f32 tensor declared f16
    assert ops.dense_matmul_workspace_bytes(0, 16, 64, torch.float32, torch.float32) == 0

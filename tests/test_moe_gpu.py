"""GPU parity of the MoE glue kernels and of the whole quantized MoE FFN block against the CPU specification."""
import numpy as np
import pytest
import torch

from _util import acts, assert_matmul_close, weights
from hf2q_amd import ops
from hf2q_amd.ops import HQ_Q4_0, HQ_Q4_K, HQ_Q5_K, HQ_Q6_K, HQ_Q8_0, GgmlQuantizedMatmulParams

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,E,K", [(1, 256, 8), (8, 256, 8), (3, 4, 2), (5, 60, 4), (2, 1000, 64)])
def test_softmax_topk_matches_cpu_spec(oracle, dev, T, E, K):
    logits = (np.random.default_rng(E + K).standard_normal((T, E)) * 3).astype(np.float32)
    want_i, want_w = oracle.softmax_topk_renorm(logits, T, E, K)
    ids = torch.empty(T * K, dtype=torch.int32, device=dev)
    w = torch.empty(T * K, device=dev)
    ops.dispatch_moe_softmax_topk(torch.from_numpy(logits).to(dev), ids, w, T, E, K)
    assert np.array_equal(ids.cpu().numpy().astype(np.uint32), want_i)
    assert np.allclose(w.cpu().numpy(), want_w, rtol=1e-5, atol=1e-7)
    assert np.allclose(w.cpu().numpy().reshape(T, K).sum(1), 1.0, atol=1e-5)


def test_softmax_topk_known_answers_and_ties(dev):
    # gpu_ffn.rs:3577-3593 style: logits [1,2,3,4], top-2 -> experts 3, 2
    ids = torch.empty(2, dtype=torch.int32, device=dev)
    w = torch.empty(2, device=dev)
    ops.dispatch_moe_softmax_topk(torch.tensor([[1., 2., 3., 4.]], device=dev), ids, w, 1, 4, 2)
    assert ids.tolist() == [3, 2]
    e = np.exp(np.float64([4, 3]) - 4)
    assert np.allclose(w.cpu().numpy(), e / e.sum(), rtol=1e-6)
    # equal probabilities keep ascending expert order, like a stable sort
    ops.dispatch_moe_softmax_topk(torch.tensor([[0., 5., 5., 5., 1.]], device=dev), ids, w, 1, 5, 2)
    assert ids.tolist() == [1, 2] and np.allclose(w.cpu().numpy(), [0.5, 0.5])
    with pytest.raises(ops.HqError):   # ffn.rs:203: top-k cannot exceed num_experts
        ops.dispatch_moe_softmax_topk(torch.zeros(1, 4, device=dev), ids, w, 1, 4, 5)


def test_silu_mul_known_values(dev):
    # gpu_ffn.rs:3558-3574
    g = torch.tensor([0.0, 1.0, -1.0, 2.0], device=dev)
    u = torch.tensor([5.0, 2.0, 2.0, 0.5], device=dev)
    out = torch.empty(4, device=dev)
    ops.dispatch_silu_mul(g, u, out)
    want = [0.0, 0.7310586 * 2, -0.26894143 * 2, 2 / (1 + np.exp(-2.0)) * 0.5]
    assert np.allclose(out.cpu().numpy(), want, rtol=1e-6, atol=1e-7)


def test_weighted_reduce_and_shared_gate_linearity(dev):
    T, K, H = 3, 4, 64
    g = torch.Generator(device="cpu").manual_seed(1)
    y, w = torch.randn(T * K, H, generator=g), torch.rand(T * K, generator=g)
    sh, lg, res = torch.randn(T, H, generator=g), torch.randn(T, generator=g), torch.randn(T, H, generator=g)
    out = torch.empty(T, H, device=dev)
    ops.dispatch_moe_weighted_reduce(y.to(dev), w.to(dev), out, T, K, H, sh.to(dev), lg.to(dev), res.to(dev))
    want = (y.view(T, K, H) * w.view(T, K, 1)).sum(1) + torch.sigmoid(lg)[:, None] * sh + res
    assert torch.allclose(out.cpu(), want, rtol=1e-5, atol=1e-6)
    # gpu_ffn.rs:3493-3551: with a zero logit the shared expert enters with weight exactly 1/2
    ops.dispatch_moe_weighted_reduce(y.to(dev), w.to(dev), out, T, K, H, sh.to(dev), torch.zeros(T, device=dev))
    assert torch.allclose(out.cpu(), (y.view(T, K, H) * w.view(T, K, 1)).sum(1) + 0.5 * sh, rtol=1e-5, atol=1e-6)
    ops.dispatch_moe_weighted_reduce(y.to(dev), w.to(dev), out, T, K, H)
    assert torch.allclose(out.cpu(), (y.view(T, K, H) * w.view(T, K, 1)).sum(1), rtol=1e-5, atol=1e-6)


def test_dense_gemv_bf16(oracle, dev):
    m, n, k = 3, 70, 2048
    w = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(weights(1, n, k, 0.05)))
    x = acts(2, m, k)
    wd = torch.from_numpy(w).to(dev).to(torch.bfloat16)
    for xd, xr in ((torch.from_numpy(x).to(dev), x),
                   (torch.from_numpy(x).to(dev).to(torch.bfloat16), oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(x)))):
        y = torch.empty(m, n, device=dev)
        ops.dense_gemv_bf16_f32(xd, wd, y, m, n, k)
        ref = xr.astype(np.float64) @ w.astype(np.float64).T
        assert np.abs(y.cpu().numpy() - ref).max() <= 1e-5 * np.abs(ref).max()


@pytest.mark.parametrize("m,n,k", [(2048, 256, 2048), (100, 70, 528), (33, 1, 2048), (32, 33, 16)])
def test_dense_bf16_product_of_many_rows(oracle, dev, m, n, k):
    """The router of a prefill chunk: many bf16 activation rows take the matrix-core form (exact products, f32 sums),
    edges in every dimension; the pair form gives the same bits as two calls; f32 activations keep the GEMV form."""
    w = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(weights(3 + n, n, k, 0.05)))
    xb = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(acts(4 + m, m, k)))
    wd = torch.from_numpy(w).to(dev).to(torch.bfloat16)
    xd = torch.from_numpy(xb).to(dev).to(torch.bfloat16)
    y = torch.full((m, n), float("nan"), device=dev)
    ops.dense_gemv_bf16_f32(xd, wd, y, m, n, k)
    ref = xb.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(y.cpu().numpy() - ref).max() <= 1e-5 * np.abs(ref).max()
    yf = torch.empty(m, n, device=dev)
    ops.dense_gemv_bf16_f32(torch.from_numpy(xb).to(dev), wd, yf, m, n, k)  # the same values as f32
    assert (y - yf).abs().max().item() <= 2e-5 * np.abs(ref).max()
    # f32 activations that are no bf16 values: split into three bf16 terms, the products stay exact
    xf = acts(5 + m, m, k)
    xf[0, :4] = [np.inf, -3.0e38, 1e-40, 0.0]
    ops.dense_gemv_bf16_f32(torch.from_numpy(xf).to(dev), wd, yf, m, n, k)
    with np.errstate(invalid="ignore", over="ignore"):
        reff = xf.astype(np.float64) @ w.astype(np.float64).T
    got = yf.cpu().numpy()
    assert np.abs(got[1:] - reff[1:]).max() <= 1e-5 * np.abs(reff[1:]).max()
    fin = np.isfinite(reff[0]) & (np.abs(reff[0]) < 3e38)
    assert np.array_equal(np.isinf(got[0]), np.isinf(reff[0]) | ~fin) or np.isinf(got[0]).all()
    w2 = torch.from_numpy(oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(weights(9, 1, k, 0.05)))).to(dev).to(torch.bfloat16)
    ya, yb = torch.empty(m, n, device=dev), torch.empty(m, 1, device=dev)
    ops.dense_gemv_bf16_f32_pair(xd, wd, ya, n, w2, yb, 1, m, k)
    y1 = torch.empty(m, 1, device=dev)
    ops.dense_gemv_bf16_f32(xd, w2, y1, m, 1, k)
    assert torch.equal(ya, y) and torch.equal(yb, y1)


@pytest.mark.parametrize("T", [1, 8])
@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0])
def test_moe_block_matches_cpu_spec(oracle, dev, T, t):
    """moe_ffn_cpu_ref (ffn.rs:179-336) over the dequantised weights vs the device block."""
    H, E, K, I, SI = 512, 16, 4, 256, 256
    rng = np.random.default_rng(100 + T)
    bf = lambda a: oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(a))  # noqa: E731
    router = bf((rng.standard_normal((E, H)) * 0.1).astype(np.float32))
    sgl = bf((rng.standard_normal((1, H)) * 0.05).astype(np.float32))
    raw = {nm: weights(seed, n, k, 0.05) for nm, seed, n, k in
           (("eg", 1, E * I, H), ("eu", 2, E * I, H), ("ed", 3, E * H, I), ("sg", 4, SI, H), ("su", 5, SI, H), ("sd", 6, H, SI))}
    q = {nm: oracle.quantize(a, a.shape[1], t, threads=8) for nm, a in raw.items()}
    dq = {nm: oracle.dequantize(q[nm], t).reshape(raw[nm].shape) for nm in raw}
    x = acts(7, T, H)
    want = oracle.moe_ffn(x, H, E, K, I, SI, router, dq["eg"], dq["eu"], dq["ed"], sgl[0], dq["sg"], dq["su"], dq["sd"])

    dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    w = ops.MoeFfnWeightsGpuQ(dv(router).to(torch.bfloat16), dv(q["eg"]), dv(q["eu"]), dv(q["ed"]),
                              dv(sgl).to(torch.bfloat16), dv(q["sg"]), dv(q["su"]), dv(q["sd"]), t, H, E, K, I, SI)
    s = ops.MoeFfnScratch(w, T, dev)
    out = torch.full((T, H), float("nan"), device=dev)
    ops.build_moe_ffn_layer_gpu_q_into(dv(x), w, s, out)
    got = out.cpu().numpy()
    scale = np.abs(want).max()
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= 2e-4 * scale, np.abs(got - want).max() / scale
    # with a residual
    res = acts(9, T, H)
    ops.build_moe_ffn_layer_gpu_q_into(dv(x), w, s, out, residual=dv(res))
    assert np.abs(out.cpu().numpy() - (want + res)).max() <= 2e-4 * np.abs(want + res).max()


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q8_0])
def test_moe_block_prefill_sized_matches_cpu_spec(oracle, dev, t):
    """A prefill-sized block (48 rows per expert): the three mul_mat_id products take the expert-sorted tile GEMM
    and the dense ones the m > 8 route, both of which round the weights once to f16; a smaller call through the
    same scratch falls back to the per-row form."""
    H, E, K, I, SI, T = 512, 8, 4, 256, 256, 96
    rng = np.random.default_rng(171)
    bf = lambda a: oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(a))  # noqa: E731
    router = bf((rng.standard_normal((E, H)) * 0.1).astype(np.float32))
    sgl = bf((rng.standard_normal((1, H)) * 0.05).astype(np.float32))
    raw = {nm: weights(seed, n, k, 0.05) for nm, seed, n, k in
           (("eg", 1, E * I, H), ("eu", 2, E * I, H), ("ed", 3, E * H, I), ("sg", 4, SI, H), ("su", 5, SI, H), ("sd", 6, H, SI))}
    q = {nm: oracle.quantize(a, a.shape[1], t, threads=8) for nm, a in raw.items()}
    dq = {nm: oracle.dequantize(q[nm], t).reshape(raw[nm].shape) for nm in raw}
    x = acts(7, T, H)
    want = oracle.moe_ffn(x, H, E, K, I, SI, router, dq["eg"], dq["eu"], dq["ed"], sgl[0], dq["sg"], dq["su"], dq["sd"])
    dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    w = ops.MoeFfnWeightsGpuQ(dv(router).to(torch.bfloat16), dv(q["eg"]), dv(q["eu"]), dv(q["ed"]),
                              dv(sgl).to(torch.bfloat16), dv(q["sg"]), dv(q["su"]), dv(q["sd"]), t, H, E, K, I, SI)
    s = ops.MoeFfnScratch(w, T, dev)
    assert s.id_mm is not None and s.id_mm.numel() > 0
    out = torch.full((T, H), float("nan"), device=dev)
    ops.build_moe_ffn_layer_gpu_q_into(dv(x), w, s, out)
    got = out.cpu().numpy()
    scale = np.abs(want).max()
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= 2e-3 * scale, np.abs(got - want).max() / scale
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    # two f16-rounded products in sequence (gate / up, then down): a few 1e-4 of the rms each
    assert np.sqrt(np.mean((got - want).astype(np.float64) ** 2)) <= 2e-3 * rms
    out12 = torch.full((12, H), float("nan"), device=dev)
    ops.build_moe_ffn_layer_gpu_q_into(dv(x[:12]), w, s, out12)
    assert np.abs(out12.cpu().numpy() - want[:12]).max() <= 2e-3 * scale
    # the weight-row scales kept from load time: the same bits, for bf16 activations too
    xb = dv(x).to(torch.bfloat16)
    plain = torch.empty_like(out)
    ops.build_moe_ffn_layer_gpu_q_into(xb, w, s, plain)
    w.prepare_prefill()
    assert w.row_scales is not None and len(w.row_scales) == 6
    for xin, ref in ((dv(x), out), (xb, plain)):
        kept = torch.full((T, H), float("nan"), device=dev)
        ops.build_moe_ffn_layer_gpu_q_into(xin, w, s, kept)
        assert torch.equal(kept, ref)


def _moe_weights(oracle, dev, t, H, E, K, I, SI, seed=0):
    rng = np.random.default_rng(300 + seed)
    bf = lambda a: oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(a))  # noqa: E731
    router = bf((rng.standard_normal((E, H)) * 0.1).astype(np.float32))
    sgl = bf((rng.standard_normal((1, H)) * 0.05).astype(np.float32))
    dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    q = {nm: dv(oracle.quantize(weights(sd + seed, n, k, 0.05), k, t, threads=8)) for nm, sd, n, k in
         (("eg", 1, E * I, H), ("eu", 2, E * I, H), ("ed", 3, E * H, I), ("sg", 4, SI, H), ("su", 5, SI, H), ("sd", 6, H, SI))}
    return ops.MoeFfnWeightsGpuQ(dv(router).to(torch.bfloat16), q["eg"], q["eu"], q["ed"], dv(sgl).to(torch.bfloat16),
                                 q["sg"], q["su"], q["sd"], t, H, E, K, I, SI)


@pytest.mark.parametrize("T", [1, 3, 8])
@pytest.mark.parametrize("t,xdt", [(HQ_Q4_K, torch.float32), (HQ_Q4_K, torch.bfloat16), (HQ_Q6_K, torch.float32),
                                   (HQ_Q8_0, torch.float32)])
def test_moe_block_batched_launches_equal_separate_dispatches(oracle, dev, T, t, xdt):
    """Five launches (batched phases, SwiGLU folded into the down projections) against the twelve
    separate dispatches: the same kernels' arithmetic in the same order, so every bit must agree.
    The routed and shared experts differ in width (inter 256 / shared 512), so the jobs of one
    launch differ in n and in k."""
    H, E, K, I, SI = 512, 16, 4, 256, 512
    w = _moe_weights(oracle, dev, t, H, E, K, I, SI, seed=T)
    x = torch.from_numpy(acts(11 + T, T, H)).to(dev).to(xdt)
    res = torch.from_numpy(acts(12, T, H)).to(dev)
    outs = []
    # separate dispatches; batched with the softmax / top-k as its own launch; batched with the routing worked out
    # inside the gate / up launch (four launches)
    for batched, route_in_launch in ((False, False), (True, False), (True, True)):
        s = ops.MoeFfnScratch(w, T, dev)
        s.ids.fill_(-1)
        s.topk_w.fill_(float("nan"))
        out = torch.full((T, H), float("nan"), device=dev)
        ops.build_moe_ffn_layer_gpu_q_into(x, w, s, out, residual=res, batched=batched, route_in_launch=route_in_launch)
        outs.append((out.cpu(), s.gate.cpu(), s.up.cpu(), s.sh_gate.cpu(), s.sh_up.cpu(), s.down.cpu(), s.sh_down.cpu(),
                     s.logits.cpu(), s.sh_logit.cpu(), s.ids.cpu(), s.topk_w.cpu()))
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert torch.equal(a, b)
    assert torch.isfinite(outs[2][0]).all()


def test_batched_block_refuses_prefill_sized_token_counts(oracle, dev):
    H, E, K, I, SI = 256, 4, 2, 256, 256
    w = _moe_weights(oracle, dev, HQ_Q4_K, H, E, K, I, SI)
    s = ops.MoeFfnScratch(w, 9, dev)
    x, out = torch.zeros(9, H, device=dev), torch.empty(9, H, device=dev)
    with pytest.raises(ValueError):
        ops.build_moe_ffn_layer_gpu_q_into(x, w, s, out, batched=True)
    ops.build_moe_ffn_layer_gpu_q_into(x, w, s, out)  # default falls back to separate dispatches
    assert torch.equal(out.cpu(), torch.zeros(9, H))


def test_qmatmul_batch_swiglu_against_cpu_spec(oracle, dev):
    """down(silu(gate) * up) of one launch against the float64 product over the dequantised weights."""
    rows, n, k, t = 5, 96, 768, HQ_Q4_K
    wq = oracle.quantize(weights(21, n, k, 0.05), k, t, threads=8)
    wd = oracle.dequantize(wq, t).reshape(n, k).astype(np.float64)
    g, u = acts(22, rows, k), acts(23, rows, k)
    act = (g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64)))) * u
    y = torch.full((rows, n), float("nan"), device=dev)
    dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    ops.quantized_matmul_batch_ggml([ops.QmatmulJob(dv(g), dv(wq), y, rows, n, k, input_up=dv(u))], t)
    assert_matmul_close(y.cpu().numpy(), act @ wd.T, "swiglu-fused dense job")


def test_qmatmul_batch_argument_errors(dev):
    z = lambda *s, dt=torch.float32: torch.zeros(*s, dtype=dt, device=dev)  # noqa: E731
    w = z(144 * 8, dt=torch.uint8)
    job = ops.QmatmulJob(z(1, 256), w, z(1, 8), 1, 8, 256)
    with pytest.raises(ops.HqError):  # more jobs than one launch takes
        ops.quantized_matmul_batch_ggml([job] * 5, HQ_Q4_K)
    with pytest.raises(ops.HqError):  # dense jobs are decode-sized
        ops.quantized_matmul_batch_ggml([ops.QmatmulJob(z(9, 256), w, z(9, 8), 9, 8, 256), job], HQ_Q4_K)
    with pytest.raises(ops.HqError):  # the folded SwiGLU reads f32 activations
        ops.quantized_matmul_batch_ggml([ops.QmatmulJob(z(1, 256, dt=torch.bfloat16), w, z(1, 8), 1, 8, 256,
                                                        input_up=z(1, 256))], HQ_Q4_K)
    with pytest.raises(ops.HqError):  # expert stride smaller than one expert
        ops.quantized_matmul_batch_ggml([ops.QmatmulJob(z(1, 256), w, z(2, 8), 1, 8, 256, ids=z(2, dt=torch.int32),
                                                        top_k=2, n_experts=1, expert_stride=100), job], HQ_Q4_K)
    ops.quantized_matmul_batch_ggml([], HQ_Q4_K)


def test_dense_gemv_bf16_pair_equals_two_calls(dev):
    m, na, nb, k = 3, 37, 1, 1024
    g = torch.Generator(device="cpu").manual_seed(5)
    x = torch.randn(m, k, generator=g).to(dev)
    wa = (torch.randn(na, k, generator=g) * 0.05).to(dev).to(torch.bfloat16)
    wb = (torch.randn(nb, k, generator=g) * 0.05).to(dev).to(torch.bfloat16)
    ya, yb, ya2, yb2 = (torch.empty(m, n, device=dev) for n in (na, nb, na, nb))
    ops.dense_gemv_bf16_f32(x, wa, ya, m, na, k)
    ops.dense_gemv_bf16_f32(x, wb, yb, m, nb, k)
    ops.dense_gemv_bf16_f32_pair(x, wa, ya2, na, wb, yb2, nb, m, k)
    assert torch.equal(ya.cpu(), ya2.cpu()) and torch.equal(yb.cpu(), yb2.cpu())


@pytest.mark.parametrize("m", [1, 4])
@pytest.mark.parametrize("t,xdt", [(HQ_Q4_K, torch.bfloat16), (HQ_Q4_K, torch.float32), (HQ_Q6_K, torch.bfloat16)])
def test_dense_ffn_batched_equals_separate_dispatches_and_cpu_spec(oracle, dev, m, t, xdt):
    """dense_swiglu (ffn.rs:91-112) over the dequantised weights; two launches against four: gate and up bit for bit, the
    output to rounding (the down rows are five super-blocks long: as a call of its own the down GEMV takes the flat walk,
    inside the batched launch the kernel of 4-wave workgroups, which add a row's parts in another order)."""
    H, I = 512, 1280
    raw = {"g": weights(31, I, H, 0.05), "u": weights(32, I, H, 0.05), "d": weights(33, H, I, 0.05)}
    q = {k_: oracle.quantize(v, v.shape[1], t, threads=8) for k_, v in raw.items()}
    dq = {k_: oracle.dequantize(q[k_], t).reshape(raw[k_].shape).astype(np.float64) for k_ in raw}
    dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    w = ops.DenseFfnWeightsGpuQ(dv(q["g"]), dv(q["u"]), dv(q["d"]), t, H, I)
    x = dv(acts(34 + m, m, H)).to(xdt)
    outs = []
    for batched in (False, True):
        g, u, a = (torch.full((m, I), float("nan"), device=dev) for _ in range(3))
        out = torch.full((m, H), float("nan"), device=dev)
        ops.build_dense_ffn_layer_gpu_q_into(x, w, g, u, a, out, batched=batched)
        outs.append((out.cpu(), g.cpu(), u.cpu()))
    assert torch.equal(outs[0][1], outs[1][1]) and torch.equal(outs[0][2], outs[1][2])
    # (one row: another order of the same exact products; four rows: the separate down product runs on the matrix cores, its f32
    # activations as bf16 hi + lo parts)
    assert (outs[0][0] - outs[1][0]).abs().max().item() <= (2e-6 if m == 1 else 1e-4) * outs[0][0].abs().max().item()
    xr = x.float().cpu().numpy().astype(np.float64)
    gate, up = xr @ dq["g"].T, xr @ dq["u"].T
    want = (gate / (1 + np.exp(-gate)) * up) @ dq["d"].T
    assert_matmul_close(outs[1][0].numpy(), want, "dense FFN")


@pytest.mark.parametrize("t", [HQ_Q4_K, HQ_Q6_K])
def test_dense_ffn_prefill_with_workspace_equals_the_allocating_calls(oracle, dev, t):
    """A prefill-sized dense FFN with caller scratch (gate, up with the gating in its epilogue, down; nothing
    allocated) gives the bits of the four separate dispatches."""
    H, I, m = 512, 1024, 300
    dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    w = ops.DenseFfnWeightsGpuQ(dv(oracle.quantize(weights(1, I, H, 0.05), H, t, threads=8)),
                                dv(oracle.quantize(weights(2, I, H, 0.05), H, t, threads=8)),
                                dv(oracle.quantize(weights(3, H, I, 0.05), I, t, threads=8)), t, H, I)
    x = dv(acts(4, m, H)).to(torch.bfloat16)
    bufs = [torch.empty(m, I, device=dev) for _ in range(3)]
    out0, out1 = torch.empty(m, H, device=dev), torch.full((m, H), float("nan"), device=dev)
    ops.build_dense_ffn_layer_gpu_q_into(x, w, *bufs, out0)
    need = ops.dense_ffn_workspace_bytes(w, m, torch.bfloat16)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    bufs2 = [torch.full((m, I), float("nan"), device=dev) for _ in range(3)]
    ops.build_dense_ffn_layer_gpu_q_into(x, w, *bufs2, out1, workspace=ws)
    assert torch.equal(out0, out1) and torch.equal(bufs[2], bufs2[2])


@pytest.mark.parametrize("T", [1, 2, 5, 8])
@pytest.mark.parametrize("t,td", [(HQ_Q4_K, HQ_Q4_K), (HQ_Q5_K, HQ_Q6_K), (HQ_Q6_K, HQ_Q6_K), (HQ_Q5_K, HQ_Q5_K), (HQ_Q4_K, HQ_Q6_K)])
def test_moe_block_one_launch_equals_batched_dispatches_and_cpu_spec(oracle, dev, T, t, td):
    """hq_moe_ffn_decode (the whole block in one launch, workgroups handing results to each other through the
    scratch) at the Qwen3.6-35B-A3B expert shape, fewer experts: the bits of the batched dispatches, the CPU
    specification within the block's tolerance, and the same answer on repeated calls over one scratch (the call
    counter in the scratch tells fresh hand-overs from the previous call's)."""
    H, E, K, I, SI = 2048, 24, 8, 512, 512
    rng = np.random.default_rng(500 + T)
    bf = lambda a: oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(a))  # noqa: E731
    router = bf((rng.standard_normal((E, H)) * 0.1).astype(np.float32))
    sgl = bf((rng.standard_normal((1, H)) * 0.05).astype(np.float32))
    raw = {nm: weights(seed + T, n, k, 0.05) for nm, seed, n, k in
           (("eg", 31, E * I, H), ("eu", 32, E * I, H), ("ed", 33, E * H, I), ("sg", 34, SI, H), ("su", 35, SI, H), ("sd", 36, H, SI))}
    ty = {nm: (td if nm in ("ed", "sd") else t) for nm in raw}  # Q5_K / Q6_K is the reference model's own mix
    q = {nm: oracle.quantize(a, a.shape[1], ty[nm], threads=8) for nm, a in raw.items()}
    dq = {nm: oracle.dequantize(q[nm], ty[nm], threads=8).reshape(raw[nm].shape) for nm in raw}
    xb = bf(acts(37 + T, T, H))
    res = acts(38, T, H)
    want = oracle.moe_ffn(xb, H, E, K, I, SI, router, dq["eg"], dq["eu"], dq["ed"], sgl[0], dq["sg"], dq["su"], dq["sd"]) + res

    dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    w = ops.MoeFfnWeightsGpuQ(dv(router).to(torch.bfloat16), dv(q["eg"]), dv(q["eu"]), dv(q["ed"]),
                              dv(sgl).to(torch.bfloat16), dv(q["sg"]), dv(q["su"]), dv(q["sd"]), t, H, E, K, I, SI,
                              down_type=None if td == t else td)
    x = dv(xb).to(torch.bfloat16)
    assert ops.moe_ffn_decode_fused_supported(x, w)
    s = ops.MoeFfnScratch(w, T, dev)
    ref = torch.full((T, H), float("nan"), device=dev)
    ops.build_moe_ffn_layer_gpu_q_into(x, w, s, ref, residual=dv(res), batched=True)
    ids_ref, w_ref = s.ids.clone(), s.topk_w.clone()
    for call in range(3):
        s.ids.fill_(-1)
        s.topk_w.fill_(float("nan"))
        out = torch.full((T, H), float("nan"), device=dev)
        ops.build_moe_ffn_layer_gpu_q_into(x, w, s, out, residual=dv(res))  # default: the one-launch form
        torch.cuda.synchronize()
        assert int(s.fused[4:8].view(torch.int32).item()) == 0, "a wait inside the launch ran out"
        assert int(s.fused[0:4].view(torch.int32).item()) == call + 1
        assert torch.equal(s.ids, ids_ref) and torch.equal(s.topk_w, w_ref)
        assert torch.equal(out, ref), f"call {call}: max diff {(out - ref).abs().max().item()}"
    got = out.cpu().numpy()
    assert np.abs(got - want).max() <= 2e-4 * np.abs(want).max(), np.abs(got - want).max() / np.abs(want).max()


@pytest.mark.parametrize("T", [9, 20, 48])
def test_moe_block_of_up_to_48_tokens_runs_as_one_launch_per_eight(oracle, dev, T):
    """9 .. 48 tokens: the block is the one-launch form over eight tokens at a time, sharing one scratch -- the bits of
    separate calls over the chunks, the routing of every token written out, the separate dispatches within tolerance;
    49 tokens take the separate dispatches."""
    H, E, K, I, SI = 2048, 24, 8, 512, 512
    w = _moe_weights(oracle, dev, HQ_Q4_K, H, E, K, I, SI, seed=T)
    x = torch.from_numpy(acts(3 + T, T, H)).to(dev).to(torch.bfloat16)
    res = torch.from_numpy(acts(4 + T, T, H)).to(dev)
    assert ops.moe_ffn_decode_fused_supported(x, w)
    assert not ops.moe_ffn_decode_fused_supported(torch.zeros(49, H, device=dev, dtype=torch.bfloat16), w)
    s = ops.MoeFfnScratch(w, T, dev)
    s.ids.fill_(-1)
    out = torch.full((T, H), float("nan"), device=dev)
    ops.build_moe_ffn_layer_gpu_q_into(x, w, s, out, residual=res)
    torch.cuda.synchronize()
    assert int(s.fused[0:4].view(torch.int32).item()) == (T + 7) // 8, "one launch per eight tokens"
    assert int(s.fused[4:8].view(torch.int32).item()) == 0
    ids_all = s.ids.clone()
    assert (ids_all >= 0).all() and (ids_all < E).all()
    s8 = ops.MoeFfnScratch(w, 8, dev)
    for t0 in range(0, T, 8):
        t1 = min(T, t0 + 8)
        part = torch.full((t1 - t0, H), float("nan"), device=dev)
        ops.build_moe_ffn_layer_gpu_q_into(x[t0:t1].contiguous(), w, s8, part, residual=res[t0:t1].contiguous())
        assert torch.equal(part, out[t0:t1])
        assert torch.equal(s8.ids[: (t1 - t0) * K], ids_all[t0 * K:t1 * K])
    # the separate dispatches (other kernels, other rounding) agree within the block's tolerance
    sep = torch.empty_like(out)
    ops.build_moe_ffn_layer_gpu_q_into(x, w, s, sep, residual=res, fused=False)
    assert (sep - out).abs().max().item() <= 2e-3 * out.abs().max().item()


@pytest.mark.parametrize("T", [1, 8])
def test_moe_block_one_launch_replays_from_a_hip_graph(oracle, dev, T):
    """Three consecutive layers' worth of hq_moe_ffn_decode over ONE scratch, recorded into a HIP graph (the call
    counter in the scratch keeps counting across replays, nothing is cleared in between): four replays with the
    activations rewritten and eager calls and synchronisations in between, every replay equal to the eager result."""
    H, E, K, I, SI = 2048, 32, 8, 512, 512
    layers = [_moe_weights(oracle, dev, HQ_Q4_K, H, E, K, I, SI, seed=40 + i) for i in range(3)]
    x = torch.zeros(T, H, device=dev, dtype=torch.bfloat16)
    res = torch.from_numpy(acts(61, T, H)).to(dev)
    assert ops.moe_ffn_decode_fused_supported(x, layers[0])
    s = ops.MoeFfnScratch(layers[0], T, dev)
    outs = [torch.empty(T, H, device=dev) for _ in layers]
    for w, o in zip(layers, outs):  # warm-up outside the capture
        ops.build_moe_ffn_layer_gpu_q_into(x, w, s, o, residual=res)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            for w, o in zip(layers, outs):
                ops.build_moe_ffn_layer_gpu_q_into(x, w, s, o, residual=res)
    torch.cuda.synchronize()
    calls = int(s.fused[0:4].view(torch.int32).item())
    for rep in range(4):
        x.copy_(torch.from_numpy(acts(70 + rep, T, H)).to(dev).to(torch.bfloat16))
        for o in outs:
            o.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        calls += 3
        assert int(s.fused[0:4].view(torch.int32).item()) == calls
        assert int(s.fused[4:8].view(torch.int32).item()) == 0, "a wait inside the launch ran out"
        for i, w in enumerate(layers):  # eager: the batched dispatches (other kernels, the same bits)
            want = torch.empty(T, H, device=dev)
            ops.build_moe_ffn_layer_gpu_q_into(x, w, s, want, residual=res, batched=True)
            torch.cuda.synchronize()
            assert torch.equal(got[i], want), f"replay {rep}, layer {i}: max diff {(got[i] - want).abs().max().item()}"
        ops.build_moe_ffn_layer_gpu_q_into(x, layers[0], s, outs[0], residual=res)  # an eager one-launch call in between
        calls += 1
        torch.cuda.synchronize()


def test_moe_block_one_launch_rejects_other_shapes(oracle, dev):
    H, E, K, I, SI = 512, 16, 4, 256, 512
    w = _moe_weights(oracle, dev, HQ_Q4_K, H, E, K, I, SI)
    s = ops.MoeFfnScratch(w, 2, dev)
    assert s.fused is None
    x = torch.zeros(2, H, device=dev, dtype=torch.bfloat16)
    assert not ops.moe_ffn_decode_fused_supported(x, w)
    with pytest.raises(ops.HqError) as e:
        ops.moe_ffn_decode_fused(x, w, s, torch.empty(2, H, device=dev))
    assert e.value.status == 2


def test_moe_block_falls_back_when_the_one_launch_scratch_is_too_small(oracle, dev):
    """The default route takes the one-launch form only with a scratch of the size the library asks for; with a smaller one
    the block runs as separate dispatches (same bits), it does not raise."""
    H, E, K, I, SI, T = 2048, 32, 4, 512, 512, 2
    w = _moe_weights(oracle, dev, HQ_Q4_K, H, E, K, I, SI)
    x = torch.from_numpy(acts(5, T, H)).to(dev).to(torch.bfloat16)
    s = ops.MoeFfnScratch(w, T, dev)
    assert s.fused is not None and s.fused.numel() >= ops.moe_ffn_decode_fused_bytes(x, w) > 0
    ref = torch.empty(T, H, device=dev)
    ops.build_moe_ffn_layer_gpu_q_into(x, w, s, ref)
    s.fused = s.fused[:256]
    out = torch.full((T, H), float("nan"), device=dev)
    ops.build_moe_ffn_layer_gpu_q_into(x, w, s, out)
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    with pytest.raises(ops.HqError):
        ops.moe_ffn_decode_fused(x, w, s, out)


DENSE_DECODE_CASES = [  # (hidden, inter, gate / up type, down type)
    (4096, 12288, HQ_Q4_K, HQ_Q4_K), (2816, 4096, HQ_Q5_K, HQ_Q6_K), (2048, 8192, HQ_Q4_K, HQ_Q6_K), (1536, 8960, HQ_Q4_K, HQ_Q4_K),
    (4096, 12288, HQ_Q6_K, HQ_Q6_K), (4096, 11008, HQ_Q8_0, HQ_Q8_0), (2048, 5632, HQ_Q4_0, HQ_Q4_0), (1024, 512, HQ_Q5_K, HQ_Q5_K),
]


@pytest.mark.parametrize("xdt", ["bf16", "f32"])
@pytest.mark.parametrize("H,I,tg,td", DENSE_DECODE_CASES)
def test_dense_ffn_decode_one_launch_equals_separate_dispatches_and_cpu_spec(oracle, dev, H, I, tg, td, xdt):
    """hq_dense_ffn_decode against (a) the separate dispatches -- gate + up as one batched launch, hq_silu_mul, the down
    product over the f32 activations -- bit for bit, (b) dense_swiglu_cpu_ref (ffn.rs:91-112) over the dequantised weights
    in float64; twice in a row on one scratch (the second call must not see the first call's words as its own), with a
    residual, and replayed from a HIP graph."""
    g = torch.Generator(device=dev)
    g.manual_seed(H + I + tg)
    qz = lambda n, k, t: ops.quantize_ggml(torch.randn(n * k, generator=g, device=dev).mul_(0.02), k, t)  # noqa: E731
    w = ops.DenseFfnWeightsGpuQ(qz(I, H, tg), qz(I, H, tg), qz(H, I, td), tg, H, I, down_type=td)
    x32 = torch.randn(1, H, generator=g, device=dev)
    x = x32.to(torch.bfloat16) if xdt == "bf16" else x32
    need = ops.dense_ffn_decode_scratch_bytes(w, x.dtype)
    assert need > 0
    scratch = torch.zeros(need, dtype=torch.uint8, device=dev)
    # (a) the separate dispatches
    gate, up, act, ref = (torch.full((1, n), float("nan"), device=dev) for n in (I, I, I, H))
    ops.quantized_matmul_batch_ggml([ops.QmatmulJob(x, w.gate_q, gate, 1, I, H), ops.QmatmulJob(x, w.up_q, up, 1, I, H)], tg)
    ops.dispatch_silu_mul(gate, up, act)
    ops.quantized_matmul_ggml(act, w.down_q, ref, GgmlQuantizedMatmulParams(1, H, I, td))
    out = torch.full((1, H), float("nan"), device=dev)
    ops.dense_ffn_decode(x, w, out, scratch)
    assert torch.equal(out, ref)
    # gate + up + SwiGLU as one launch (the decode route's two-launch form): the same activations bit for bit
    pgu = GgmlQuantizedMatmulParams(1, I, H, tg)
    if ops.quantized_matmul_swiglu_decode_supported(pgu, x.dtype):
        act2 = torch.full((1, I), float("nan"), device=dev)
        ops.quantized_matmul_swiglu_decode(x, w.gate_q, w.up_q, act2, pgu)
        assert torch.equal(act2, act)
    else:
        assert I * H < 4 * 1024 * 1024  # only small matrices are left to the separate calls
    # second call on the same scratch, other activations and a residual
    x2 = (x32 * 0.5 + 0.25).to(x.dtype)
    res = torch.randn(1, H, generator=g, device=dev)
    ops.quantized_matmul_batch_ggml([ops.QmatmulJob(x2, w.gate_q, gate, 1, I, H), ops.QmatmulJob(x2, w.up_q, up, 1, I, H)], tg)
    ops.dispatch_silu_mul(gate, up, act)
    ops.quantized_matmul_ggml(act, w.down_q, ref, GgmlQuantizedMatmulParams(1, H, I, td))
    out2 = torch.full((1, H), float("nan"), device=dev)
    ops.dense_ffn_decode(x2, w, out2, scratch, residual=res)
    assert torch.equal(out2, ref + res)
    assert ops.handover_status(scratch) == 0
    # (b) the CPU specification in float64 over the dequantised weights
    deq = lambda q, n, k, t: ops.dequantize_ggml(q, n * k, t).double().view(n, k)  # noqa: E731
    xd = x.double()
    gd, ud = xd @ deq(w.gate_q, I, H, tg).T, xd @ deq(w.up_q, I, H, tg).T
    want = ((gd / (1 + torch.exp(-gd))) * ud) @ deq(w.down_q, H, I, td).T
    from _util import assert_matmul_close
    assert_matmul_close(out.cpu().numpy(), want.cpu().numpy(), f"dense ffn {H}x{I}")
    # replayed from a HIP graph, with eager work between the replays
    side = torch.cuda.Stream()
    gr = torch.cuda.CUDAGraph()
    out3 = torch.empty_like(out)
    with torch.cuda.stream(side):
        with torch.cuda.graph(gr, stream=side):
            ops.dense_ffn_decode(x, w, out3, scratch)
    for _ in range(3):
        out3.fill_(float("nan"))
        gr.replay()
        torch.cuda.synchronize()
        assert torch.equal(out3, out)
        ops.dense_ffn_decode(x2, w, out2, scratch, residual=res)
        torch.cuda.synchronize()


def test_dense_ffn_decode_rejects_what_it_does_not_take(dev):
    w = ops.DenseFfnWeightsGpuQ(None, None, None, HQ_Q6_K, 4096, 12288, down_type=HQ_Q4_K)
    assert ops.dense_ffn_decode_scratch_bytes(w, torch.bfloat16) == 0  # type mix outside the list
    w = ops.DenseFfnWeightsGpuQ(None, None, None, HQ_Q4_K, 8192, 32768)
    assert ops.dense_ffn_decode_scratch_bytes(w, torch.float32) == 0   # activations do not fit a CU's LDS
    w = ops.DenseFfnWeightsGpuQ(None, None, None, HQ_Q4_K, 4096, 12288)
    assert ops.dense_ffn_decode_scratch_bytes(w, torch.bfloat16) >= 12288 * 8


def test_hand_over_waits_give_up_at_the_spin_limit_and_report_it(oracle, dev):
    """A polling limit of zero makes every wait inside the one-launch blocks give up at once: all kernels still exit, the
    scratch's error word says so, and the next call with the default limit is right again."""
    from hf2q_amd import lib
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    H, I, t = 4096, 12288, HQ_Q4_K
    qz = lambda n, k: ops.quantize_ggml(torch.randn(n * k, generator=g, device=dev).mul_(0.02), k, t)  # noqa: E731
    w = ops.DenseFfnWeightsGpuQ(qz(I, H), qz(I, H), qz(H, I), t, H, I)
    x = torch.randn(1, H, generator=g, device=dev).to(torch.bfloat16)
    scratch = torch.zeros(ops.dense_ffn_decode_scratch_bytes(w, x.dtype), dtype=torch.uint8, device=dev)
    good, out = torch.empty(1, H, device=dev), torch.empty(1, H, device=dev)
    ops.dense_ffn_decode(x, w, good, scratch)
    assert ops.handover_status(scratch) == 0
    L = lib.load()
    try:
        L.hq_set_handover_spin_limit(1)
        for _ in range(3):
            ops.dense_ffn_decode(x, w, out, scratch)
        torch.cuda.synchronize()
        status = ops.handover_status(scratch)
    finally:
        L.hq_set_handover_spin_limit(0)
    # (with a limit of one poll a wait may still find everything in place; three launches of 256 workgroups never all do)
    assert status != 0
    scratch.zero_()  # after a reported time-out the scratch starts over
    ops.dense_ffn_decode(x, w, out, scratch)
    assert torch.equal(out, good) and ops.handover_status(scratch) == 0


def _moe_weights_mixed(oracle, dev, t, td, H, E, K, I, SI, seed=0):
    w = _moe_weights(oracle, dev, t, H, E, K, I, SI, seed=seed)
    if td != t:
        dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
        w.expert_down = dv(oracle.quantize(weights(3 + seed, E * H, I, 0.05), I, td, threads=8))
        w.shared_down = dv(oracle.quantize(weights(6 + seed, H, SI, 0.05), SI, td, threads=8))
        w.down_type = td
    return w


@pytest.mark.parametrize("T", [1, 3, 8, 9, 40, 96, 300])
@pytest.mark.parametrize("t,td,xdt", [(HQ_Q4_K, HQ_Q4_K, torch.bfloat16), (HQ_Q5_K, HQ_Q6_K, torch.float32), (HQ_Q8_0, HQ_Q8_0, torch.bfloat16)])
def test_moe_block_as_one_library_call_equals_the_dispatches_made_by_hand(oracle, dev, T, t, td, xdt):
    """hq_moe_ffn_prefill (one C call, one scratch, any token count; also the reference's real type mix: gate / up Q5_K, down
    Q6_K) against build_moe_ffn_layer_gpu_q_into's own sequence of dispatches: bit for bit, routing included; with row scales
    kept from load time as well."""
    H, E, K, I, SI = 512, 8, 4, 256, 256
    w = _moe_weights_mixed(oracle, dev, t, td, H, E, K, I, SI, seed=T)
    x = torch.from_numpy(acts(21 + T, T, H)).to(dev).to(xdt)
    res = torch.from_numpy(acts(22, T, H)).to(dev)
    s = ops.MoeFfnScratch(w, T, dev)
    want = torch.full((T, H), float("nan"), device=dev)
    ops.build_moe_ffn_layer_gpu_q_into(x, w, s, want, residual=res, fused=False)
    need = ops.moe_ffn_prefill_scratch_bytes(w, T, x.dtype)
    assert need > 0
    scratch = torch.full((need,), 0xA5, dtype=torch.uint8, device=dev)  # contents irrelevant
    got = torch.full((T, H), float("nan"), device=dev)
    ids = torch.full((T * K,), -1, dtype=torch.int32, device=dev)
    wts = torch.full((T * K,), float("nan"), device=dev)
    ops.moe_ffn_prefill(x, w, got, scratch, residual=res, route_ids=ids, route_weights=wts)
    assert torch.isfinite(got).all() and torch.equal(got, want)
    assert torch.equal(ids, s.ids[:T * K]) and torch.equal(wts, s.topk_w[:T * K])
    w.prepare_prefill()
    got2 = torch.full((T, H), float("nan"), device=dev)
    ops.moe_ffn_prefill(x, w, got2, scratch, residual=res)
    assert torch.equal(got2, want)
    # too small a scratch is refused before anything runs
    with pytest.raises(ops.HqError):
        ops.moe_ffn_prefill(x, w, got2, scratch[:need - 256], residual=res)


def test_moe_block_mixed_types_match_cpu_spec(oracle, dev):
    """gate / up Q5_K with down Q6_K (the reference model's mix, docs/ADR-028...:4942-4946) against moe_ffn_cpu_ref over the
    dequantised weights, at one token (decode dispatches) and at 96 (grouped tiles)."""
    H, E, K, I, SI = 512, 8, 4, 256, 256
    t, td = HQ_Q5_K, HQ_Q6_K
    rng = np.random.default_rng(77)
    bf = lambda a: oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(a))  # noqa: E731
    router = bf((rng.standard_normal((E, H)) * 0.1).astype(np.float32))
    sgl = bf((rng.standard_normal((1, H)) * 0.05).astype(np.float32))
    raw = {nm: (weights(seed, n, k, 0.05), ty) for nm, seed, n, k, ty in
           (("eg", 1, E * I, H, t), ("eu", 2, E * I, H, t), ("ed", 3, E * H, I, td), ("sg", 4, SI, H, t), ("su", 5, SI, H, t), ("sd", 6, H, SI, td))}
    q = {nm: oracle.quantize(a, a.shape[1], ty, threads=8) for nm, (a, ty) in raw.items()}
    dq = {nm: oracle.dequantize(q[nm], raw[nm][1]).reshape(raw[nm][0].shape) for nm in raw}
    dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    w = ops.MoeFfnWeightsGpuQ(dv(router).to(torch.bfloat16), dv(q["eg"]), dv(q["eu"]), dv(q["ed"]), dv(sgl).to(torch.bfloat16),
                              dv(q["sg"]), dv(q["su"]), dv(q["sd"]), t, H, E, K, I, SI, down_type=td)
    for T, tol in ((1, 2e-4), (96, 2e-3)):
        x = acts(7 + T, T, H)
        want = oracle.moe_ffn(x, H, E, K, I, SI, router, dq["eg"], dq["eu"], dq["ed"], sgl[0], dq["sg"], dq["su"], dq["sd"])
        scratch = torch.empty(ops.moe_ffn_prefill_scratch_bytes(w, T, torch.float32), dtype=torch.uint8, device=dev)
        out = torch.full((T, H), float("nan"), device=dev)
        ops.moe_ffn_prefill(dv(x), w, out, scratch)
        got = out.cpu().numpy()
        assert np.isfinite(got).all() and np.abs(got - want).max() <= tol * np.abs(want).max()


@pytest.mark.parametrize("m", [1, 4, 8, 9, 64, 300])
@pytest.mark.parametrize("H,I,tg,td,xdt", [(4096, 8192, HQ_Q4_K, HQ_Q4_K, torch.bfloat16), (512, 1024, HQ_Q4_K, HQ_Q6_K, torch.float32),
                                           (1024, 12288, HQ_Q8_0, HQ_Q8_0, torch.bfloat16)])
def test_dense_ffn_as_one_library_call_equals_the_dispatches_made_by_hand(oracle, dev, m, H, I, tg, td, xdt):
    """hq_dense_ffn against build_dense_ffn_layer_gpu_q_into (decode: gate + up + SwiGLU launch or batched launches; prefill:
    gate, gated up, down with a workspace): bit for bit."""
    g = torch.Generator(device=dev)
    g.manual_seed(H + I + m)
    qz = lambda n, k, t: ops.quantize_ggml(torch.randn(n * k, generator=g, device=dev).mul_(0.02), k, t)  # noqa: E731
    w = ops.DenseFfnWeightsGpuQ(qz(I, H, tg), qz(I, H, tg), qz(H, I, td), tg, H, I, down_type=td)
    x = torch.randn(m, H, generator=g, device=dev).to(xdt)
    gate, up, act = (torch.full((m, I), float("nan"), device=dev) for _ in range(3))
    want = torch.full((m, H), float("nan"), device=dev)
    nws = ops.dense_ffn_workspace_bytes(w, m, x.dtype)
    ws = torch.empty(nws, dtype=torch.uint8, device=dev) if nws else None
    ops.build_dense_ffn_layer_gpu_q_into(x, w, gate, up, act, want, workspace=ws)
    scratch = torch.full((ops.dense_ffn_scratch_bytes(w, m, x.dtype),), 0x5A, dtype=torch.uint8, device=dev)
    got = torch.full((m, H), float("nan"), device=dev)
    ops.dense_ffn(x, w, got, scratch)
    assert torch.isfinite(got).all() and torch.equal(got, want)

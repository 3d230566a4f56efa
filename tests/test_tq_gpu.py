"""GPU parity of the TurboQuant-style KV path: rotation, write-side encode, decode attention."""
import numpy as np
import pytest
import torch

from hf2q_amd import ops
from hf2q_amd.ops import FlashAttnVecTqHbParams

pytestmark = pytest.mark.gpu


def _nrmse(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.sqrt(((a - b) ** 2).sum() / (b ** 2).sum()))


@pytest.mark.parametrize("hd", [256, 512])
def test_fwht_sign_bit_exact_and_self_inverse(oracle, dev, hd):
    x = np.random.default_rng(hd).standard_normal((5, hd)).astype(np.float32)
    b = torch.from_numpy(x).to(dev)
    ops.dispatch_fwht_sign_premult_f32(b, 5, hd)
    want = oracle.fwht_sign_premult(x, 5, hd)
    assert np.array_equal(b.cpu().numpy().view(np.uint32), want.view(np.uint32))
    ops.dispatch_fwht_sign_undo_f32(b, 5, hd)
    assert np.array_equal(b.cpu().numpy().view(np.uint32), oracle.fwht_sign_undo(want, 5, hd).view(np.uint32))
    assert np.allclose(b.cpu().numpy(), x, atol=1e-5)  # undo(premult(x)) = x


def _oracle_cache(oracle, kv, n_kv, hd, cap, start=0):
    codes = np.zeros((n_kv, cap, hd), np.uint8)
    norms = np.zeros((n_kv, cap, max(1, hd // 256)), np.float32)
    for t in range(kv.shape[0]):
        oracle.tq_encode_int8(kv[t], n_kv, hd, cap, (start + t) % cap, codes, norms)
    return codes, norms


@pytest.mark.parametrize("hd", [256, 512])
def test_encode_byte_equal_to_oracle(oracle, dev, hd):
    rng = np.random.default_rng(3)
    n_kv, cap, n_tok, start = 2, 40, 37, 6   # wraps around the ring: slots 6..39, 0..2
    kv = rng.standard_normal((n_tok, n_kv, hd)).astype(np.float32)
    kv[5] = 0.0                               # an all-zero token: scale 0, codes 0
    want_c, want_n = _oracle_cache(oracle, kv, n_kv, hd, cap, start)
    codes, norms = ops.alloc_tq_kv(n_kv, cap, hd, dev)
    ops.hadamard_quantize_kv(torch.from_numpy(kv).to(dev), codes, norms, start)
    assert np.array_equal(codes.cpu().numpy(), want_c)
    assert np.array_equal(norms.cpu().numpy().view(np.uint32), want_n.view(np.uint32))
    # kv_cache.rs:4205: encoding a sequence equals encoding token by token
    c2, n2 = ops.alloc_tq_kv(n_kv, cap, hd, dev)
    for t in range(n_tok):
        ops.hadamard_quantize_kv(torch.from_numpy(kv[t:t + 1]).to(dev), c2, n2, start + t)
    assert torch.equal(c2, codes) and torch.equal(n2, norms)
    # kv_cache.rs:3383: only the written slots change
    assert not codes[:, 3:6].any() and not norms[:, 3:6].any()


def _attend(dev, q, kc, kn, vc, vn, p, lut=None):
    tmp = torch.empty(ops.tq_tmp_buffer_bytes(p.num_heads, p.head_dim, p.kv_seq_len) // 4, device=dev)
    out = torch.full((p.num_heads, p.head_dim), float("nan"), device=dev)
    ops.flash_attn_vec_tq_hb(torch.from_numpy(q).to(dev), torch.from_numpy(kc).to(dev), torch.from_numpy(kn).to(dev),
                             torch.from_numpy(vc).to(dev), torch.from_numpy(vn).to(dev), out, tmp, p,
                             None if lut is None else torch.from_numpy(lut).to(dev))
    return out.cpu().numpy()


def _assert_attn_close(got, ref, what):
    assert np.isfinite(got).all(), what
    scale = np.abs(ref).max(axis=1, keepdims=True)
    # softmax in fp32 over exact dequantised values: 1e-3 of each head's output magnitude
    assert (np.abs(got - ref) <= 1e-3 * scale).all(), f"{what}: max err {np.abs(got - ref).max()} vs scale {scale.min()}"
    assert _nrmse(got, ref) < 1e-4, f"{what}: nrmse {_nrmse(got, ref)}"


CASES = [  # nh, nkv, n, cap, kwargs
    (16, 2, 1, 8, {}),
    (16, 2, 33, 40, {}),
    (16, 2, 700, 1024, {}),
    (8, 4, 257, 300, {}),                                    # group of 2
    (4, 4, 100, 128, {}),                                    # no grouping
    (32, 2, 130, 256, {}),                                   # group of 16 = two chunks of 8
    (16, 2, 500, 512, {"mask_type": 1}),
    (16, 2, 500, 512, {"mask_type": 2, "sliding_window": 100}),
    (16, 2, 512, 512, {"mask_type": 2, "sliding_window": 300, "ring_start": 77}),
    (16, 2, 300, 512, {"softcap": 5.0}),
    (16, 2, 9000, 9000, {}),                                 # several tiles per wave
]


@pytest.mark.parametrize("nh,nkv,n,cap,kw", CASES)
def test_attention_matches_f64_oracle(oracle, dev, nh, nkv, n, cap, kw):
    hd = 256
    rng = np.random.default_rng(nh * n + cap)
    k = rng.standard_normal((min(n, cap), nkv, hd)).astype(np.float32)
    v = rng.standard_normal((min(n, cap), nkv, hd)).astype(np.float32)
    kc, kn = _oracle_cache(oracle, k, nkv, hd, cap)
    vc, vn = _oracle_cache(oracle, v, nkv, hd, cap)
    q = oracle.fwht_sign_premult(rng.standard_normal((nh, hd)).astype(np.float32), nh, hd)
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 1.0 / 16.0, **kw)
    ref = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, hd, n, cap, p.scale, p.mask_type, p.sliding_window,
                              p.softcap, p.ring_start)
    _assert_attn_close(_attend(dev, q, kc, kn, vc, vn, p), ref, f"attn {nh}/{nkv} n={n} {kw}")


def _raw_cache(rng, nkv, cap, hd, norm_lo, norm_hi, log_uniform=False):
    codes = rng.integers(-127, 128, (nkv, cap, hd)).astype(np.int8).view(np.uint8)
    if log_uniform:
        norms = np.exp(rng.uniform(np.log(norm_lo), np.log(norm_hi), (nkv, cap, hd // 256)))
    else:
        norms = rng.uniform(norm_lo, norm_hi, (nkv, cap, hd // 256))
    return codes, norms.astype(np.float32)


CASES_512 = [  # nh, nkv, n, cap, kwargs
    (16, 2, 1, 8, {}),
    (16, 2, 700, 1024, {}),
    (8, 4, 257, 300, {"softcap": 4.0}),
    (32, 2, 130, 256, {"mask_type": 1}),
    (16, 2, 512, 512, {"mask_type": 2, "sliding_window": 300, "ring_start": 77}),
    (16, 2, 5000, 5000, {}),
]


@pytest.mark.parametrize("nh,nkv,n,cap,kw", CASES_512)
def test_attention_head_dim_512(oracle, dev, nh, nkv, n, cap, kw):
    """head_dim 512 (kv_cache.rs:2010-2012): two 256-blocks per row, each with its own norm and its own rotation."""
    hd = 512
    rng = np.random.default_rng(nh * n + cap + 1)
    k = rng.standard_normal((min(n, cap), nkv, hd)).astype(np.float32)
    v = rng.standard_normal((min(n, cap), nkv, hd)).astype(np.float32)
    v[:, :, 256:] *= 7.0  # the two blocks of a row get clearly different norms
    kc, kn = _oracle_cache(oracle, k, nkv, hd, cap)
    vc, vn = _oracle_cache(oracle, v, nkv, hd, cap)
    q = oracle.fwht_sign_premult(rng.standard_normal((nh, hd)).astype(np.float32), nh, hd)
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 1.0 / 22.6, **kw)
    ref = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, hd, n, cap, p.scale, p.mask_type, p.sliding_window,
                              p.softcap, p.ring_start)
    got = _attend(dev, q, kc, kn, vc, vn, p)
    _assert_attn_close(got, ref, f"attn d512 {nh}/{nkv} n={n} {kw}")
    # the fused rotations give the bits of the three-dispatch chain here too
    qraw = rng.standard_normal((nh, hd)).astype(np.float32)
    args = [torch.from_numpy(x).to(dev) for x in (kc, kn, vc, vn)]
    tmp = torch.empty(ops.tq_tmp_buffer_bytes(nh, hd, n) // 4, device=dev)
    qd = torch.from_numpy(qraw).to(dev)
    ops.dispatch_fwht_sign_premult_f32(qd, nh, hd)
    sep = torch.empty(nh, hd, device=dev)
    ops.flash_attn_vec_tq_hb(qd, *args, sep, tmp, p)
    ops.dispatch_fwht_sign_undo_f32(sep, nh, hd)
    both = torch.full((nh, hd), float("nan"), device=dev)
    pf = FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 1.0 / 22.6, fuse_fwht_pre=1, **kw)
    ops.flash_attn_vec_tq_hb(torch.from_numpy(qraw).to(dev), *args, both, tmp, pf, undo_rotation=True)
    assert torch.equal(sep, both)


def test_attention_head_dim_512_table_form(oracle, dev):
    """The reference's D = 512 convention (table value * norm / 16 / scale_factor_d512) with 8- and 5-bit tables."""
    hd, nh, nkv, n, cap = 512, 16, 2, 200, 256
    for bits, sf in ((8, 1.0), (5, 1.4142135)):
        rng = np.random.default_rng(90 + bits)
        kc = rng.integers(0, 1 << bits, (nkv, cap, hd), dtype=np.uint8)
        vc = rng.integers(0, 1 << bits, (nkv, cap, hd), dtype=np.uint8)
        kn = rng.uniform(5, 20, (nkv, cap, 2)).astype(np.float32)
        vn = rng.uniform(5, 20, (nkv, cap, 2)).astype(np.float32)
        lut = np.zeros(256, np.float32)
        lut[: 1 << bits] = np.sort(rng.standard_normal(1 << bits)).astype(np.float32) * 2
        q = rng.standard_normal((nh, hd)).astype(np.float32)
        p = FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 1.0 / 22.6, scale_factor_d512=sf, codebook_bits=bits)
        ref = oracle.tq_attention(q, kc, kn, vc, vn, lut, nh, nkv, hd, n, cap, p.scale, scale_factor_d512=sf)
        _assert_attn_close(_attend(dev, q, kc, kn, vc, vn, p, lut), ref, f"d512 {bits}-bit table")


@pytest.mark.parametrize("case", ["q_large_mean", "q_tiny", "q_huge", "v_norm_range", "v_norm_zeros", "even_attention",
                                  "peaked", "extreme_codes"])
def test_attention_adversarial_operands(oracle, dev, case):
    """Operands that stress the kernel's internal number formats (scaled half-precision operands with a
    constant offset on the codes): a query far from zero mean, queries of very small and very large magnitude, value
    norms over many orders of magnitude or zero, evenly spread and sharply peaked attention, codes at
    the ends of their range.  Same bar as the random cases."""
    hd, nh, nkv, n, cap = 256, 16, 2, 1500, 1536
    rng = np.random.default_rng(sum(case.encode()))
    kc, kn = _raw_cache(rng, nkv, cap, hd, 0.005, 0.02)
    vc, vn = _raw_cache(rng, nkv, cap, hd, 0.005, 0.02)
    q = rng.standard_normal((nh, hd)).astype(np.float32)
    if case == "q_large_mean":
        q = (3.0 + 0.1 * q).astype(np.float32)
    elif case == "q_tiny":
        q = (q * np.logspace(-30, -3, nh)[:, None]).astype(np.float32)
    elif case == "q_huge":
        q = (q * np.float32(1e20)).astype(np.float32)
        kn = (kn * np.float32(1e-20)).astype(np.float32)
    elif case == "v_norm_range":
        vc, vn = _raw_cache(rng, nkv, cap, hd, 1e-12, 1e6, log_uniform=True)
    elif case == "v_norm_zeros":
        vn[:, ::3] = 0.0
        vn[:, 700:900] = 0.0
    elif case == "even_attention":
        q = (q * np.float32(1e-4)).astype(np.float32)
    elif case == "peaked":
        kn[:, 611] = 0.3
        q[:8] = kc[0, 611].view(np.int8).astype(np.float32) / 40
        q[8:] = kc[1, 611].view(np.int8).astype(np.float32) / 40
    elif case == "extreme_codes":
        kc = rng.choice(np.array([-128, -127, 127], np.int8), (nkv, cap, hd)).view(np.uint8)
        vc = rng.choice(np.array([-128, 127], np.int8), (nkv, cap, hd)).view(np.uint8)
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 1.0 / 16.0)
    ref = oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, hd, n, cap, p.scale)
    _assert_attn_close(_attend(dev, q, kc, kn, vc, vn, p), ref, case)


def test_attention_lut_form(oracle, dev):
    hd, nh, nkv, n, cap = 256, 16, 2, 200, 256
    rng = np.random.default_rng(8)
    kc = rng.integers(0, 256, (nkv, cap, hd), dtype=np.uint8)
    vc = rng.integers(0, 256, (nkv, cap, hd), dtype=np.uint8)
    kn = rng.uniform(5, 20, (nkv, cap, 1)).astype(np.float32)
    vn = rng.uniform(5, 20, (nkv, cap, 1)).astype(np.float32)
    lut = np.sort(rng.standard_normal(256)).astype(np.float32) * 2  # an arbitrary (non-linear) 256-entry codebook
    q = rng.standard_normal((nh, hd)).astype(np.float32)
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 1.0 / 16.0)
    ref = oracle.tq_attention(q, kc, kn, vc, vn, lut, nh, nkv, hd, n, cap, p.scale)
    _assert_attn_close(_attend(dev, q, kc, kn, vc, vn, p, lut), ref, "lut form")


@pytest.mark.parametrize("bits", [5, 6])
def test_attention_small_codebooks(oracle, dev, bits):
    """5- and 6-bit caches: one code per byte below 2^bits, values from the caller's centroid table."""
    hd, nh, nkv, n, cap = 256, 8, 2, 150, 160
    rng = np.random.default_rng(80 + bits)
    kc = rng.integers(0, 1 << bits, (nkv, cap, hd), dtype=np.uint8)
    vc = rng.integers(0, 1 << bits, (nkv, cap, hd), dtype=np.uint8)
    kn = rng.uniform(5, 20, (nkv, cap, 1)).astype(np.float32)
    vn = rng.uniform(5, 20, (nkv, cap, 1)).astype(np.float32)
    lut = np.zeros(256, np.float32)
    lut[: 1 << bits] = np.sort(rng.standard_normal(1 << bits)).astype(np.float32) * 2
    q = rng.standard_normal((nh, hd)).astype(np.float32)
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 1.0 / 16.0, codebook_bits=bits)
    ref = oracle.tq_attention(q, kc, kn, vc, vn, lut, nh, nkv, hd, n, cap, p.scale)
    _assert_attn_close(_attend(dev, q, kc, kn, vc, vn, p, lut), ref, f"{bits}-bit codebook")


def test_fused_pre_rotation_equals_separate_dispatch(oracle, dev):
    hd, nh, nkv, n, cap = 256, 16, 2, 300, 512
    rng = np.random.default_rng(12)
    kc, kn = _oracle_cache(oracle, rng.standard_normal((n, nkv, hd)).astype(np.float32), nkv, hd, cap)
    vc, vn = _oracle_cache(oracle, rng.standard_normal((n, nkv, hd)).astype(np.float32), nkv, hd, cap)
    q = rng.standard_normal((nh, hd)).astype(np.float32)
    sep = _attend(dev, oracle.fwht_sign_premult(q, nh, hd), kc, kn, vc, vn, FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 0.0625))
    fused = _attend(dev, q, kc, kn, vc, vn, FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 0.0625, fuse_fwht_pre=1))
    assert np.array_equal(sep, fused)  # forward_mlx.rs:4646-4652: the fused path is bit-identical


def test_one_call_attention_chain_replays_from_a_hip_graph(oracle, dev):
    """The decode step's attention (split with the query rotation inside, merge with the output rotation inside: two
    launches, caller-owned tmp, no allocation) recorded into a HIP graph: four replays with the query rewritten and an
    eager call in between, every replay equal to the eager result."""
    hd, nh, nkv, n, cap = 256, 16, 2, 3000, 4096
    rng = np.random.default_rng(77)
    kc, kn = _oracle_cache(oracle, rng.standard_normal((n, nkv, hd)).astype(np.float32), nkv, hd, cap)
    vc, vn = _oracle_cache(oracle, rng.standard_normal((n, nkv, hd)).astype(np.float32), nkv, hd, cap)
    dv = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    kc, kn, vc, vn = dv(kc), dv(kn), dv(vc), dv(vn)
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 0.0625, fuse_fwht_pre=1)
    q = torch.zeros(nh, hd, device=dev)
    out = torch.empty(nh, hd, device=dev)
    tmp = torch.empty(ops.tq_tmp_buffer_bytes(nh, hd, n) // 4, device=dev)
    ops.flash_attn_vec_tq_hb(q, kc, kn, vc, vn, out, tmp, p, undo_rotation=True)  # warm-up outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            ops.flash_attn_vec_tq_hb(q, kc, kn, vc, vn, out, tmp, p, undo_rotation=True)
    torch.cuda.synchronize()
    for rep in range(4):
        q.copy_(dv(rng.standard_normal((nh, hd)).astype(np.float32)))
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = torch.empty_like(out)
        ops.flash_attn_vec_tq_hb(q, kc, kn, vc, vn, want, tmp, p, undo_rotation=True)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {rep}"
        assert torch.isfinite(got).all()


@pytest.mark.parametrize("n,cap,kw", [(300, 512, {}), (5000, 5000, {}), (512, 512, {"mask_type": 2, "sliding_window": 200, "ring_start": 31})])
def test_fused_post_rotation_equals_separate_dispatch(oracle, dev, n, cap, kw):
    """Attention whose merge pass applies the inverse rotation gives the bits of attention followed by
    dispatch_fwht_sign_undo_f32; with the fused pre-rotation as well, the bits of the three-dispatch chain."""
    hd, nh, nkv = 256, 16, 2
    rng = np.random.default_rng(n)
    m = min(n, cap)
    kc, kn = _oracle_cache(oracle, rng.standard_normal((m, nkv, hd)).astype(np.float32), nkv, hd, cap)
    vc, vn = _oracle_cache(oracle, rng.standard_normal((m, nkv, hd)).astype(np.float32), nkv, hd, cap)
    q = rng.standard_normal((nh, hd)).astype(np.float32)
    args = [torch.from_numpy(x).to(dev) for x in (kc, kn, vc, vn)]
    tmp = torch.empty(ops.tq_tmp_buffer_bytes(nh, hd, n) // 4, device=dev)

    qd = torch.from_numpy(q).to(dev)
    ops.dispatch_fwht_sign_premult_f32(qd, nh, hd)
    sep = torch.empty(nh, hd, device=dev)
    ops.flash_attn_vec_tq_hb(qd, *args, sep, tmp, FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 0.0625, **kw))
    ops.dispatch_fwht_sign_undo_f32(sep, nh, hd)

    post = torch.full((nh, hd), float("nan"), device=dev)
    ops.flash_attn_vec_tq_hb(qd, *args, post, tmp, FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 0.0625, **kw), undo_rotation=True)
    assert torch.equal(sep, post)
    both = torch.full((nh, hd), float("nan"), device=dev)
    ops.flash_attn_vec_tq_hb(torch.from_numpy(q).to(dev), *args, both, tmp,
                             FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 0.0625, fuse_fwht_pre=1, **kw), undo_rotation=True)
    assert torch.equal(sep, both)


def test_end_to_end_against_unquantised_attention(oracle, dev):
    """The reference's litmus (kv_cache.rs:3959-4117): rotate q, attend over the 8-bit cache, rotate back, compare
    with plain f32 attention.  kv_seq_len = 1 must return V[h / heads_per_kv]; gate NRMSE < 0.15."""
    hd, nh, nkv, cap = 256, 16, 2, 64
    rng = np.random.default_rng(21)
    for n in (1, 48):
        k = rng.standard_normal((n, nkv, hd)).astype(np.float32)
        v = rng.standard_normal((n, nkv, hd)).astype(np.float32)
        q = rng.standard_normal((nh, hd)).astype(np.float32)
        kcod, knrm = ops.alloc_tq_kv(nkv, cap, hd, dev)
        vcod, vnrm = ops.alloc_tq_kv(nkv, cap, hd, dev)
        ops.hadamard_quantize_kv(torch.from_numpy(k).to(dev), kcod, knrm, 0)
        ops.hadamard_quantize_kv(torch.from_numpy(v).to(dev), vcod, vnrm, 0)
        qd = torch.from_numpy(q).to(dev)
        ops.dispatch_fwht_sign_premult_f32(qd, nh, hd)
        out = torch.empty(nh, hd, device=dev)
        tmp = torch.empty(ops.tq_tmp_buffer_bytes(nh, hd, n) // 4, device=dev)
        ops.flash_attn_vec_tq_hb(qd, kcod, knrm, vcod, vnrm, out, tmp, FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 0.0625))
        ops.dispatch_fwht_sign_undo_f32(out, nh, hd)
        exact = np.zeros((nh, hd))
        for h in range(nh):
            s = (k[:, h // 8].astype(np.float64) @ q[h].astype(np.float64)) * 0.0625
            pr = np.exp(s - s.max())
            pr /= pr.sum()
            exact[h] = pr @ v[:, h // 8].astype(np.float64)
        e = _nrmse(out.cpu().numpy(), exact)
        assert e < 0.15 and e < 0.02, f"n={n}: nrmse {e}"


@pytest.mark.parametrize("hd", [256, 512])
@pytest.mark.parametrize("unrotate", [False, True])
def test_bulk_dequantize_bit_exact(oracle, dev, hd, unrotate):
    """dequant_seq_to_temp_f32[_unrotated] (kv_cache.rs:431-583): a range of cache positions back to f32,
    head-major; every element is one rounding of norm * code, the rotation is the bit-exact FWHT."""
    rng = np.random.default_rng(hd + unrotate)
    nkv, cap, start, n = 3, 50, 7, 41
    codes = rng.integers(0, 256, (nkv, cap, hd), dtype=np.uint8)
    norms = rng.uniform(1e-3, 3.0, (nkv, cap, hd // 256)).astype(np.float32)
    want = oracle.tq_dequantize(codes, norms, None, nkv, hd, cap, start, n, unrotate=unrotate)
    dst = torch.full((nkv, n, hd), float("nan"), device=dev)
    ops.tq_dequantize_hb_kv_seq(torch.from_numpy(codes).to(dev), torch.from_numpy(norms).to(dev), dst, nkv, hd, cap, start, n,
                                unrotate=unrotate)
    assert np.array_equal(dst.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # table form: lut[code] * norm / 16 (/ scale_factor_d512 at 512)
    lut = (np.sort(rng.standard_normal(256)) * 2).astype(np.float32)
    want = oracle.tq_dequantize(codes, norms, lut, nkv, hd, cap, start, n, unrotate=unrotate)
    ops.tq_dequantize_hb_kv_seq(torch.from_numpy(codes).to(dev), torch.from_numpy(norms).to(dev), dst, nkv, hd, cap, start, n,
                                lut256=torch.from_numpy(lut).to(dev), unrotate=unrotate)
    assert np.array_equal(dst.cpu().numpy().view(np.uint32), want.view(np.uint32))
    if hd == 512 and not unrotate:  # a scale factor that is no power of two: two roundings instead of one
        want = oracle.tq_dequantize(codes, norms, lut, nkv, hd, cap, start, n, scale_factor_d512=1.3)
        ops.tq_dequantize_hb_kv_seq(torch.from_numpy(codes).to(dev), torch.from_numpy(norms).to(dev), dst, nkv, hd, cap,
                                    start, n, scale_factor_d512=1.3, lut256=torch.from_numpy(lut).to(dev))
        assert np.allclose(dst.cpu().numpy(), want, rtol=3e-7, atol=0)


def test_encode_then_bulk_dequantize_recovers_the_input(dev):
    """The reference's round-trip gate (kv_cache.rs:497-520, NRMSE threshold 0.15 at production cache shape):
    encode a sequence, dequantise it un-rotated, compare with the f32 input."""
    nkv, hd, cap, n, start = 2, 256, 4096, 1000, 100
    gen = torch.Generator(device=dev)
    gen.manual_seed(4)
    kv = torch.randn(n, nkv, hd, generator=gen, device=dev)
    codes, norms = ops.alloc_tq_kv(nkv, cap, hd, dev)
    ops.hadamard_quantize_kv(kv, codes, norms, start)
    dst = torch.empty(nkv, n, hd, device=dev)
    ops.tq_dequantize_hb_kv_seq(codes, norms, dst, nkv, hd, cap, start, n, unrotate=True)
    e = _nrmse(dst.permute(1, 0, 2).cpu().numpy(), kv.cpu().numpy())
    assert e < 0.15 and e < 0.01, e
    with pytest.raises(ops.HqError) as err:  # kv_cache.rs:427-428
        ops.tq_dequantize_hb_kv_seq(codes, norms, dst, nkv, hd, cap, cap - 10, 11)
    assert err.value.status == 1


@pytest.mark.parametrize("hd", [256, 512])
def test_capture_and_restore_of_a_token_range(dev, hd):
    """Cache positions -> version-2 envelope in host memory -> another cache: indices and norms byte-equal, the
    envelope parses with the oracle's parser, positions outside the range are untouched."""
    from oracle import tqp
    nkv, cap, start, n = 3, 64, 9, 40
    gen = torch.Generator(device=dev)
    gen.manual_seed(hd)
    codes, norms = ops.alloc_tq_kv(nkv, cap, hd, dev)
    ops.hadamard_quantize_kv(torch.randn(cap, nkv, hd, generator=gen, device=dev), codes, norms, 0)
    payload = ops.capture_tq_kv(codes, norms, nkv, hd, cap, start, n)
    h, idx, nrm = tqp.unpack(payload)
    assert (h.codec_version, h.bits_per_coord, h.head_dim, h.n_kv_heads, h.n_tokens, h.flags, h.scale) == (2, 8, hd, nkv, n, 1, 1.0)
    assert idx == codes[:, start:start + n].contiguous().cpu().numpy().tobytes()
    assert nrm == norms.view(nkv, cap, -1)[:, start:start + n].contiguous().cpu().numpy().tobytes()
    codes2, norms2 = ops.alloc_tq_kv(nkv, cap, hd, dev)
    codes2.fill_(0x55)
    norms2.fill_(7.0)
    ops.restore_tq_kv(payload, codes2, norms2, nkv, hd, cap, start + 3)
    assert torch.equal(codes2[:, start + 3:start + 3 + n], codes[:, start:start + n])
    assert torch.equal(norms2.view(nkv, cap, -1)[:, start + 3:start + 3 + n], norms.view(nkv, cap, -1)[:, start:start + n])
    assert (codes2[:, :start + 3] == 0x55).all() and (codes2[:, start + 3 + n:] == 0x55).all()
    assert (norms2.view(nkv, cap, -1)[:, :start + 3] == 7.0).all() and (norms2.view(nkv, cap, -1)[:, start + 3 + n:] == 7.0).all()
    with pytest.raises(ops.HqError):  # would run past the capacity
        ops.restore_tq_kv(payload, codes2, norms2, nkv, hd, cap, cap - n + 1)
    with pytest.raises(ops.HqError):  # another cache shape
        ops.restore_tq_kv(payload, codes2, norms2, nkv + 1, hd, cap, 0)


def test_argument_errors(dev):
    nh, nkv, hd, cap = 16, 2, 256, 32
    kc, kn = ops.alloc_tq_kv(nkv, cap, hd, dev)
    q = torch.zeros(nh, hd, device=dev)
    out = torch.zeros(nh, hd, device=dev)
    tmp = torch.zeros(1 << 16, device=dev)

    def call(**kw):
        base = dict(num_heads=nh, num_kv_heads=nkv, head_dim=hd, kv_seq_len=4, kv_capacity=cap, scale=1.0)
        base.update(kw)
        ops.flash_attn_vec_tq_hb(q, kc, kn, kc, kn, out, tmp, FlashAttnVecTqHbParams(**base))

    call()
    for bad in (dict(kv_seq_len=0),                 # kv_cache.rs:3816 rejects_kv_seq_len_zero
                dict(kv_seq_len=cap + 1),           # kv_cache.rs:331-333
                dict(head_dim=128), dict(codebook_bits=7), dict(num_kv_heads=3), dict(mask_type=3)):
        with pytest.raises(ops.HqError) as e:
            call(**bad)
        assert e.value.status == 1
    for unsupported in (dict(codebook_bits=5),):
        with pytest.raises(ops.HqError) as e:
            call(**unsupported)
        assert e.value.status == 2
    with pytest.raises(ops.HqError):                # scratch too small
        ops.flash_attn_vec_tq_hb(q, kc, kn, kc, kn, out, tmp[:8], FlashAttnVecTqHbParams(nh, nkv, hd, 4, cap, 1.0))
    with pytest.raises(ops.HqError):
        ops.dispatch_fwht_sign_premult_f32(q, nh, 128)

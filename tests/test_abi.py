"""CPU-only checks of the C ABI: the library loads, exports every symbol the
header declares, and rejects bad arguments before touching a GPU."""
import ctypes
import os
import re

import pytest

from hf2q_amd import lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "hf2q_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = lib.load()
    names = _declared_symbols()
    assert len(names) >= 9
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/hf2q_hip.h but not exported"
        assert n in lib.SIGNATURES, f"{n} has no ctypes signature in hf2q_amd/lib.py"
    assert sorted(lib.SIGNATURES) == names


def test_block_geometry():
    # ggml_type.rs:60-135
    L = lib.load()
    assert (L.hq_block_elems(lib.HQ_Q4_K), L.hq_block_bytes(lib.HQ_Q4_K)) == (256, 144)
    assert (L.hq_block_elems(lib.HQ_Q6_K), L.hq_block_bytes(lib.HQ_Q6_K)) == (256, 210)
    assert (L.hq_block_elems(lib.HQ_Q8_0), L.hq_block_bytes(lib.HQ_Q8_0)) == (32, 34)
    assert (L.hq_block_elems(lib.HQ_Q5_K), L.hq_block_bytes(lib.HQ_Q5_K)) == (256, 176)  # q5_k.rs:57-59
    assert (L.hq_block_elems(lib.HQ_Q4_0), L.hq_block_bytes(lib.HQ_Q4_0)) == (32, 18)    # q4_0.rs:24-25
    assert L.hq_block_elems(3) == 0 and L.hq_block_bytes(10) == 0  # Q4_1, Q2_K: not built


def test_workspace_queries_follow_the_routing():
    """Pure host arithmetic (no GPU call): which shapes take a tile kernel and how much scratch that needs."""
    L = lib.load()
    for t, kq in ((lib.HQ_Q4_K, 256), (lib.HQ_Q5_K, 256), (lib.HQ_Q6_K, 256), (lib.HQ_Q8_0, 128), (lib.HQ_Q4_0, 128)):
        bb, be = L.hq_block_bytes(t), L.hq_block_elems(t)
        # dense: up to 8 rows never need scratch, nor do 16 rows of Q4_K / Q5_K (two chunks of eight through the
        # small-batch kernel); beyond that every type has small tiles (64 or 128 token rows) and needs the f16
        # activations (+ row scales) when k suits the tile kernel -- and the partial sums where k is cut into slices
        # (64 x 64 x 8192 Q4_K: one tile, four slices)
        assert L.hq_qmatmul_ggml_workspace_bytes(8, 512, 4 * kq, lib.HQ_BF16, t) == 0
        if t in (lib.HQ_Q4_K, lib.HQ_Q5_K):
            assert L.hq_qmatmul_ggml_workspace_bytes(16, 512, 4 * kq, lib.HQ_BF16, t) == 0
            assert L.hq_qmatmul_ggml_workspace_bytes(64, 64, 8192, lib.HQ_BF16, t) >= 64 * 8192 * 2 + 4 * 64 * 64 * 4
        else:
            assert L.hq_qmatmul_ggml_workspace_bytes(9, 512, 4 * kq, lib.HQ_BF16, t) >= 9 * 4 * kq * 2
        assert L.hq_qmatmul_ggml_workspace_bytes(17, 512, 4 * kq, lib.HQ_BF16, t) >= 17 * 4 * kq * 2
        need = L.hq_qmatmul_ggml_workspace_bytes(512, 512, 4 * kq, lib.HQ_BF16, t)
        assert need >= 512 * 4 * kq * 2 and need % 256 == 0
        if be == 32:
            assert L.hq_qmatmul_ggml_workspace_bytes(512, 512, 96, lib.HQ_BF16, t) == 0  # k % 128 != 0: no tile kernel
        # mul_mat_id: the grouped route wants >= 256 routed rows, >= 3 per expert and a contiguous stack
        n, k, E = 128, 2 * kq, 8
        stride = n * (k // be) * bb
        assert L.hq_qmatmul_id_ggml_workspace_bytes(64, 4, n, k, E, stride, t) > 0
        assert L.hq_qmatmul_id_ggml_workspace_bytes(64, 4, n, k, E, stride + 32, t) == 0  # padded stack
        assert L.hq_qmatmul_id_ggml_workspace_bytes(8, 4, n, k, E, stride, t) == 0        # decode-sized
    assert L.hq_qmatmul_id_ggml_workspace_bytes(64, 4, 128, 512, 8, 128 * 2 * 144, 10) == 0  # not a type of the library


def test_k_slices_never_start_past_the_end_of_a_row():
    """hq_qmatmul_ggml_k_slices for every k / 256 up to 130 and a spread of (m, n): the slices cover k, none is empty, and the
    last one starts inside the row (k = 8448, 8704, 8960, 10496, 10752, 12544 once gave eight slices of which the last began
    past it).  Pure host arithmetic: no GPU."""
    L = lib.load()
    s, per = ctypes.c_uint32(), ctypes.c_uint32()
    cut = 0
    for t in (lib.HQ_Q4_K, lib.HQ_Q5_K, lib.HQ_Q6_K, lib.HQ_Q8_0, lib.HQ_Q4_0):
        for nsb in range(1, 131):
            for m, n in ((9, 64), (17, 64), (64, 1536), (100, 130), (128, 4096), (200, 640), (256, 64), (256, 12288), (257, 64), (2048, 64)):
                lib.check(L.hq_qmatmul_ggml_k_slices(m, n, nsb * 256, t, ctypes.byref(s), ctypes.byref(per)))
                assert s.value >= 1 and per.value >= 1
                assert s.value * per.value >= nsb, (t, m, n, nsb, s.value, per.value)
                assert (s.value - 1) * per.value < nsb, (t, m, n, nsb, s.value, per.value)
                if m > 256:
                    assert s.value == 1
                cut += s.value > 1
    assert cut > 1000  # the query does describe cut products
    assert L.hq_qmatmul_ggml_k_slices(17, 64, 100, lib.HQ_Q4_K, ctypes.byref(s), ctypes.byref(per)) == lib.HQ_ERR_INVALID_ARGUMENT
    assert L.hq_qmatmul_ggml_k_slices(17, 64, 256, lib.HQ_Q4_K, None, ctypes.byref(per)) == lib.HQ_ERR_INVALID_ARGUMENT


def test_empty_inputs_are_accepted_without_work():
    """Zero rows / tokens / elements: HQ_OK before any launch (the pointers here are never dereferenced); an empty
    attention cache is an error, as there is nothing to attend to."""
    L = lib.load()
    fake = ctypes.c_void_p(0x1000)
    assert L.hq_qmatmul_ggml(None, fake, lib.HQ_BF16, fake, fake, 0, 8, 256, lib.HQ_Q4_K) == lib.HQ_OK
    assert L.hq_qmatmul_ggml_ws(None, fake, lib.HQ_BF16, fake, fake, 0, 8, 256, lib.HQ_Q6_K, None, 0) == lib.HQ_OK
    assert L.hq_qmatmul_id_ggml(None, fake, lib.HQ_F32, fake, fake, fake, None, 0, 0, 2, 8, 256, 4, 8 * 144, lib.HQ_Q4_K) == lib.HQ_OK
    assert L.hq_qmatmul_ggml_ws_prepared(None, fake, lib.HQ_BF16, fake, fake, fake, 0, 8, 256, lib.HQ_Q6_K, None, 0) == lib.HQ_OK
    assert L.hq_qmatmul_id_ggml_prepared(None, fake, lib.HQ_F32, fake, fake, fake, fake, None, 0, 0, 2, 8, 256, 4, 8 * 144, lib.HQ_Q4_K) == lib.HQ_OK
    assert L.hq_weight_row_scales_ggml(None, fake, fake, 0, 256, lib.HQ_Q4_K) == lib.HQ_OK
    assert L.hq_qmatmul_id_swiglu_ggml(None, fake, lib.HQ_BF16, fake, fake, None, None, fake, fake, None, 0, 0, 8, 128, 512, 8, 128 * 2 * 144, lib.HQ_Q4_K) == lib.HQ_OK
    assert L.hq_dequant_ggml(None, fake, fake, lib.HQ_F32, 0, lib.HQ_Q8_0) == lib.HQ_OK
    assert L.hq_quantize_ggml(None, fake, 0, 256, lib.HQ_Q5_K, fake) == lib.HQ_OK
    assert L.hq_moe_softmax_topk(None, fake, fake, fake, 0, 256, 8) == lib.HQ_OK
    assert L.hq_moe_weighted_reduce(None, fake, fake, None, None, None, fake, 0, 8, 2048) == lib.HQ_OK
    assert L.hq_silu_mul(None, fake, fake, fake, 0) == lib.HQ_OK
    assert L.hq_dense_gemv_bf16(None, fake, lib.HQ_F32, fake, fake, 0, 4, 16) == lib.HQ_OK
    assert L.hq_fwht_sign_premult_f32(None, fake, 0, 256) == lib.HQ_OK
    p = lib.TqAttnParams(16, 2, 256, 0, 64, 0.0625, 0, 0, 0.0, 0, 1.0, 8, 0, 1)
    assert L.hq_flash_attn_vec_tq(None, fake, fake, fake, fake, fake, None, fake, fake, 1 << 20, ctypes.byref(p)) == lib.HQ_ERR_INVALID_ARGUMENT
    assert "kv_seq_len" in lib.last_error()


def test_argument_errors_are_reported_not_fatal():
    L = lib.load()
    fake = ctypes.c_void_p(0x1000)  # never dereferenced: validation fails first
    # k not a multiple of the block size (quantizer.rs:57-71)
    assert L.hq_qmatmul_ggml(None, fake, lib.HQ_F32, fake, fake, 1, 8, 300, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    assert "multiple of the block size" in lib.last_error()
    # unsupported ggml type (forward_mlx.rs:9884-9886)
    assert L.hq_qmatmul_ggml(None, fake, lib.HQ_F32, fake, fake, 1, 8, 256, 10) == lib.HQ_ERR_UNSUPPORTED  # Q2_K
    assert L.hq_dequant_ggml(None, fake, fake, lib.HQ_F32, 100, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    # misaligned Q4_K weights
    assert L.hq_qmatmul_ggml(None, fake, lib.HQ_F32, ctypes.c_void_p(0x1002), fake, 1, 8, 256, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    assert "aligned" in lib.last_error()
    # null buffers
    assert L.hq_qmatmul_ggml(None, None, lib.HQ_F32, fake, fake, 1, 8, 256, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    # id form: expert stride smaller than an expert
    assert L.hq_qmatmul_id_ggml(None, fake, lib.HQ_F32, fake, fake, fake, None, 0, 1, 2, 8, 256, 4, 100, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    # the prepared forms want the scales; the scales call wants whole blocks and a type of the library
    assert L.hq_qmatmul_ggml_ws_prepared(None, fake, lib.HQ_BF16, fake, None, fake, 64, 8, 256, lib.HQ_Q4_K, fake, 1 << 20) == lib.HQ_ERR_INVALID_ARGUMENT
    assert "w_row_scales" in lib.last_error()
    assert L.hq_qmatmul_id_ggml_prepared(None, fake, lib.HQ_F32, fake, None, fake, fake, None, 0, 1, 2, 8, 256, 4, 8 * 144, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    assert L.hq_weight_row_scales_ggml(None, fake, fake, 8, 300, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    assert L.hq_weight_row_scales_ggml(None, fake, fake, 8, 256, 10) == lib.HQ_ERR_UNSUPPORTED
    assert L.hq_weight_row_scales_ggml(None, fake, None, 8, 256, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    # the SwiGLU form of mul_mat_id: both stacks' scales or neither; no form for this shape / type -> unsupported, said so
    assert L.hq_qmatmul_id_swiglu_ggml(None, fake, lib.HQ_BF16, fake, fake, fake, None, fake, fake, fake, 1 << 20, 64, 4, 128, 512, 8, 128 * 2 * 144, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    assert L.hq_qmatmul_id_swiglu_ggml(None, fake, lib.HQ_BF16, fake, None, None, None, fake, fake, fake, 1 << 20, 64, 4, 128, 512, 8, 128 * 2 * 144, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    assert L.hq_qmatmul_id_swiglu_ggml(None, fake, lib.HQ_BF16, fake, fake, None, None, fake, fake, fake, 1 << 20, 64, 4, 128, 512, 8, 128 * 2 * 210, lib.HQ_Q6_K) == lib.HQ_ERR_UNSUPPORTED
    assert L.hq_qmatmul_id_swiglu_ggml_workspace_bytes(64, 4, 128, 512, 8, 128 * 2 * 144, lib.HQ_Q4_K) > L.hq_qmatmul_id_ggml_workspace_bytes(64, 4, 128, 512, 8, 128 * 2 * 144, lib.HQ_Q4_K) > 0
    assert L.hq_qmatmul_id_swiglu_ggml(None, fake, lib.HQ_BF16, fake, fake, None, None, fake, fake, None, 0, 64, 4, 128, 512, 8, 128 * 2 * 144, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    assert "scratch" in lib.last_error()
    # batched form: too many jobs, a prefill-sized dense job, SwiGLU over bf16 activations
    jobs = (lib.QmatmulJob * 5)()
    for j in jobs:
        j.x, j.w, j.y, j.rows, j.top_k, j.n, j.k, j.n_experts = 0x1000, 0x1000, 0x1000, 1, 1, 8, 256, 1
    assert L.hq_qmatmul_batch_ggml(None, jobs, 5, lib.HQ_F32, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    assert L.hq_qmatmul_batch_ggml(None, None, 2, lib.HQ_F32, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    jobs[1].rows = 9
    assert L.hq_qmatmul_batch_ggml(None, jobs, 2, lib.HQ_F32, lib.HQ_Q4_K) == lib.HQ_ERR_UNSUPPORTED
    jobs[1].rows, jobs[1].x_up = 1, 0x1000
    assert L.hq_qmatmul_batch_ggml(None, jobs, 2, lib.HQ_BF16, lib.HQ_Q4_K) == lib.HQ_ERR_INVALID_ARGUMENT
    assert "x_up" in lib.last_error()
    assert L.hq_qmatmul_batch_ggml(None, jobs, 0, lib.HQ_F32, lib.HQ_Q4_K) == lib.HQ_OK
    assert L.hq_dense_gemv_bf16_pair(None, fake, lib.HQ_F32, fake, fake, 4, fake, fake, 1, 1, 12) == lib.HQ_ERR_INVALID_ARGUMENT
    assert L.hq_quantize_ggml(None, fake, 512, 300, lib.HQ_Q4_K, fake) == lib.HQ_ERR_INVALID_ARGUMENT
    assert L.hq_quantize_ggml(None, fake, 768, 512, lib.HQ_Q4_K, fake) == lib.HQ_ERR_INVALID_ARGUMENT
    with pytest.raises(lib.HqError):
        lib.check(lib.HQ_ERR_INVALID_ARGUMENT)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(FileNotFoundError):
        lib.load()


def test_flat_walk_plan_covers_every_row_with_no_empty_window():
    """hq_gemv_flat_plan for every row length of whole units up to 130 super-blocks / 400 blocks and a spread of row counts:
    a task is a power-of-two number of rows, its windows are within a wave's capacity, together they cover the task's
    units, and none of them is empty (only the last may be ragged)."""
    L = lib.load()
    outs = [ctypes.c_uint32() for _ in range(5)]
    refs = [ctypes.byref(o) for o in outs]
    for t, ue, cap, kmax in ((lib.HQ_Q4_K, 256, 16, 130), (lib.HQ_Q6_K, 256, 16, 130), (lib.HQ_Q8_0, 32, 64, 400)):
        for units in range(2, kmax + 1):
            for n in (1, 63, 512, 4096, 5120, 151936):
                lib.check(L.hq_gemv_flat_plan(n, units * ue, t, 4096, *refs))
                bu, r, st, uwe, capacity = (o.value for o in outs)
                assert bu == units and capacity == cap
                assert r >= 1 and r & (r - 1) == 0 and r <= cap
                assert 1 <= uwe <= cap and st >= 1
                assert st * uwe >= r * bu > (st - 1) * uwe, (t, units, n, r, st, uwe)
    # the shapes behind the ragged windows: 68 super-blocks a row on 4096 waves, 5120 rows -> two rows in nine windows
    lib.check(L.hq_gemv_flat_plan(5120, 17408, lib.HQ_Q4_K, 4096, *refs))
    assert [o.value for o in outs] == [68, 2, 9, 16, 16]
    assert L.hq_gemv_flat_plan(16, 256, lib.HQ_Q4_K, 4096, *refs) == lib.HQ_ERR_INVALID_ARGUMENT   # a single unit per row
    assert L.hq_gemv_flat_plan(16, 512, lib.HQ_Q4_K, 0, *refs) == lib.HQ_ERR_INVALID_ARGUMENT
    assert L.hq_gemv_flat_plan(16, 512, lib.HQ_Q4_K, 4096, None, *refs[1:]) == lib.HQ_ERR_INVALID_ARGUMENT

"""GGUF file -> device -> matmul: tensors loaded through the reader drive the kernels like directly
uploaded blocks do."""
import numpy as np
import pytest
import torch

from _util import acts, assert_matmul_close, weights
from hf2q_amd import ops
from hf2q_amd.ops import HQ_Q4_K, HQ_Q6_K, GgmlQuantizedMatmulIdParams, GgmlQuantizedMatmulParams
from oracle import gguf as W

pytestmark = pytest.mark.gpu


def test_gguf_tensors_drive_gemv_and_mul_mat_id(oracle, dev, tmp_path):
    n, k, E, top_k = 96, 512, 4, 2
    dense = oracle.quantize(weights(1, n, k), k, HQ_Q6_K, threads=8)
    stack = oracle.quantize(weights(2, E * n, k), k, HQ_Q4_K, threads=8)
    path = str(tmp_path / "m.gguf")
    W.write(path, [("general.architecture", W.STRING, "test")],
            [("output.weight", [k, n], HQ_Q6_K, dense.tobytes()), ("blk.0.ffn_gate_exps.weight", [k, n, E], HQ_Q4_K, stack.tobytes())])
    with ops.GgufFile.open(path) as g:
        di, si = g.tensor_info("output.weight"), g.tensor_info("blk.0.ffn_gate_exps.weight")
        wd, ws = g.load_tensor("output.weight", dev), g.load_tensor("blk.0.ffn_gate_exps.weight", dev)
    assert (di.ggml_dtype, di.rows, di.cols) == (HQ_Q6_K, n, k) and si.shape == (k, n, E)
    assert torch.equal(wd.cpu(), torch.from_numpy(dense)) and torch.equal(ws.cpu(), torch.from_numpy(stack))

    x = acts(3, 2, k)
    y = torch.empty(2, n, device=dev)
    ops.quantized_matmul_ggml(torch.from_numpy(x).to(dev), wd, y, GgmlQuantizedMatmulParams(2, di.rows, di.cols, di.ggml_dtype))
    assert_matmul_close(y.cpu().numpy(), oracle.qmatmul_f64(x, dense, 2, n, k, HQ_Q6_K), "gemv from gguf")

    ids = np.array([3, 0, 1, 3], dtype=np.int32)
    stride = si.byte_len // si.shape[2]   # forward_mlx.rs:2438-2460
    yid = torch.empty(2 * top_k, n, device=dev)
    ops.quantized_matmul_id_ggml(torch.from_numpy(x).to(dev), ws, torch.from_numpy(ids).to(dev), yid,
                                 GgmlQuantizedMatmulIdParams(2, top_k, n, k, E, stride, HQ_Q4_K))
    per = stack.reshape(E, -1)
    for p, e in enumerate(ids):
        ref = oracle.qmatmul_f64(x[p // top_k:p // top_k + 1], per[e], 1, n, k, HQ_Q4_K)
        assert_matmul_close(yid[p].cpu().numpy(), ref, f"mul_mat_id row {p} from gguf")


def test_gguf_float_tensors_take_the_dense_routes_of_dispatch_qmatmul(oracle, dev, tmp_path):
    """An f32 router projection and an f16 tensor whose rows are not whole super-blocks (forward_mlx.rs:9820-9917), loaded
    as MlxQWeight and multiplied through dispatch_qmatmul at one row and at a prompt's worth."""
    k, n_r, n_d = 704, 128, 96
    rng = np.random.default_rng(5)
    router = (rng.standard_normal((n_r, k)) * 0.05).astype(np.float32)
    down = (rng.standard_normal((n_d, k)) * 0.05).astype(np.float16)
    blocks = oracle.quantize(weights(4, n_d, 768), 768, HQ_Q4_K, threads=8)
    path = str(tmp_path / "f.gguf")
    W.write(path, [("general.architecture", W.STRING, "test")],
            [("blk.0.ffn_gate_inp.weight", [k, n_r], ops.GGML_F32, router.tobytes()),
             ("blk.0.ffn_down.weight", [k, n_d], ops.GGML_F16, down.tobytes()), ("blk.0.ffn_up.weight", [768, n_d], HQ_Q4_K, blocks.tobytes())])
    with ops.GgufFile.open(path) as g:
        wr, wdn, wq = (g.load_weight(nm, dev) for nm in ("blk.0.ffn_gate_inp.weight", "blk.0.ffn_down.weight", "blk.0.ffn_up.weight"))
    assert (wr.buffer.dtype, wr.rows, wr.cols) == (torch.float32, n_r, k) and (wdn.buffer.dtype, wdn.rows, wdn.cols) == (torch.float16, n_d, k)
    assert wq.buffer.dtype == torch.uint8 and wq.ggml_dtype == HQ_Q4_K
    assert torch.equal(wr.buffer.cpu().view(n_r, k), torch.from_numpy(router)) and torch.equal(wdn.buffer.cpu().view(n_d, k), torch.from_numpy(down))
    for m in (1, 20):
        x = acts(m, m, k)
        xd = torch.from_numpy(x).to(dev)
        for w, host in ((wr, router), (wdn, down)):
            y = torch.full((m, w.rows), float("nan"), device=dev)
            ops.dispatch_qmatmul(xd, w, y, m)
            xv = x.astype(np.float16) if (m > 8 and host.dtype == np.float16) else x
            ref = xv.astype(np.float64) @ host.astype(np.float64).T
            assert np.abs(y.cpu().numpy() - ref).max() <= (1e-5 if m <= 8 else 1e-3) * np.abs(ref).max()
    x = acts(9, 1, 768)
    y = torch.empty(1, n_d, device=dev)
    ops.dispatch_qmatmul(torch.from_numpy(x).to(dev), wq, y, 1)
    assert_matmul_close(y.cpu().numpy(), oracle.qmatmul_f64(x, blocks, 1, n_d, 768, HQ_Q4_K), "block weight through load_weight")

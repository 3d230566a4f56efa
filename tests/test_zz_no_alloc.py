"""hq_flash_attn_vec_tq_static (the entry point that allocates nothing: its scratch is a static device array) against
hq_flash_attn_vec_tq with caller scratch: the same kernels, so the outputs must be bit-identical.  Two calls in a
row through the C ABI, the second over a shorter context, then a shape beyond the static buffer."""
import numpy as np
import pytest
import torch

from hf2q_amd import lib, ops
from hf2q_amd.ops import FlashAttnVecTqHbParams

pytestmark = pytest.mark.gpu


def _cache(dev, n_kv, cap, hd, seed):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    kc, kn = ops.alloc_tq_kv(n_kv, cap, hd, dev)
    vc, vn = ops.alloc_tq_kv(n_kv, cap, hd, dev)
    ops.hadamard_quantize_kv(torch.randn(cap, n_kv, hd, generator=g, device=dev), kc, kn, 0)
    ops.hadamard_quantize_kv(torch.randn(cap, n_kv, hd, generator=g, device=dev), vc, vn, 0)
    return kc, kn, vc, vn


@pytest.mark.parametrize("hd, nh, nkv", [(256, 16, 2), (512, 8, 2)])
def test_static_scratch_attention_equals_caller_scratch(dev, hd, nh, nkv):
    cap = 4096
    cache = _cache(dev, nkv, cap, hd, 11)
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    q = torch.randn(nh, hd, generator=g, device=dev)
    # two calls in a row on one GPU share the static buffer: the second is smaller and must not see the first's data
    for n, undo, fuse in ((4096, True, 1), (777, False, 0), (33, True, 0)):
        p = FlashAttnVecTqHbParams(nh, nkv, hd, n, cap, 1.0 / 16.0, fuse_fwht_pre=fuse)
        tmp = torch.empty(ops.tq_tmp_buffer_bytes(nh, hd, n) // 4, device=dev)
        want = torch.full((nh, hd), float("nan"), device=dev)
        ops.flash_attn_vec_tq_hb(q, *cache, want, tmp, p, undo_rotation=undo)
        got = torch.full((nh, hd), float("nan"), device=dev)
        ops.flash_attn_vec_tq_hb_static(q, *cache, got, p, undo_rotation=undo)
        torch.cuda.synchronize()
        assert torch.isfinite(want).all()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), f"kv_seq_len {n}: static scratch differs"


def test_static_scratch_rejects_shapes_beyond_the_buffer(dev):
    nh, nkv, hd, n = 64, 8, 512, 32768  # 64 heads x 2 blocks x 128 splits x 1032 B = 16.9 MB > 4 MiB
    assert ops.tq_tmp_buffer_bytes(nh, hd, n) > (4 << 20)
    cache = _cache(dev, nkv, 64, hd, 3)
    q = torch.zeros(nh, hd, device=dev)
    out = torch.zeros(nh, hd, device=dev)
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, n, 1.0 / 16.0)
    with pytest.raises(lib.HqError) as e:
        ops.flash_attn_vec_tq_hb_static(q, *cache, out, p)
    assert e.value.status == lib.HQ_ERR_INVALID_ARGUMENT and "static buffer" in e.value.message

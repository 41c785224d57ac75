"""GPU parity of reshape_and_cache (the older paged-cache layout) against the CPU oracle, bit for bit.
Shapes follow tests/test_attention_ops.py:1254-1322 of the reference."""
import random

import pytest
import torch

import flag_gems
from flag_gems.patches import patch_vllm_all
from oracle import torch_ref as O

from helpers import gems_assert_equal

pytestmark = pytest.mark.gpu


def _caches(num_blocks, block_size, heads, head_size, dtype, dev):
    x = 16 // torch.tensor([], dtype=dtype).element_size()
    kc = torch.randn(num_blocks, heads, head_size // x, block_size, x, dtype=dtype, device=dev)
    vc = torch.randn(num_blocks, heads, head_size, block_size, dtype=dtype, device=dev)
    return kc, vc


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("head_size", [64, 80, 120, 256])
@pytest.mark.parametrize("block_size", [8, 16, 32])
@pytest.mark.parametrize("num_blocks", [1024, 10000])
def test_reshape_and_cache(gpu, dtype, head_size, block_size, num_blocks):
    random.seed(0); torch.manual_seed(0)
    num_tokens, num_heads = 42, 8
    slots = torch.tensor(random.sample(range(num_blocks * block_size), num_tokens), dtype=torch.long, device=gpu)
    qkv = torch.randn(num_tokens, 3, num_heads, head_size, dtype=dtype, device=gpu)
    _, key, value = qkv.unbind(dim=1)  # strided views
    kc, vc = _caches(num_blocks, block_size, num_heads, head_size, dtype, gpu)
    ref_k, ref_v = O.reshape_and_cache(key, value, kc, vc, slots)
    k_scale = (key.amax() / 64.0).to(torch.float32); v_scale = (value.amax() / 64.0).to(torch.float32)
    flag_gems.reshape_and_cache(key, value, kc, vc, slots, "auto", k_scale, v_scale)
    gems_assert_equal(kc, ref_k); gems_assert_equal(vc, ref_v)  # written cells and the untouched rest


def test_reshape_and_cache_edges_and_hook(gpu):
    torch.manual_seed(1)
    H, D, bs, nb = 2, 24, 4, 9
    key = torch.randn(7, H, D, dtype=torch.float16, device=gpu); value = torch.randn_like(key)
    kc = torch.zeros(nb, H, D // 8, bs, 8, dtype=torch.float16, device=gpu)
    vc = torch.zeros(nb, H, D, bs, dtype=torch.float16, device=gpu)
    # negative slots are padding, a slot past the last block is dropped; int32 slots; fewer slots than key rows
    slots = torch.tensor([5, -1, 0, 35, nb * bs + 2], dtype=torch.int32, device=gpu)
    ref_k, ref_v = O.reshape_and_cache(key, value, kc, vc, torch.tensor([5, -1, 0, 35, -1]))
    flag_gems.reshape_and_cache(key, value, kc, vc, slots, "auto", None, None)
    gems_assert_equal(kc, ref_k); gems_assert_equal(vc, ref_v)
    assert int((vc != 0).sum()) <= 3 * H * D and int((vc != 0).any(1).any(1).sum()) == 3
    # the vLLM hook takes a 2-D slot mapping
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    patch_vllm_all.custom_gems_write_to_paged_cache(key[:4], value[:4], kc2, vc2,
                                                    torch.tensor([[5, 0], [35, 8]], device=gpu), "auto", None, None)
    ref_k, ref_v = O.reshape_and_cache(key[:4], value[:4], torch.zeros_like(kc), torch.zeros_like(vc), torch.tensor([5, 0, 35, 8]))
    gems_assert_equal(kc2, ref_k); gems_assert_equal(vc2, ref_v)
    # empty; shape checks happen on the host
    flag_gems.reshape_and_cache(key[:0], value[:0], kc, vc, slots[:0], "auto", None, None)
    with pytest.raises(AssertionError):
        flag_gems.reshape_and_cache(key, value, kc, vc.transpose(2, 3), slots, "auto", None, None)
    with pytest.raises(AssertionError):
        flag_gems.reshape_and_cache(key, value, kc[:, :, :2], vc, slots, "auto", None, None)

"""vLLM hooks (reference: src/flag_gems/patches/).  vLLM is not installed here, so the installer runs
against a stand-in module tree that has the classes and the `_C::silu_and_mul` schema it touches; what the
replacement methods compute is checked on the GPU in tests/test_gpu_modules.py."""
import sys
import types

import pytest
import torch

import flag_gems
from flag_gems.patches import patch_util, patch_vllm_all


def _fake_vllm(monkeypatch):
    names = {
        "vllm.attention.ops.paged_attn": ["PagedAttention"],
        "vllm.model_executor.layers.activation": ["SiluAndMul"],
        "vllm.model_executor.layers.layernorm": ["RMSNorm"],
        "vllm.model_executor.layers.rotary_embedding": ["RotaryEmbedding"],
        "vllm.v1.attention.backends.flash_attn": ["FlashAttentionImpl"],
    }
    classes = {}
    for mod_name, cls_names in names.items():
        parts = mod_name.split(".")
        for i in range(1, len(parts) + 1):
            sub = ".".join(parts[:i])
            if sub not in sys.modules:
                monkeypatch.setitem(sys.modules, sub, types.ModuleType(sub))
        for c in cls_names:
            cls = type(c, (), {"forward_cuda": lambda self, *a: "native", "forward": lambda self, *a: "native",
                               "write_to_paged_cache": staticmethod(lambda *a: "native")})
            setattr(sys.modules[mod_name], c, cls)
            classes[c] = cls
    return classes


def test_installer_needs_vllm():
    if "vllm" in sys.modules:
        pytest.skip("a vllm module is loaded")
    with pytest.raises(ImportError):
        flag_gems.apply_gems_patches_to_vllm(verbose=False)


def test_installer_patches_methods_and_library_kernel(monkeypatch, capsys):
    classes = _fake_vllm(monkeypatch)
    # the schema vLLM's extension defines; a CPU kernel stands for its native implementation
    define = torch.library.Library("_C", "FRAGMENT")
    define.define("silu_and_mul(Tensor! out, Tensor input) -> ()")
    seen = []
    monkeypatch.setattr(patch_vllm_all, "custom_silu_and_mul", lambda out, input: seen.append(tuple(input.shape)))
    monkeypatch.setattr(patch_util, "_libs", {})
    real_impl = torch.library.Library.impl
    keys = []

    def impl(self, name, fn, key=""):
        keys.append((name, key))
        return real_impl(self, name, fn, "CPU")  # no GPU here: same registration path, CPU key

    monkeypatch.setattr(torch.library.Library, "impl", impl)
    flag_gems.apply_gems_patches_to_vllm(verbose=True)
    out = capsys.readouterr().out
    assert classes["RMSNorm"].forward_cuda is patch_vllm_all.custom_gems_rms_forward_cuda
    assert classes["RotaryEmbedding"].forward_cuda is patch_vllm_all.custom_gems_rope_forward_cuda
    assert classes["SiluAndMul"].forward_cuda is patch_vllm_all.custom_gems_silu_and_mul
    assert classes["FlashAttentionImpl"].forward is patch_vllm_all.custom_gems_flash_attention_impl_forward
    assert classes["PagedAttention"].write_to_paged_cache is patch_vllm_all.custom_gems_write_to_paged_cache
    assert keys == [("silu_and_mul", "CUDA")]
    torch.ops._C.silu_and_mul(torch.empty(2, 4), torch.ones(2, 8))
    assert seen == [(2, 8)]
    for line in ("Patched RMSNorm.forward_cuda with FLAGGEMS custom_gems_rms_forward_cuda",
                 "Patched torch.ops._C.silu_and_mul with FLAGGEMS", "Left TritonMLAImpl._forward_decode on vLLM"):
        assert line in out
    del define


def test_patch_util_contract():
    class K:
        def f(self):
            return 1

    old = patch_util.patch_module_method(K, "f", lambda self: 2, verbose=False)
    assert K().f() == 2 and old(K()) == 1
    assert patch_util.patch_module_method(K, "g", lambda self: 3, verbose=False) is None and K().g() == 3
    with pytest.raises(ValueError):
        patch_util.patch_vllm_lib("_other", "x", lambda: None, "CUDA", verbose=False)


def test_attention_hook_early_exits():
    impl = types.SimpleNamespace(kv_cache_dtype="auto", use_irope=False)
    f = patch_vllm_all.custom_gems_flash_attention_impl_forward
    out = torch.zeros(1)
    assert f(impl, None, None, None, None, None, None, output=out) is out  # profiling pass: no metadata
    with pytest.raises(AssertionError):
        f(impl, None, None, None, None, None, object(), output=None)
    with pytest.raises(NotImplementedError):
        f(impl, None, None, None, None, None, object(), output=out, output_scale=torch.ones(1))
    impl.kv_cache_dtype = "fp8_e4m3"
    with pytest.raises(NotImplementedError):
        f(impl, None, None, None, None, None, object(), output=out)


# ---- what the replacement methods compute (GPU, against the CPU oracle) ------------------------------------------
from oracle import torch_ref as O  # noqa: E402

from helpers import gems_assert_close  # noqa: E402


@pytest.mark.gpu
def test_vllm_rms_hook(gpu):
    torch.manual_seed(0)
    dtype, n = torch.bfloat16, 4096
    layer = types.SimpleNamespace(weight=torch.randn(n, device=gpu, dtype=dtype), variance_epsilon=1e-5)
    x = torch.randn(37, n, device=gpu, dtype=dtype)
    out = patch_vllm_all.custom_gems_rms_forward_cuda(layer, x)
    gems_assert_close(out, O.rms_norm(x, layer.weight, 1e-5), dtype, reduce_dim=n)
    res = torch.randn_like(x)
    ref_x, ref_res = O.fused_add_rms_norm(x, res, layer.weight, 1e-5)
    ox, ores = patch_vllm_all.custom_gems_rms_forward_cuda(layer, x.clone(), res.clone())
    gems_assert_close(ox, ref_x, dtype, reduce_dim=n)
    gems_assert_close(ores, ref_res, dtype)


def _vllm_cos_sin_cache(rotary_dim, max_pos, base, device):
    # the layout of vLLM's RotaryEmbedding buffer: [max_position, rotary_dim], cos half then sin half
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    freqs = torch.outer(torch.arange(max_pos, dtype=torch.float32), inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1).to(device)


@pytest.mark.gpu
@pytest.mark.parametrize("rotary_dim", [128, 64])
@pytest.mark.parametrize("neox", [True, False])
@pytest.mark.parametrize("with_offsets", [False, True])
def test_vllm_rope_hook(gpu, rotary_dim, neox, with_offsets):
    torch.manual_seed(1)
    tokens, hq, hk, hs, max_pos, dtype = 53, 8, 2, 128, 512, torch.bfloat16
    layer = types.SimpleNamespace(cos_sin_cache=_vllm_cos_sin_cache(rotary_dim, max_pos, 10000.0, gpu), head_size=hs,
                                  rotary_dim=rotary_dim, is_neox_style=neox)
    q = torch.randn(tokens, hq * hs, device=gpu, dtype=dtype)
    k = torch.randn(tokens, hk * hs, device=gpu, dtype=dtype)
    pos = torch.randint(0, max_pos // 2, (tokens,), device=gpu)
    off = torch.randint(0, max_pos // 2, (tokens,), device=gpu) if with_offsets else None
    eff = pos if off is None else pos + off
    q3, k3 = q.view(tokens, hq, hs).clone(), k.view(tokens, hk, hs).clone()
    cos, sin = layer.cos_sin_cache.chunk(2, dim=-1)
    rq, rk = O.apply_rotary_pos_emb(q3[..., :rotary_dim], k3[..., :rotary_dim], cos, sin, eff, not neox)
    ref_q, ref_k = q3.double().cpu(), k3.double().cpu()
    ref_q[..., :rotary_dim] = rq
    ref_k[..., :rotary_dim] = rk
    oq, ok = patch_vllm_all.custom_gems_rope_forward_cuda(layer, pos, q, k, off)
    assert oq.shape == q.shape and ok.shape == k.shape
    gems_assert_close(oq.view(tokens, hq, hs), ref_q, dtype)
    gems_assert_close(ok.view(tokens, hk, hs), ref_k, dtype)


@pytest.mark.gpu
def test_vllm_silu_hooks(gpu):
    torch.manual_seed(2)
    dtype, d = torch.bfloat16, 11008
    x = torch.randn(33, 2 * d, device=gpu, dtype=dtype)
    ref = O.silu_and_mul(x[:, :d], x[:, d:])
    gems_assert_close(patch_vllm_all.custom_gems_silu_and_mul(None, x), ref, dtype)
    out = torch.empty(33, d, device=gpu, dtype=dtype)
    patch_vllm_all.custom_silu_and_mul(out, x)
    gems_assert_close(out, ref, dtype)


@pytest.mark.gpu
def test_vllm_attention_hook(gpu):
    """One scheduler step of the v1 backend: three sequences (a prefill chunk on top of cached keys, a decode
    token, a fresh prefill); the step's K/V rows go into the paged cache first and are attended to."""
    torch.manual_seed(3)
    dtype, hq, hk, d, page, pages_total = torch.bfloat16, 8, 2, 128, 16, 64
    seqs = [(5, 40), (1, 300), (17, 17)]  # (query tokens of this step, keys after this step)
    qlens = [s[0] for s in seqs]; klens = [s[1] for s in seqs]
    n = sum(qlens)
    pages_per_seq = (max(klens) + page - 1) // page
    assert len(seqs) * pages_per_seq <= pages_total
    table = torch.randperm(pages_total)[: len(seqs) * pages_per_seq].view(len(seqs), pages_per_seq).to(torch.int32)
    slots = []
    for i, (ql, kl) in enumerate(seqs):
        for p in range(kl - ql, kl):
            slots.append(int(table[i, p // page]) * page + p % page)
    kv_cache = torch.randn(2, pages_total, page, hk, d, device=gpu, dtype=dtype)
    before = kv_cache.clone()
    # two padding tokens behind the real ones, as in a captured-size batch
    query = torch.randn(n + 2, hq, d, device=gpu, dtype=dtype)
    key = torch.randn(n + 2, hk, d, device=gpu, dtype=dtype)
    value = torch.randn(n + 2, hk, d, device=gpu, dtype=dtype)
    slot_mapping = torch.tensor(slots + [-1, -1], dtype=torch.int64, device=gpu)
    meta = types.SimpleNamespace(
        num_actual_tokens=n, slot_mapping=slot_mapping, use_cascade=False, local_attn_metadata=None,
        query_start_loc=torch.tensor([0] + qlens, dtype=torch.int32, device=gpu).cumsum(0, dtype=torch.int32),
        seq_lens=torch.tensor(klens, dtype=torch.int32, device=gpu), max_query_len=max(qlens), max_seq_len=max(klens),
        block_table=table.to(gpu), scheduler_metadata=None,
    )
    one = torch.ones(1, device=gpu)
    layer = types.SimpleNamespace(_q_scale=one, _k_scale=one, _v_scale=one)
    impl = types.SimpleNamespace(kv_cache_dtype="auto", use_irope=False, scale=d ** -0.5, alibi_slopes=None,
                                 sliding_window=(-1, -1), logits_soft_cap=0.0)
    output = torch.full((n + 2, hq, d), 7.0, device=gpu, dtype=dtype)
    ret = patch_vllm_all.custom_gems_flash_attention_impl_forward(impl, layer, query, key, value, kv_cache, meta,
                                                                  output=output)
    assert ret is output
    kc, vc = O.reshape_and_cache_flash(key, value, before[0], before[1], slot_mapping)
    assert torch.equal(kv_cache[0].cpu(), kc) and torch.equal(kv_cache[1].cpu(), vc)  # the scatter is bit-exact
    ref = O.paged_attention(query[:n], kc, vc, qlens, klens, table, d ** -0.5, causal=True, compute_dtype=torch.float32)
    torch.testing.assert_close(output[:n].float().cpu(), ref, atol=2e-2, rtol=1e-2)
    assert (output[n:] == 7.0).all()  # rows past num_actual_tokens are not touched

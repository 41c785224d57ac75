"""Writes tests/golden/golden_v1.npz: small seeded inputs and the expected outputs the CPU oracle
(oracle/torch_ref.py, PyTorch ATen on the host) gives for them.

The reference ships no golden vectors for this path (all of its expectations are computed live
from torch), and its own implementation needs a GPU plus Triton, so it is read, not run; these
fixtures freeze the oracle's outputs so that (a) a later change of the oracle or of the torch
build shows up as a diff and (b) the GPU kernels are compared against committed numbers as well as
against the live oracle.  Inputs are stored as float32 values that are exactly representable in
the dtype named in the key (so loading and casting is lossless); expected outputs are float64.

Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import torch_ref as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden_v1.npz")


def rnd(gen, shape, dtype, scale=1.0):
    return (torch.randn(shape, generator=gen) * scale).to(dtype)


def main():
    g = torch.Generator().manual_seed(20251125)
    d = {}
    bf16, f16 = torch.bfloat16, torch.float16

    # rms_norm / fused_add_rms_norm: 4 x 8 (bf16) and 3 x 40 (fp16)
    for tag, dt, shape in (("bf16", bf16, (4, 8)), ("f16", f16, (3, 40))):
        x, r = rnd(g, shape, dt), rnd(g, shape, dt)
        w = (torch.rand(shape[-1], generator=g) + 0.5).to(dt)
        d[f"rms_{tag}_x"], d[f"rms_{tag}_r"], d[f"rms_{tag}_w"] = x.float().numpy(), r.float().numpy(), w.float().numpy()
        d[f"rms_{tag}_y"] = O.rms_norm(x, w, 1e-5).double().numpy()
        y, s = O.fused_add_rms_norm(x, r, w, 1e-5)
        d[f"fused_{tag}_y"], d[f"fused_{tag}_res"] = y.numpy(), s.numpy()

    # softmax 5 x 33 with -inf entries and one fully masked row
    x = rnd(g, (5, 33), bf16, 2.0)
    x[x < -1.0] = float("-inf")
    x[3] = float("-inf")
    d["softmax_bf16_x"] = x.float().numpy()
    d["softmax_bf16_y"] = O.softmax(x, -1).numpy()

    # mm / addmm 7 x 24 x 9
    a, b, bias = rnd(g, (7, 24), f16), rnd(g, (24, 9), f16), rnd(g, (9,), f16)
    d["mm_f16_a"], d["mm_f16_b"], d["mm_f16_bias"] = a.float().numpy(), b.float().numpy(), bias.float().numpy()
    d["mm_f16_c"] = O.mm(a, b).numpy()
    d["addmm_f16_c"] = O.addmm(bias, a, b, alpha=-0.999, beta=100.001).numpy()

    # rope: 2 x 5 tokens, (3, 1) heads, D = 16, both pairings, with position ids
    q, k = rnd(g, (2, 5, 3, 16), bf16), rnd(g, (2, 5, 1, 16), bf16)
    cos, sin = O.rope_cos_sin(32, 16)
    pos = torch.randint(0, 32, (2, 5), generator=g)
    d["rope_q"], d["rope_k"], d["rope_pos"] = q.float().numpy(), k.float().numpy(), pos.numpy()
    d["rope_cos"], d["rope_sin"] = cos.numpy(), sin.numpy()
    for inter in (False, True):
        oq, ok = O.apply_rotary_pos_emb(q, k, cos, sin, pos, inter)
        d[f"rope_oq_{int(inter)}"], d[f"rope_ok_{int(inter)}"] = oq.numpy(), ok.numpy()

    # silu_and_mul 3 x 10
    a, b = rnd(g, (3, 10), f16, 3.0), rnd(g, (3, 10), f16)
    d["silu_a"], d["silu_b"] = a.float().numpy(), b.float().numpy()
    d["silu_y"] = O.silu_and_mul(a, b).numpy()

    # paged attention: 3 sequences (q, kv) = (1, 20), (5, 18), (9, 9); 4 query heads over 2 kv heads;
    # D = 16; page size 4; 12 pages
    qlens, klens = [1, 5, 9], [20, 18, 9]
    q = rnd(g, (sum(qlens), 4, 16), bf16)
    kc, vc = rnd(g, (12, 4, 2, 16), bf16), rnd(g, (12, 4, 2, 16), bf16)
    bt = torch.randint(0, 12, (3, 5), generator=g, dtype=torch.int32)
    d["attn_q"], d["attn_kc"], d["attn_vc"], d["attn_bt"] = q.float().numpy(), kc.float().numpy(), vc.float().numpy(), bt.numpy()
    d["attn_qlens"], d["attn_klens"] = np.array(qlens), np.array(klens)
    out, lse = O.paged_attention(q, kc, vc, qlens, klens, bt, 0.25, causal=True, compute_dtype=torch.float64, return_lse=True)
    d["attn_out"], d["attn_lse"] = out.numpy(), lse.double().numpy()

    # cache scatter: 6 tokens into 5 pages of 4 slots, 2 heads x 8; one padding token
    key, val = rnd(g, (6, 2, 8), bf16), rnd(g, (6, 2, 8), bf16)
    kc0, vc0 = rnd(g, (5, 4, 2, 8), bf16), rnd(g, (5, 4, 2, 8), bf16)
    slots = torch.tensor([7, 0, -1, 19, 12, 5])
    kc1, vc1 = O.reshape_and_cache_flash(key, val, kc0, vc0, slots)
    d["cache_key"], d["cache_val"], d["cache_kc0"], d["cache_vc0"] = (t.float().numpy() for t in (key, val, kc0, vc0))
    d["cache_slots"] = slots.numpy()
    d["cache_kc1"], d["cache_vc1"] = kc1.float().numpy(), vc1.float().numpy()

    np.savez_compressed(OUT, **d)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(d), "arrays")


if __name__ == "__main__":
    main()

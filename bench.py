#!/usr/bin/env python3
"""Benchmark of the MI355X-native FlagGems operator path on ONE GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extra] [--no-cpu] [--settle-ms T]

A "step" is one pass of one operator over one batch of synthetic input that is already resident in
HBM.  The headline workload (the JSON line's metric/value) is the softmax configuration of
BASELINE.json: softmax over the last axis of a [131072, 2048] bf16 tensor, ~N(0, 4) with 1 % of the
entries at -inf.  Its 1 GiB of algorithmic traffic (read + write of one tensor) is larger than the
256 MB Infinity Cache, so the rate is an HBM rate.  The other configurations (fused_add_rms_norm,
the three GEMMs, varlen GQA prefill attention, the decoder layer) are measured in the same run and
reported under "configs", each with its own roofline entry.

Timing: an untimed run-in of T ms of the workload's own steps (the part throttles for ~40 ms of work after
any pause, see timed() below; --settle-ms 0 switches it off and shows that transient instead of the
sustained rate), W untimed warm-up steps, then exactly K steps bracketed by torch.cuda.synchronize() on
both sides (one GPU, so the barrier is the synchronize).  ms_per_step / value come from the wall clock
around the K steps; roofline.achieved comes from HIP events recorded on the stream the kernels are
launched on (torch's current stream) around the same K steps.

cpu_baseline: the CPU oracle (PyTorch ATen on the host, the computation the reference's --ref cpu
tests use as ground truth) timed on this machine's cores on a bounded sample of the same workload.
It is a reported baseline, never the thing optimised.
"""
import argparse
import json
import math
import random
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16/fp16 MFMA, published


def _die_multi_gpu(n):
    print(
        "bench.py: this build measures one GPU only (--gpus %d requested). The operator path has no "
        "collective; run it with --gpus 1." % n,
        file=sys.stderr,
    )
    sys.exit(2)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="softmax_c2")
    ap.add_argument("--no-extra", action="store_true", help="measure only --workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--settle-ms", type=float, default=200.0,
                    help="untimed run-in of each workload before its warm-up steps, in ms of its own steps (0: none)")
    return ap.parse_args()


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        _die_multi_gpu(max(args.gpus, int(os.environ.get("WORLD_SIZE", "1"))))

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    import flag_gems
    from flaggems_amd import _C
    from flaggems_amd.ops import _gemm

    if not os.path.exists(_C.LIB_PATH):  # load what is built; build only if nothing is
        import __graft_entry__

        __graft_entry__.build()
    _C.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    bf16 = torch.bfloat16

    # ------------------------------------------------------------------------------------------
    def timed(run, steps, warmup):
        """(wall ms per step, event ms per step) for `steps` calls of run(i).

        Run-in: after any pause of the GPU (10 ms is enough: the set-up of a workload, the CPU baseline before
        it) the part's power management lets two launches through at full rate, throttles the next ones by
        20-25 % and recovers over the following ~40 ms of continuous work (a bf16 GEMM of 8192^3, TFLOP/s per
        launch: 1300 1310 1120 990 1000 1080 1110 1140 ... 1335 from the 40th launch on; the vendor library's
        GEMM traces the same curve).  A few warm-up steps of a millisecond each end inside that trough, so each
        workload first repeats its own step for --settle-ms of wall time, untimed; the warm-up steps and the
        timed steps follow without a pause."""
        if args.settle_ms > 0:
            t_end = time.perf_counter() + args.settle_ms * 1e-3
            i = 0
            while time.perf_counter() < t_end:
                for _ in range(4):
                    run(i)
                    i += 1
                torch.cuda.synchronize()
        for i in range(warmup):
            run(i)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(steps):
            run(i)
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps

    def roofline(bound, work, ev_ms, traffic=None):
        if bound == "hbm":
            ach = work / ev_ms / 1e6  # GB/s
            return {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": traffic}
        ach = work / ev_ms / 1e9  # TFLOP/s
        return {"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(ach / MFMA_PEAK_TFLOPS, 4), "traffic": traffic}

    def cpu_time(fn, min_seconds=2.0, max_reps=5):
        fn()  # warm-up
        ts = []
        t_all = time.perf_counter()
        while len(ts) < max_reps and (len(ts) < 1 or time.perf_counter() - t_all < min_seconds):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        ts.sort()
        return ts[len(ts) // 2]

    # HBM bytes per launch of the dominant kernel, from rocprofv3 FETCH_SIZE + WRITE_SIZE runs scaled by what the
    # same counters read for a plain 512 MiB copy (profiles/hbm_traffic_all_configs.txt holds the runs and their
    # commands); measured on the kernels the default build ships (tests/golden/device_code_manifest.txt pins them)
    TRAFFIC = {
        "softmax_c2": 1073780000,
        "fused_add_rms_norm_c1": 134340000,
        "fused_add_rms_norm_c1_fp32": 268600000,
        "mm_c3a_8192": 1771210000,
        "mm_c3b_skinny": 122530000,
        "addmm_c3c": 745590000,
        "flash_attn_c4": 770080000,
        "flash_attn_decode": 1075240000,
    }

    cores = torch.get_num_threads()
    from oracle import torch_ref as O  # the checker, used here only for the cpu_baseline leg

    # ------------------------------------------------------------------------------------------
    # workloads: each returns dict(run, work, bound, unit_note, cpu=(fn, sample_work, sample_note), dtype)
    # ------------------------------------------------------------------------------------------
    def wl_softmax_c2():
        g = torch.Generator(device="cpu").manual_seed(0)
        M, N = 131072, 2048
        x = torch.empty(M, N, dtype=bf16, device=dev)
        chunk = 8192
        for r in range(0, M, chunk):  # generated on the host generator in slices to bound host memory
            xs = torch.randn(chunk, N, generator=g) * 2.0
            xs[torch.rand(chunk, N, generator=g) < 0.01] = float("-inf")
            x[r:r + chunk] = xs.to(bf16).to(dev)
        state = {}

        def run(i):
            state["y"] = flag_gems.softmax(x, -1)

        sample = x[:32768].cpu()

        def cpu():
            O.softmax(sample, -1)

        return dict(run=run, work=2 * M * N * 2, bound="hbm", dtype="bf16", traffic=TRAFFIC.get("softmax_c2"),
                    workload="softmax dim=-1 [131072,2048] bf16, N(0,4) with 1% -inf (BASELINE.json configs[1])",
                    cpu=(cpu, 2 * 32768 * N * 2, "oracle softmax (torch CPU, fp64 upcast) on the first 32768 rows"))

    def wl_fused_add_rms_norm_c1(dt=bf16):
        torch.manual_seed(0)
        eb = 2 if dt is bf16 else 4
        M, N = 4096, 4096
        sets = 6 if dt is bf16 else 3  # 6 x 64 MiB (3 x 128 MiB) of x+residual: rotates through more than the 256 MB cache
        xs = [torch.randn(M, N).to(dt).to(dev) for _ in range(sets)]
        rs = [torch.randn(M, N).to(dt).to(dev) for _ in range(sets)]
        w = (torch.rand(N) + 0.5).to(dt).to(dev)

        def run(i):
            flag_gems.fused_add_rms_norm(xs[i % sets], rs[i % sets], [N], w, 1e-6)

        xc, rc, wc = torch.randn(M, N), torch.randn(M, N), torch.rand(N) + 0.5

        def cpu():
            O.fused_add_rms_norm(xc, rc, wc, 1e-6)

        return dict(run=run, work=4 * M * N * eb + N * eb, bound="hbm", dtype="bf16" if dt is bf16 else "f32",
                    traffic={2: TRAFFIC.get("fused_add_rms_norm_c1"), 4: TRAFFIC.get("fused_add_rms_norm_c1_fp32")}[eb],
                    workload="fused_add_rms_norm [4096,4096] %s, eps 1e-6 (configs[0]%s)"
                             % ("bf16" if dt is bf16 else "fp32", " shape" if dt is bf16 else ", its stated precision"),
                    cpu=(cpu, 4 * M * N * 4 + N * 4, "oracle fused_add_rms_norm (torch CPU, fp32 in / fp64 math) on the full [4096,4096]"))

    def wl_softmax_backward():
        torch.manual_seed(0)
        M, N = 131072, 2048
        y = torch.softmax(torch.randn(M, N, device=dev) * 2.0, -1).to(bf16)
        g = torch.randn(M, N, device=dev).to(bf16)
        state = {}

        def run(i):
            state["dx"] = flag_gems.softmax_backward(g, y, 1, bf16)

        ys, gs = y[:16384].cpu(), g[:16384].cpu()

        def cpu():
            O.softmax_backward(gs, ys, 1)

        return dict(run=run, work=3 * M * N * 2, bound="hbm", dtype="bf16",
                    workload="softmax backward dim=-1 [131072,2048] bf16 (grad_out, out -> grad_in)",
                    cpu=(cpu, 3 * 16384 * N * 2, "oracle softmax_backward (torch CPU, fp64 upcast) on the first 16384 rows"))

    def wl_rms_norm_backward():
        torch.manual_seed(0)
        M, N = 16384, 4096
        x = torch.randn(M, N).to(bf16).to(dev).requires_grad_(True)
        w = (torch.rand(N) + 0.5).to(bf16).to(dev).requires_grad_(True)
        dy = torch.randn(M, N).to(bf16).to(dev)
        y = flag_gems.rms_norm(x, [N], w, 1e-6)
        state = {}

        def run(i):
            state["g"] = torch.autograd.grad(y, (x, w), dy, retain_graph=True)

        xs, ds, wc = x.detach()[:2048].cpu(), dy[:2048].cpu(), w.detach().cpu()

        def cpu():
            O.rms_norm_grads(xs, wc, 1e-6, ds)

        return dict(run=run, work=3 * M * N * 2 + 2 * N * 2, bound="hbm", dtype="bf16",
                    workload="rms_norm backward [16384,4096] bf16: dx and dweight through autograd "
                             "(one kernel + the sum of its partial rows)",
                    cpu=(cpu, 3 * 2048 * N * 2, "oracle rms_norm_grads (torch CPU autograd, fp64) on the first 2048 rows"))

    def wl_mm(M, N, K, name, b_t=False, bias=False, bound="mfma", key=None):
        def make():
            torch.manual_seed(0)
            a = (torch.randn(M, K) / math.sqrt(K)).to(bf16).to(dev)
            b = ((torch.randn(N, K) / math.sqrt(K)).to(bf16).to(dev).t() if b_t
                 else (torch.randn(K, N) / math.sqrt(K)).to(bf16).to(dev))
            # a bandwidth-bound problem streams its weights: rotate through copies of B that together exceed
            # the 256 MB last-level cache, so the rate is an HBM rate (what a decoding model sees)
            copies = 1
            if bound == "hbm":
                copies = max(3, -(-320 * 2 ** 20 // (N * K * 2)))
            bs_ = [b] + [b.clone() if not b_t else b.t().clone().t() for _ in range(copies - 1)]
            bi = (torch.randn(N) * 0.02).to(bf16).to(dev) if bias else None
            state = {}

            def run(i):
                bb = bs_[i % copies]
                state["c"] = flag_gems.addmm(bi, a, bb) if bias else flag_gems.mm(a, bb)

            rows = min(M, 512)
            ac, bc = a[:rows].cpu().float(), b.cpu().float()

            def cpu():
                torch.mm(ac, bc)

            if bound == "hbm":
                work = (M * K + K * N + M * N) * 2
                cw = (rows * K + K * N + rows * N) * 2
            else:
                work = M * N * (2 * K + 1) if bias else 2 * M * N * K
                cw = 2 * rows * N * K
            d = dict(run=run, work=work, bound=bound, dtype="bf16", workload=name,
                     cpu=(cpu, cw, "torch.mm on the host in fp32, first %d rows of A" % rows))
            d["post"] = lambda: {"schedule": {1: "data-parallel", 2: "stream-K"}.get(_gemm.last_schedule())}
            d["traffic"] = TRAFFIC.get(key)
            if copies > 1:
                d["workload"] += " [B rotated through %d copies = %d MB]" % (copies, copies * N * K * 2 // 2 ** 20)
            return d
        return make

    def build_paged(lens, Hk, D, bs, k, v):
        nblk = sum((l + bs - 1) // bs for l in lens)
        perm = torch.randperm(nblk, generator=torch.Generator().manual_seed(0))
        bt = torch.zeros(len(lens), (max(lens) + bs - 1) // bs, dtype=torch.int32)
        slots, o = [], 0
        for i, l in enumerate(lens):
            n = (l + bs - 1) // bs
            bt[i, :n] = perm[o:o + n]
            o += n
            t = torch.arange(l)
            slots.append(bt[i, t // bs].long() * bs + t % bs)
        slots = torch.cat(slots).to(dev)
        kc = torch.zeros(nblk, bs, Hk, D, dtype=bf16, device=dev)
        vc = torch.zeros_like(kc)
        flag_gems.reshape_and_cache_flash(k, v, kc, vc, slots, "auto", None, None)
        return kc, vc, bt.to(dev), slots

    def wl_attn_c4():
        L = torch.randint(512, 4097, (16,), generator=torch.Generator().manual_seed(0)).tolist()
        Hq, Hk, D, bs = 32, 8, 128, 16
        tot = sum(L)
        torch.manual_seed(0)
        q = torch.randn(tot, Hq, D).to(bf16).to(dev)
        k = torch.randn(tot, Hk, D).to(bf16).to(dev)
        v = torch.randn(tot, Hk, D).to(bf16).to(dev)
        kc, vc, bt, _ = build_paged(L, Hk, D, bs, k, v)
        cu = torch.tensor([0] + L, dtype=torch.int32).cumsum(0, dtype=torch.int32).to(dev)
        sk = torch.tensor(L, dtype=torch.int32, device=dev)
        state = {}

        def run(i):
            state["o"] = flag_gems.flash_attn_varlen_func(q, kc, vc, max(L), cu, max(L), seqused_k=sk, causal=True, block_table=bt)

        flops = sum(4 * D * Hq * l * (l + 1) // 2 for l in L)
        i_short = min(range(16), key=lambda i: L[i])
        ls = L[i_short]
        off = sum(L[:i_short])
        qc = q[off:off + ls].cpu()
        kcc, vcc, btc = kc.cpu(), vc.cpu(), bt[i_short:i_short + 1].cpu()

        def cpu():
            O.paged_attention(qc, kcc, vcc, [ls], [ls], btc, D ** -0.5, compute_dtype=torch.float32)

        return dict(run=run, work=flops, bound="mfma", dtype="bf16", traffic=TRAFFIC.get("flash_attn_c4"),
                    workload="flash_attn_varlen_func causal GQA prefill, 16 seqs U[512,4096] (sum 35846), 32q/8kv heads, D 128, page 16 (configs[3])",
                    cpu=(cpu, 4 * D * Hq * ls * (ls + 1) // 2, "oracle paged attention (torch CPU fp32) on the shortest sequence (%d tokens)" % ls))

    def wl_decode():
        # single-token queries over a paged cache (the decode side of configs[3]): a stream over K and V
        B, S, Hq, Hk, D, bs = 64, 4096, 32, 8, 128, 16
        torch.manual_seed(0)
        nblk = B * (S // bs)
        bt = torch.randperm(nblk, generator=torch.Generator().manual_seed(0)).int().view(B, -1).to(dev)
        kc = torch.randn(nblk, bs, Hk, D, device=dev).to(bf16)
        vc = torch.randn(nblk, bs, Hk, D, device=dev).to(bf16)
        q = torch.randn(B, Hq, D, device=dev).to(bf16)
        cu = torch.arange(B + 1, dtype=torch.int32, device=dev)
        sk = torch.full((B,), S, dtype=torch.int32, device=dev)

        def run(i):
            flag_gems.flash_attn_varlen_func(q, kc, vc, 1, cu, S, seqused_k=sk, causal=True, block_table=bt)

        qc, kcc, vcc, btc = q[:1].cpu(), kc.cpu(), vc.cpu(), bt[:1].cpu()

        def cpu():
            O.paged_attention(qc, kcc, vcc, [1], [S], btc, D ** -0.5, compute_dtype=torch.float32)

        return dict(run=run, work=2 * B * S * Hk * D * 2 + 2 * B * Hq * D * 2, bound="hbm", dtype="bf16",
                    traffic=TRAFFIC.get("flash_attn_decode"),
                    workload="flash_attn_varlen_func decode: 64 seqs x 4096 keys, 1 query token each, 32q/8kv heads, D 128, page 16",
                    cpu=(cpu, 2 * S * Hk * D * 2, "oracle paged attention (torch CPU fp32) on one sequence"))

    def wl_mixed():
        # what a serving engine with chunked prefill sends in one call: many decoding sequences and a few prefill chunks
        Hq, Hk, D, bs = 32, 8, 128, 16
        rng = random.Random(0)
        lens = [(1, rng.randint(2048, 4096)) for _ in range(60)] + [(512, 512 + 1024 * i) for i in range(4)]
        qlens, klens = [l[0] for l in lens], [l[1] for l in lens]
        nblk = sum((k + bs - 1) // bs for k in klens)
        torch.manual_seed(0)
        q = torch.randn(sum(qlens), Hq, D, device=dev).to(bf16)
        kc = torch.randn(nblk, bs, Hk, D, device=dev).to(bf16)
        vc = torch.randn(nblk, bs, Hk, D, device=dev).to(bf16)
        cu = torch.tensor([0] + qlens, dtype=torch.int32).cumsum(0, dtype=torch.int32).to(dev)
        sk = torch.tensor(klens, dtype=torch.int32, device=dev)
        perm = torch.randperm(nblk, generator=torch.Generator().manual_seed(0))
        bt = torch.zeros(len(lens), (max(klens) + bs - 1) // bs, dtype=torch.int32)
        o = 0
        for i, k in enumerate(klens):
            n = (k + bs - 1) // bs
            bt[i, :n] = perm[o:o + n]
            o += n
        bt = bt.to(dev)

        def run(i):
            flag_gems.flash_attn_varlen_func(q, kc, vc, max(qlens), cu, max(klens), seqused_k=sk, causal=True, block_table=bt)

        qc, kcc, vcc, btc = q[:1].cpu(), kc.cpu(), vc.cpu(), bt[:1].cpu()

        def cpu():
            O.paged_attention(qc, kcc, vcc, [1], [klens[0]], btc, D ** -0.5, compute_dtype=torch.float32)

        kv_bytes = 2 * sum(klens) * Hk * D * 2  # every K and V row once per KV head
        return dict(run=run, work=kv_bytes + 2 * sum(qlens) * Hq * D * 2, bound="hbm", dtype="bf16",
                    workload="flash_attn_varlen_func mixed batch: 60 decoding sequences of 2048-4096 keys + 4 prefill chunks of "
                             "512 tokens behind 0-3072 cached keys, 32q/8kv heads, D 128, page 16 (bytes: K/V once per KV head)",
                    cpu=(cpu, 2 * klens[0] * Hk * D * 2, "oracle paged attention (torch CPU fp32) on the first sequence"))

    def wl_sdpa():
        # dense causal attention through scaled_dot_product_attention (the caller's (batch, heads, seq, d) tensors
        # are used in place as a virtual paged cache)
        B, H, Hk, S, D = 8, 32, 8, 4096, 128
        torch.manual_seed(0)
        q = torch.randn(B, H, S, D, device=dev).to(bf16)
        k = torch.randn(B, Hk, S, D, device=dev).to(bf16)
        v = torch.randn(B, Hk, S, D, device=dev).to(bf16)

        def run(i):
            flag_gems.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)

        rows = 64
        qc, kc_, vc_ = q[:1, :, S - rows:].transpose(1, 2).cpu(), k[:1].transpose(1, 2).cpu(), v[:1].transpose(1, 2).cpu()

        def cpu():
            O.dense_attention(qc, kc_, vc_, D ** -0.5, causal=True)

        return dict(run=run, work=4 * D * H * B * S * (S + 1) // 2, bound="mfma", dtype="bf16",
                    workload="scaled_dot_product_attention causal, batch 8 x 4096 tokens, 32q/8kv heads, D 128",
                    cpu=(cpu, 4 * D * H * rows * S, "oracle dense attention (torch CPU fp32), last %d query rows of one sequence" % rows))

    def wl_layer_c5():
        torch.manual_seed(0)
        Hd, H, D, F, bs, B, S = 4096, 32, 128, 11008, 16, 8, 2048
        T = B * S
        wqkv = (torch.randn(3 * Hd, Hd) * 0.02).to(bf16).to(dev)
        wo = (torch.randn(Hd, Hd) * 0.02).to(bf16).to(dev)
        wgu = (torch.randn(2 * F, Hd) * 0.02).to(bf16).to(dev)
        wd = (torch.randn(Hd, F) * 0.02).to(bf16).to(dev)
        n1 = torch.ones(Hd, dtype=bf16, device=dev)
        n2 = torch.ones(Hd, dtype=bf16, device=dev)
        h = torch.randn(T, Hd).to(bf16).to(dev)
        pos = torch.arange(S).repeat(B).to(dev)
        cos, sin = O.rope_cos_sin(S, D, device=dev)
        lens = [S] * B
        zk = torch.zeros(T, H, D, dtype=bf16, device=dev)
        kc, vc, bt, slots = build_paged(lens, H, D, bs, zk, zk)
        del zk
        cu = torch.arange(0, T + 1, S, dtype=torch.int32, device=dev)
        sk = torch.full((B,), S, dtype=torch.int32, device=dev)
        lib = torch.library.Library("aten", "IMPL")
        flag_gems.enable(lib=lib)
        marks = []

        def run(i, record=None):
            def mark(name):
                if record is not None:
                    e = torch.cuda.Event(enable_timing=True)
                    e.record()
                    record.append((name, e))
            mark("start")
            x = torch.nn.functional.rms_norm(h, [Hd], n1, 1e-5); mark("rms_norm")
            qkv = torch.mm(x, wqkv.t()); mark("mm_qkv")
            q, k, v = (qkv[:, j * Hd:(j + 1) * Hd].view(T, H, D) for j in range(3))
            flag_gems.apply_rotary_pos_emb(q, k, cos, sin, pos, False, inplace=True); mark("rope")
            flag_gems.reshape_and_cache_flash(k, v, kc, vc, slots, "auto", None, None); mark("reshape_and_cache_flash")
            a = flag_gems.flash_attn_varlen_func(q, kc, vc, S, cu, S, seqused_k=sk, causal=True, block_table=bt); mark("flash_attn_varlen")
            o = torch.mm(a.view(T, Hd), wo.t()); mark("mm_o")
            y, r = flag_gems.fused_add_rms_norm(o, h.clone(), [Hd], n2, 1e-5); mark("fused_add_rms_norm(+clone)")
            gu = torch.mm(y, wgu.t()); mark("mm_gate_up")
            act = flag_gems.silu_and_mul(gu[:, :F], gu[:, F:]); mark("silu_and_mul")
            out = torch.mm(act, wd.t()); mark("mm_down")
            out += r; mark("residual_add")
            return out

        lin = 2 * T * Hd * (3 * Hd + Hd + 2 * F + F)
        att = B * 4 * D * H * S * (S + 1) // 2
        e2 = 2  # bytes per element
        # algorithmic work of every operator of the layer: (bound, flop or bytes)
        op_work = {
            "rms_norm": ("hbm", 2 * T * Hd * e2 + Hd * e2),
            "mm_qkv": ("mfma", 2 * T * Hd * 3 * Hd),
            "rope": ("hbm", 2 * 2 * T * Hd * e2),
            "reshape_and_cache_flash": ("hbm", 2 * 2 * T * Hd * e2),
            "flash_attn_varlen": ("mfma", att),
            "mm_o": ("mfma", 2 * T * Hd * Hd),
            "fused_add_rms_norm(+clone)": ("hbm", (4 + 2) * T * Hd * e2 + Hd * e2),
            "mm_gate_up": ("mfma", 2 * T * Hd * 2 * F),
            "silu_and_mul": ("hbm", 3 * T * F * e2),
            "mm_down": ("mfma", 2 * T * F * Hd),
            "residual_add": ("hbm", 3 * T * Hd * e2),
        }

        def post():
            reps = 3
            acc = {}
            for _ in range(reps):
                rec = []
                run(0)  # a layer ahead in the queue, so that no marked operator waits for its own launch
                run(0, rec)
                torch.cuda.synchronize()
                for (n0, e0), (n1_, e1) in zip(rec[:-1], rec[1:]):
                    acc.setdefault(n1_, []).append(e0.elapsed_time(e1))
            ops = {n: round(sorted(v)[len(v) // 2], 4) for n, v in acc.items()}
            per_op = {n: roofline(op_work[n][0], op_work[n][1], ms) for n, ms in ops.items()}
            lib._destroy()
            return {"per_op_ms": ops, "per_op_roofline": per_op, "linear_flop": lin, "attention_flop": att}

        # CPU baseline: the fp32 layer oracle on the first 256 tokens of one sequence
        cs = 256
        hc, posc = h[:cs].cpu(), pos[:cs].cpu()
        wc = [w.cpu() for w in (wqkv, wo, wgu, wd, n1, n2)]
        cosc, sinc = cos.cpu(), sin.cpu()

        def cpu():
            O.decoder_layer(hc, wc[0], wc[1], wc[2], wc[3], wc[4], wc[5], posc, cosc, sinc, 1e-5, H)

        cwork = 2 * cs * Hd * (3 * Hd + Hd + 2 * F + F) + 4 * D * H * cs * (cs + 1) // 2
        return dict(run=run, work=lin + att, bound="mfma", dtype="bf16",
                    workload="Llama-2-7B decoder layer forward under flag_gems.enable(), 8 x 2048-token prefill, paged KV (configs[4])",
                    cpu=(cpu, cwork, "layer oracle (torch CPU fp32, per-operator bf16 rounding) on the first %d tokens of one sequence" % cs),
                    post=post)

    def wl_copy_ref():
        # plain device copy of known size (torch's elementwise copy kernel): the yardstick the
        # FETCH_SIZE / WRITE_SIZE counters are scaled by; not part of the operator path
        x = torch.randn(131072, 2048, device=dev).to(bf16)
        y = torch.empty_like(x)

        def run(i):
            y.copy_(x)

        return dict(run=run, work=2 * x.numel() * 2, bound="hbm", dtype="bf16",
                    workload="reference: torch copy of a [131072,2048] bf16 tensor (512 MiB read + 512 MiB written)", cpu=None)

    def wl_mfma_ceiling(random_operands):
        # calibration, not an operator: the rate the matrix cores sustain on nothing but MFMA 16x16x32
        # bf16 (the GEMM kernels' instruction), with operand fragments of zeros or of N(0,1) values.  The chip is power-limited, so the
        # second figure -- not the 2.5 PFLOP/s of the data sheet -- is what a real bf16 GEMM can approach.
        import ctypes
        from flaggems_amd import _C
        src = (torch.randn(8 * 256 * 8, device=dev) if random_operands else torch.zeros(8 * 256 * 8, device=dev)).to(bf16)
        blocks, iters = 1024, 2048
        out = torch.empty(blocks * 256, device=dev)
        flops = ctypes.c_double(0.0)

        def run(i):
            _C.check(_C.lib().fg_mfma_probe(src.data_ptr(), out.data_ptr(), blocks, iters, ctypes.byref(flops),
                                            torch.cuda.current_stream().cuda_stream), "fg_mfma_probe")

        run(0)
        return dict(run=run, work=flops.value, bound="mfma", dtype="bf16",
                    workload="calibration: MFMA-only loop, %s operands (sustained matrix-core rate under the power limit)"
                    % ("N(0,1)" if random_operands else "all-zero"), cpu=None)

    workloads = {
        "softmax_c2": wl_softmax_c2,
        "fused_add_rms_norm_c1": wl_fused_add_rms_norm_c1,
        "fused_add_rms_norm_c1_fp32": lambda: wl_fused_add_rms_norm_c1(torch.float32),
        "softmax_backward": wl_softmax_backward,
        "rms_norm_backward": wl_rms_norm_backward,
        "mm_c3a_8192": wl_mm(8192, 8192, 8192, "mm bf16 M=N=K=8192, B row-major (configs[2]a)", key="mm_c3a_8192"),
        "mm_c3a_8192_nt": wl_mm(8192, 8192, 8192, "mm bf16 M=N=K=8192, B = W^T column-major (configs[2]a, weight layout)", b_t=True),
        "mm_c3b_skinny": wl_mm(16, 4096, 14336, "mm bf16 M=16 N=4096 K=14336, stream-K (configs[2]b)", bound="hbm",
                               key="mm_c3b_skinny"),
        "mm_c3b_skinny_nt": wl_mm(16, 4096, 14336, "mm bf16 M=16 N=4096 K=14336, B = W^T of a [N, K] weight, stream-K",
                                  b_t=True, bound="hbm"),
        "mm_chunk_1024_nt": wl_mm(1024, 12288, 4096, "mm bf16 M=1024 N=12288 K=4096, B = W^T (a 1024-token prefill chunk "
                                  "through a fused QKV weight: less than one round of 256x256 tiles)", b_t=True),
        "mm_chunk_512_nt": wl_mm(512, 4096, 4096, "mm bf16 M=512 N=4096 K=4096, B = W^T (half a round of 128x128 tiles: "
                                 "each tile cut in two)", b_t=True),
        "addmm_c3c": wl_mm(4096, 11008, 4096, "addmm bf16 M=4096 N=11008 K=4096 + bias (configs[2]c)", bias=True,
                           key="addmm_c3c"),
        "flash_attn_c4": wl_attn_c4,
        "flash_attn_decode": wl_decode,
        "flash_attn_mixed": wl_mixed,
        "sdpa_dense": wl_sdpa,
        "decoder_layer_c5": wl_layer_c5,
        "mfma_ceiling_random": lambda: wl_mfma_ceiling(True),
        "mfma_ceiling_zeros": lambda: wl_mfma_ceiling(False),
        "copy_ref": wl_copy_ref,
    }
    if args.workload not in workloads:
        print("bench.py: unknown workload %s (have: %s)" % (args.workload, ", ".join(workloads)), file=sys.stderr)
        sys.exit(2)

    def measure(name, steps, warmup, with_cpu):
        w = workloads[name]()
        wall_ms, ev_ms = timed(w["run"], steps, warmup)
        res = {"workload": w["workload"], "ms_per_step": round(wall_ms, 5), "kernel_ms": round(ev_ms, 5),
               "roofline": roofline(w["bound"], w["work"], ev_ms, w.get("traffic"))}
        if w["bound"] == "hbm":
            res["value"], res["unit"] = round(w["work"] / wall_ms / 1e6, 1), "GB/s"
        else:
            res["value"], res["unit"] = round(w["work"] / wall_ms / 1e9, 1), "TFLOP/s"
        if "post" in w and w["post"] is not None:
            res.update(w["post"]())
        if with_cpu and w.get("cpu"):
            fn, cwork, note = w["cpu"]
            t = cpu_time(fn)
            if w["bound"] == "hbm":
                res["cpu_baseline"] = {"value": round(cwork / t / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port", "sample": note}
            else:
                res["cpu_baseline"] = {"value": round(cwork / t / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port", "sample": note}
        del w
        torch.cuda.empty_cache()
        return res

    head = measure(args.workload, args.steps, args.warmup, not args.no_cpu)
    extra = {}
    if not args.no_extra:
        for name in workloads:
            if name == args.workload or name == "copy_ref":
                continue
            steps = max(3, min(args.steps, 20))
            if name == "decoder_layer_c5":
                steps = min(steps, 5)
            extra[name] = measure(name, steps, min(args.warmup, 3), not args.no_cpu)

    line = {
        "metric": "% of roofline: GB/s for norm/softmax, TFLOP/s for mm/flash-attn, 1xMI355X",
        "value": head["value"],
        "unit": head["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": args.settle_ms,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": head["workload"]},
        "roofline": head["roofline"],
        "cpu_baseline": head.get("cpu_baseline"),
        "configs": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

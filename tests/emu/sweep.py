"""Small cases in bulk, chosen to reach the kernel instantiations the library can launch: one per dispatch bucket
(row length, alignment, dtype pair, mode) of the row-wise operators, per tile and layout of the GEMM kernels, per
copy width of the cache scatter, per table dtype of the rotation.  Plain data: dictionaries for worker.py."""
VEC = {"bf16": 8, "f16": 8, "f32": 4}
FLOATS = ("bf16", "f16", "f32")
PACKS = (40, 100, 200, 400, 800, 1600, 3000, 6000)      # one row length per bucket of 16-byte packs


def sweep():
    out = []

    def add(fn, check=None, env=None, num_cu=256, **kw):
        label = " ".join("%s=%s" % (k, kw[k]) for k in sorted(kw))
        if env:
            label += " " + " ".join("%s=%s" % kv for kv in sorted(env.items()))
        out.append({"id": "sweep %s %s%s" % (fn, label, "" if num_cu == 256 else " on %d CUs" % num_cu), "fn": fn, "kw": kw,
                    "seed": len(out), "check": check or fn, "env": env or {}, "num_cu": num_cu})

    for dt in FLOATS:
        for p in PACKS:
            add("rms_norm", dtype=dt, M=2, N=p * VEC[dt])
            add("fused_add_rms_norm", dtype=dt, M=3, N=p * VEC[dt])
        for n in (33, 101, 201, 401):                      # element-aligned short rows
            add("rms_norm", dtype=dt, M=5, N=n)
            add("fused_add_rms_norm", dtype=dt, M=5, N=n)
        for p in (200, 400, 800):                          # a single row keeps the one-row-per-workgroup kernel
            add("fused_add_rms_norm", dtype=dt, M=1, N=p * VEC[dt])
        for n in (1001, 3001):                             # two-pass kernels
            add("rms_norm", dtype=dt, M=2, N=n)
            add("fused_add_rms_norm", dtype=dt, M=2, N=n)
    pairs = (("bf16", "bf16"), ("f16", "f16"), ("f32", "f32"), ("bf16", "f32"), ("f16", "f32"))
    for dt, odt in pairs:
        for log in (False, True):
            for p in PACKS:
                add("softmax", dtype=dt, out_dtype=odt, M=2, N=p * VEC[dt], K=1, log=log)
            for n in (33, 101, 201, 401, 1001):
                add("softmax", dtype=dt, out_dtype=odt, M=5, N=n, K=1, log=log)
            for n in (3001, 70001):
                add("softmax", dtype=dt, out_dtype=odt, M=2, N=n, K=1, log=log)
            add("softmax", dtype=dt, out_dtype=odt, M=2, N=37, K=50, log=log)
    # backward of softmax / log_softmax: (out dtype, grad_in dtype) pairs mirror the forward's
    for dt, gdt in (("bf16", "bf16"), ("f16", "f16"), ("f32", "f32"), ("f32", "bf16"), ("f32", "f16")):
        for log in (False, True):
            for p in (40, 100, 200, 400, 800, 1600, 3000):
                add("softmax_backward", dtype=dt, grad_in_dtype=gdt, M=2, N=p * VEC[dt], K=1, log=log)
            for n in (33, 101, 201, 401):
                add("softmax_backward", dtype=dt, grad_in_dtype=gdt, M=5, N=n, K=1, log=log)
            for n in (1001, 3001):
                add("softmax_backward", dtype=dt, grad_in_dtype=gdt, M=2, N=n, K=1, log=log)
            add("softmax_backward", dtype=dt, grad_in_dtype=gdt, M=2, N=37, K=50, log=log)
    for dt in FLOATS:
        for p in (40, 100, 200, 400, 800, 1600):
            add("rms_norm_backward", dtype=dt, M=5, N=p * VEC[dt])
        for p in (40, 100, 200, 400, 800):                 # without the weight gradient: one row per group
            add("rms_norm_backward", dtype=dt, M=3, N=p * VEC[dt], dw=False)
        add("rms_norm_backward", dtype=dt, M=3, N=301)
        add("rms_norm_backward", dtype=dt, M=4, N=64 * VEC[dt], weight=False)
    # rotation: element type x table type x (16-byte packs | single elements) x pairing
    for dt in FLOATS:
        for cdt in FLOATS:
            for inter in (False, True):
                add("rope", dtype=dt, cs_dtype=cdt, n_tokens=3, Hq=2, Hk=1, D=64, interleaved=inter)
                add("rope", dtype=dt, cs_dtype=cdt, n_tokens=3, Hq=2, Hk=1, D=20, interleaved=inter, head_pad=1)
    # cache scatter: copy width from the row bytes (16, 8, 4, 2, 1) x slot type
    for i64 in (True, False):
        for eb, hd in ((2, 64), (2, 36), (2, 34), (2, 33), (1, 33)):
            add("reshape_and_cache_flash", elem_bytes=eb, num_tokens=5, H=1, D=hd, block_size=4, num_blocks=3, slot_i64=i64)
    # GEMM fed by LDS-DMA: every tile, both B layouts, both 16-bit types; K not a multiple of 64; the epilogue with a bias
    for dt in ("bf16", "f16"):
        for layout in ("nk", "kn"):
            for bm, bn in ((256, 256), (192, 256), (256, 128), (128, 256), (128, 128)):
                add("gemm", dtype=dt, M=bm + 8, N=bn + 8, K=192, b_layout=layout, env={"FG_GEMM_TILE": "%dx%d" % (bm, bn)})
            for bm, bn in ((256, 256), (128, 128)):
                add("gemm", dtype=dt, M=bm + 8, N=bn, K=200, b_layout=layout, bias="row", env={"FG_GEMM_TILE": "%dx%d" % (bm, bn)})
            add("gemm", dtype=dt, M=384, N=256, K=512, b_layout=layout, schedule=2, num_cu=8)     # stream-K, every tile shared
            add("gemm", dtype=dt, M=768, N=256, K=512, b_layout=layout, schedule=2, num_cu=8)     # a data-parallel wave in front
            add("gemm", dtype=dt, M=512, N=512, K=200, b_layout=layout, num_cu=4)                 # 256x256 tiles, ragged K
    # skinny GEMM: 16- and 32-column tiles, 1 to 4 row blocks, with and without a bias
    for dt in ("bf16", "f16"):
        for tile in ("16", "32"):
            for m in (4, 12, 24):
                add("gemm", dtype=dt, M=m, N=96, K=1024, b_layout="nk", env={"FG_SKINNY_TILE": tile}, num_cu=8)
        add("gemm", dtype=dt, M=48, N=96, K=1024, b_layout="nk", num_cu=8)
        add("gemm", dtype=dt, M=8, N=64, K=1024, b_layout="kn", num_cu=8)
        add("gemm", dtype=dt, M=8, N=64, K=1030, b_layout="nk", num_cu=8)
    # attention: the pipelined prefill kernel and the single-token kernel, both head dims and types
    for dt in ("bf16", "f16"):
        for d in (64, 128):
            add("attention", dtype=dt, q_lens=[40, 9], k_lens=[150, 9], Hq=2, Hk=1, D=d, page_size=16)
            add("attention", dtype=dt, q_lens=[1, 1], k_lens=[150, 40], Hq=4, Hk=2, D=d, page_size=16)
    return out

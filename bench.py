#!/usr/bin/env python3
"""Benchmark of the MLA paged-decode hot path on one MI355X.

A step is one GGML_OP_FLASH_ATTN_EXT node of the DeepSeek-V2 shape through the C ABI (split-K decode kernel +
combine pass): batch 32, 128 heads, every context 8192 tokens, bf16 latent KV (576-d QK, 512-d V) in 128-token
pages behind a shuffled block table, Q ~ N(0,1), K ~ N(0,0.5).  Inputs are resident in HBM before the timed region.
The KV pool is rotated between steps (several distinct pools) so that reads are HBM traffic, not Infinity-Cache hits.

Prints ONE JSON line:  value = algorithmic KV bytes per step / step time, in GB/s (whole job, one GPU).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 / fp16 MFMA rate
KV_ROW_BYTES = 1152     # 576 bf16
FLOP_PER_TOKEN_HEAD = 2 * 576 + 2 * 512
# the commit and date at which profiles/mla_decode_kernel_c3_pmc.md's FETCH_SIZE / WRITE_SIZE readings (the `traffic` constants below) were taken
TRAFFIC_PROFILE_COMMIT = ("f539b15", "2026-11-26")


def build_workload(dev, n_seq, n_head, ctx, n_pools, seed, kv="bf16"):
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    pages_per_seq = ctx // 128
    n_pages = n_seq * pages_per_seq
    pools = []
    for _ in range(n_pools):
        kf = torch.randn((n_pages * 128, 576), generator=g, device=dev, dtype=torch.float32) * 0.5
        pools.append(kf.to(torch.bfloat16 if kv == "bf16" else torch.float16))
        del kf
    perm = torch.randperm(n_pages, generator=g, device=dev).to(torch.int32)
    block_table = perm.reshape(n_seq, pages_per_seq).contiguous()
    seq_lens = torch.full((n_seq,), ctx, dtype=torch.int32, device=dev)
    q = torch.randn((n_seq, n_head, 1, 576), generator=g, device=dev, dtype=torch.float32)
    return q, pools, block_table, seq_lens


def build_paged(dev, lens, n_head, n_tok, kv, seed):
    """Pages for sequences of the given lengths behind a shuffled block table (BASELINE configs 2, 4, 5)."""
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    nblk = [(l + 127) // 128 for l in lens]
    n_pages = sum(nblk)
    perm = torch.randperm(n_pages, generator=g, device=dev).to(torch.int32)
    bt = torch.zeros((len(lens), max(nblk)), dtype=torch.int32, device=dev)
    pos = 0
    for b, n in enumerate(nblk):
        bt[b, :n] = perm[pos:pos + n]
        pos += n
    if kv == "q8_0":
        # int8 = clip(round(N(0,1) / scale)), one fp16 scale 1/32 per block (BASELINE config 5)
        qs = torch.clamp(torch.round(torch.randn((n_pages * 128, 18, 32), generator=g, device=dev) * 32.0), -127, 127).to(torch.int8)
        pool = torch.empty((n_pages * 128, 18, 34), dtype=torch.uint8, device=dev)
        pool[:, :, 0] = 0x00
        pool[:, :, 1] = 0x28   # fp16 0x2800 = 1/32
        pool[:, :, 2:] = qs.view(torch.uint8)
        pool = pool.reshape(n_pages * 128, 612)
    else:
        pool = torch.randn((n_pages * 128, 576), generator=g, device=dev).to(torch.bfloat16 if kv == "bf16" else torch.float16).view(torch.int16)
    q = torch.randn((len(lens), n_head, n_tok, 576), generator=g, device=dev, dtype=torch.float32)
    return q, pool, bt, torch.tensor(lens, dtype=torch.int32, device=dev)


def kv_write_config(a, dev, lib, J):
    """The latent-KV cache write (include/mla_kv_write.h) on 65536 new rows through a block table: f32 rows in, cache rows
    out.  Algorithmic bytes per row: 2304 read + 1152 (bf16/f16) or 612 (Q8_0) written."""
    import torch
    n_tok, n_seq = 65536, 32
    kvt = {"bf16": J.MLA_TYPE_BF16, "f16": J.MLA_TYPE_F16, "q8_0": J.MLA_TYPE_Q8_0}[a.kv]
    row = 612 if a.kv == "q8_0" else 1152
    g = torch.Generator(device=dev)
    g.manual_seed(a.seed)
    x = torch.randn((n_tok, 576), generator=g, device=dev, dtype=torch.float32)
    pages = n_tok // 128
    cache = torch.zeros((pages * 128, row), dtype=torch.uint8, device=dev)
    bt = torch.randperm(pages, generator=g, device=dev).to(torch.int32).reshape(n_seq, pages // n_seq).contiguous()
    order = torch.randperm(n_tok, generator=g, device=dev)
    seq_ids = (order // (n_tok // n_seq)).to(torch.int32).contiguous()
    positions = (order % (n_tok // n_seq)).to(torch.int32).contiguous()
    stream = torch.cuda.current_stream(dev)

    def run(n):
        for _ in range(n):
            J.kv_write(x, cache, kvt, block_table=bt, seq_ids=seq_ids, positions=positions)

    run(a.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run(a.steps)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / a.steps
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    run(a.steps)
    e1.record(stream)
    torch.cuda.synchronize()
    kern_ms = e0.elapsed_time(e1) / a.steps
    nbytes = n_tok * (2304 + row)
    print(json.dumps({"metric": "mla_kv_cache_write_bandwidth", "value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1,
                      "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
                      "vs_baseline": None, "dtype": a.kv, "data": "synthetic",
                      "config": {"workload": "KV cache write: 65536 f32 rows of 576 -> %s cache rows through a block table (32 sequences, shuffled pages and arrival order)" % a.kv},
                      "us_per_step": ms * 1e3,
                      "roofline": {"bound": "hbm", "kernel": "mla_kv_write_kernel", "achieved": nbytes / (kern_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                                   "unit": "GB/s", "frac": nbytes / (kern_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "traffic": None,
                                   "algorithmic_bytes_per_launch": nbytes, "kernel_us": {"mean": kern_ms * 1e3}},
                      "cpu_baseline": None}))


def front_config(a, dev, lib, J):
    """The nodes either side of the attention node (include/mla_front.h) at the headline model shape (128 heads):
    absorb = q_nope [128] x wk_b [128 x 512] per head, unabsorb = wv_b [512 x 128] x kqv [512] per head, rope = q_pe
    [64] per head.  --tokens 32 is a decode step of 32 sequences (bound by the 16.8 MB weight stream: wkv_b of 32
    different layers is rotated so that it comes from HBM), --tokens 2048 a prefill chunk (bound by the matrix cores)."""
    import torch
    H, T, layers = a.heads, a.tokens, 32
    g = torch.Generator(device=dev)
    g.manual_seed(a.seed)
    stream = torch.cuda.current_stream(dev)
    if a.config == "rope":
        x = torch.randn((T, H, 64), generator=g, device=dev, dtype=torch.float32)
        pos = torch.randint(0, 163840, (T,), generator=g, device=dev, dtype=torch.int32)
        out = torch.empty_like(x)
        fn = lambda i: J.ggml_rope_ext(x, pos, n_dims=64, n_ctx_orig=4096, freq_scale=0.025, ext_factor=1.0, attn_factor=0.8, out=out)
        nbytes, flops, kernel = x.numel() * 8, 0, "mla_rope_kernel"
        what = "rotary embedding (YaRN) of q_pe: %d tokens x %d heads x 64" % (T, H)
    else:
        K, N = (128, 512) if a.config == "absorb" else (512, 128)
        w = (torch.randn((layers, H, N, K), generator=g, device=dev, dtype=torch.float32) * 0.05).to(torch.bfloat16).view(torch.int16)
        x = torch.randn((H, T, K), generator=g, device=dev, dtype=torch.float32)
        out = torch.empty((H, T, N), device=dev, dtype=torch.float32)
        fn = lambda i: J.ggml_mul_mat(w[i % layers], J.MLA_TYPE_BF16, x, out=out)
        nbytes, flops = H * N * K * 2 + x.numel() * 4 + out.numel() * 4, 2 * H * T * N * K
        kernel = "mla_mul_mat_kernel"
        what = "%s product: %d heads x [%d tokens x %d] x [%d x %d] bf16 weights (one of %d layers per step)" % (a.config, H, T, K, K, N, layers)

    def run(n):
        for i in range(n):
            fn(i)

    run(a.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run(a.steps)
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3 / a.steps
    # one launch per step: eager steps are bound by the host's launch rate, so the K steps are also replayed from a HIP graph
    side = torch.cuda.Stream(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        graph.capture_begin()
        run(a.steps)
        graph.capture_end()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    graph.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / a.steps
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    graph.replay()
    e1.record(stream)
    torch.cuda.synchronize()
    kern_ms = e0.elapsed_time(e1) / a.steps
    hbm_time, mfma_time = nbytes / (HBM_PEAK_GBPS * 1e9), flops / (MFMA_BF16_PEAK_TFLOPS * 1e12)
    if mfma_time > hbm_time:
        ach = flops / (kern_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "kernel": kernel, "achieved": ach, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": ach / MFMA_BF16_PEAK_TFLOPS}
        metric, value, unit = "mla_%s_mfma_rate" % a.config, flops / (ms * 1e-3) / 1e12, "TFLOP/s"
    else:
        ach = nbytes / (kern_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "kernel": kernel, "achieved": ach, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBPS}
        metric, value, unit = "mla_%s_bandwidth" % a.config, nbytes / (ms * 1e-3) / 1e9, "GB/s"
    roof.update({"traffic": None, "algorithmic_bytes_per_launch": nbytes, "flops_per_launch": flops, "kernel_us": {"mean": kern_ms * 1e3}})
    cpu = None
    if a.cpu_seqs > 0:
        # the same node on the host cores: the reference's compiled ggml-cpu when oracle/_ref is built, else the C restatement
        from oracle import oracle as O
        cores = min(os.cpu_count() or 1, 16)
        if a.config == "rope":
            xs, ps = x.cpu().numpy(), pos.cpu().numpy()
            prm = O.rope_params(freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)
            f = (lambda: O.ref_rope(xs, ps, prm, n_threads=cores)) if O.ref_available() else (lambda: O.rope(xs, ps, prm))
            sample, frac = "the whole workload", 1.0
        else:
            hs = min(H, 8)
            ws, xs = w[0, :hs].cpu().numpy().view("uint16"), x[:hs].cpu().numpy()
            f = (lambda: O.ref_mul_mat(ws, O.TYPE_BF16, xs, n_threads=cores)) if O.ref_available() else (lambda: O.mul_mat(ws, O.TYPE_BF16, xs))
            sample, frac = "%d of the %d heads" % (hs, H), hs / H
        f()
        best = min(_timed(f) for _ in range(3))
        cpu = {"value": nbytes * frac / best / 1e9, "unit": "GB/s", "cores": cores if O.ref_available() else 1,
               "kind": "reference" if O.ref_available() else "port", "sample": sample, "seconds": best}
    print(json.dumps({"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
                      "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
                      "dtype": "f32" if a.config == "rope" else "bf16", "data": "synthetic", "config": {"workload": what},
                      "us_per_step": ms * 1e3, "eager_us_per_step": eager_ms * 1e3, "launch": "hip graph replay of the K steps",
                      "roofline": roof, "cpu_baseline": cpu}))


def layer_config(a, dev, lib, J):
    """One decode step of one attention layer between the q / kv projections and wo, every node through the C ABI:
    rope(q_pe) and the absorb product written straight into the 576-wide Q rows, rope(k_pe) and the cache write through
    the block table (these in one dispatch, k_pe rotated on its way into the cache; --front separate: a launch each, k_pe
    rotated in place), paged attention, the un-absorb product written straight into the [token, head*128] rows.
    Config 3's shape (32 sequences, 128 heads, 8191 cached tokens + the new one); wkv_b and the KV pool of 4 layers are
    rotated between steps."""
    import torch
    B, H, ctx, layers = a.batch, a.heads, a.ctx, a.pools
    scale = 1.0 / (192.0 ** 0.5)
    _, pools, bt, sl = build_workload(dev, B, H, ctx, layers, a.seed, "bf16")
    g = torch.Generator(device=dev)
    g.manual_seed(a.seed + 1)
    wkv_b = (torch.randn((layers, H * 256 * 512), generator=g, device=dev, dtype=torch.float32) * 0.05).to(torch.bfloat16).view(torch.int16)
    q = torch.randn((B, H, 192), generator=g, device=dev, dtype=torch.float32)
    kv_new = torch.randn((B, 576), generator=g, device=dev, dtype=torch.float32) * 0.5
    pos = torch.full((B,), ctx - 1, dtype=torch.int32, device=dev)
    seq_ids = torch.arange(B, dtype=torch.int32, device=dev)
    q_states = torch.empty((H, B, 576), dtype=torch.float32, device=dev)
    attn_out = torch.empty((B, 1, H, 576), dtype=torch.float32, device=dev)
    cur = torch.empty((B, H, 128), dtype=torch.float32, device=dev)
    rope_kw = dict(n_dims=64, n_ctx_orig=4096, freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)
    k_pe = kv_new[:, 512:].unsqueeze(1)                                  # [B, 1, 64] inside the rows of 576
    attn_args = []
    for pool in pools:
        ar, _, keep = J.capi.make_args(q_states.permute(1, 0, 2).unsqueeze(2), pool.view(torch.int16), J.MLA_TYPE_BF16, dv=512,
                                       scale=scale, block_table=bt, seq_lens=sl, out=attn_out)
        attn_args.append((ar, keep))

    def step(i, st):
        w = wkv_b[i % layers]
        pool = pools[i % layers].view(torch.int16)
        if a.front == "batch":
            # the three independent nodes ahead of the attention node in one dispatch; k_pe is rotated on its way into the cache
            fb = J.FrontBatch()
            J.ggml_rope_ext(q[:, :, 128:], pos, out=q_states[:, :, 512:].permute(1, 0, 2), batch=fb, **rope_kw)
            J.ggml_mul_mat(w[:H * 512 * 128].view(H, 512, 128), J.MLA_TYPE_BF16, q[:, :, :128].permute(1, 0, 2), out=q_states[:, :, :512], batch=fb)
            J.kv_write(kv_new, pool, J.MLA_TYPE_BF16, block_table=bt, seq_ids=seq_ids, positions=pos, k_pe=kv_new[:, 512:],
                       rope=dict(pos=pos, **rope_kw), batch=fb)
            fb.launch(stream=st.value)
        else:
            J.ggml_rope_ext(q[:, :, 128:], pos, out=q_states[:, :, 512:].permute(1, 0, 2), **rope_kw)
            J.ggml_rope_ext(k_pe, pos, out=k_pe, **rope_kw)
            J.ggml_mul_mat(w[:H * 512 * 128].view(H, 512, 128), J.MLA_TYPE_BF16, q[:, :, :128].permute(1, 0, 2), out=q_states[:, :, :512])
            J.kv_write(kv_new, pool, J.MLA_TYPE_BF16, block_table=bt, seq_ids=seq_ids, positions=pos)
        rc = lib.mla_attn_launch(C.byref(attn_args[i % layers][0]), st)
        if rc != 0:
            raise RuntimeError("launch failed: %d" % rc)
        J.ggml_mul_mat(w[H * 512 * 128:].view(H, 128, 512), J.MLA_TYPE_BF16, attn_out[:, 0].permute(1, 0, 2)[:, :, :512], out=cur.permute(1, 0, 2))

    stream = torch.cuda.current_stream(dev)
    for i in range(a.warmup):
        step(i, C.c_void_p(stream.cuda_stream))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(i, C.c_void_p(stream.cuda_stream))
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3 / a.steps
    side = torch.cuda.Stream(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        graph.capture_begin()
        for i in range(a.steps):
            step(i, C.c_void_p(side.cuda_stream))
        graph.capture_end()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    graph.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / a.steps
    kv_bytes = B * ctx * KV_ROW_BYTES
    nbytes = kv_bytes + 2 * H * 512 * 128 * 2 + q.numel() * 4 + cur.numel() * 4
    print(json.dumps({"metric": "mla_decode_layer_step_bandwidth", "value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1,
                      "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
                      "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": "decode step of one MLA layer, q projection output to wo input: rope x2, absorb, cache write, paged attention (B=%d H=%d ctx=%d bf16), un-absorb; %s" % (B, H, ctx, "5 kernel launches (rope of q_pe, absorb and rope of k_pe + cache write in one dispatch)" if a.front == "batch" else "8 kernel launches")},
                      "us_per_step": ms * 1e3, "eager_us_per_step": eager_ms * 1e3, "launch": "hip graph replay of the K steps",
                      "tokens_per_s": B / (ms * 1e-3),
                      "roofline": {"bound": "hbm", "kernel": "whole step", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                   "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "traffic": None, "algorithmic_bytes_per_launch": nbytes},
                      "cpu_baseline": None}))


def _timed(f):
    t0 = time.perf_counter()
    f()
    return time.perf_counter() - t0


def other_config(a, dev, lib, J):
    """BASELINE configs 2, 4 and 5 through the same C ABI: parity-test shapes, timed here for the profiles (not the
    headline line).  One JSON line in the same format; the metric of the prefill config is its MFMA rate."""
    import numpy as np
    import torch
    scale = 1.0 / (192.0 ** 0.5)
    rng = np.random.default_rng(a.seed)
    mask = None
    if a.config == "c2":
        lens, n_head, n_tok, kv, kvt = [int(x) for x in rng.integers(512, 4097, 8)], 16, 1, "bf16", J.MLA_TYPE_BF16
        name = "BASELINE configs[1]: paged MLA decode B=8 H=16 L~U[512,4096], bf16"
    elif a.config == "c3mask":
        # the headline shape as the reference's unmodified graph presents it: no block table, one cache shared by the 32
        # sequences, one query token per sequence, membership through the f16 mask (src/llama-context.cpp:364-404)
        B, L = 32, 8192
        g = torch.Generator(device=dev)
        g.manual_seed(a.seed)
        if a.kv == "q8_0":   # --kv q8_0: the same cache as Q8_0 cells (int8 = round(N(0, 0.5) * 32), block scale 1/32)
            qs = torch.clamp(torch.round(torch.randn((B * L, 18, 32), generator=g, device=dev) * 16), -127, 127).to(torch.int8)
            pool = torch.empty((B * L, 18, 34), dtype=torch.uint8, device=dev)
            pool[:, :, 0], pool[:, :, 1] = 0x00, 0x28
            pool[:, :, 2:] = qs.view(torch.uint8)
            pool = pool.reshape(1, B * L, 612)
        else:
            pool = (torch.randn((1, B * L, 576), generator=g, device=dev) * 0.5).to(torch.bfloat16).view(torch.int16)
        H = a.heads   # (--heads 16: the same batch at tensor-parallel degree 8)
        q = torch.randn((1, H, B, 576), generator=g, device=dev)
        mask = torch.full((64, B * L), float("-inf"), dtype=torch.float16, device=dev)
        # --ragged: every sequence owns a slot of 8192 cells of the shared cache but has filled only 2048 .. 8192 of them
        lens = [int(x) for x in rng.integers(2048, 8193, B)] if a.ragged else [L] * B
        for b in range(B):
            mask[b, b * L:b * L + lens[b]] = 0
        out = torch.empty((1, B, H, 576), dtype=torch.float32, device=dev)
        n_head, n_tok, kv, kvt = H, B, ("q8_0" if a.kv == "q8_0" else "bf16"), (J.MLA_TYPE_Q8_0 if a.kv == "q8_0" else J.MLA_TYPE_BF16)
        name = "BASELINE configs[2] without the block table: one shared cache of 262144 cells, 32 query tokens x %d heads, f16 mask selects each token's %s cells" % (H, "2048..8192" if a.ragged else "8192")
    elif a.config == "c4":
        lens, n_head, n_tok, kv, kvt = [2560] * 4, 16, 512, "bf16", J.MLA_TYPE_BF16
        mask = torch.where(torch.arange(2560, device=dev)[None, :] > 2048 + torch.arange(512, device=dev)[:, None], float("-inf"), 0.0).to(torch.float16)
        name = "BASELINE configs[3]: chunked prefill B=4 H=16, 512 new on 2048 cached tokens, causal f16 mask, bf16 pages"
    elif a.config == "ragged":
        # a paged decode batch of any size with lengths uniform in [256, ctx] (more than 256 sequences: one workgroup each, longest first)
        lens, n_head, n_tok, kv, kvt = [int(x) for x in rng.integers(256, a.ctx + 1, a.batch)], a.heads, 1, "bf16", J.MLA_TYPE_BF16
        name = "paged MLA decode B=%d H=%d L~U[256,%d], bf16 pages" % (a.batch, a.heads, a.ctx)
    elif a.config == "chunk":
        # one prompt chunk of --tokens tokens behind --cached cached ones: a contiguous cache without a block table, causal f16 mask
        n_old, n_tok, n_head, kv, kvt = a.cached, a.tokens, a.heads, "bf16", J.MLA_TYPE_BF16
        n_kv = (n_old + n_tok + 31) // 32 * 32
        g = torch.Generator(device=dev)
        g.manual_seed(a.seed)
        pool = (torch.randn((1, n_kv, 576), generator=g, device=dev) * 0.5).to(torch.bfloat16).view(torch.int16)
        q = torch.randn((1, n_head, n_tok, 576), generator=g, device=dev)
        mask = torch.where(torch.arange(n_kv, device=dev)[None, :] > n_old + torch.arange(n_tok, device=dev)[:, None], float("-inf"), 0.0).to(torch.float16)
        out = torch.empty((1, n_tok, n_head, 576), dtype=torch.float32, device=dev)
        lens = [n_old + n_tok]
        name = "prompt chunk: %d new on %d cached tokens, H=%d, one contiguous bf16 cache, causal f16 mask" % (n_tok, n_old, n_head)
    else:
        lens, n_head, n_tok, kv, kvt = [int(x) for x in rng.integers(2048, 8193, 64)], 128, 1, "q8_0", J.MLA_TYPE_Q8_0
        name = "BASELINE configs[4]: paged MLA decode B=64 H=128 L~U[2048,8192], Q8_0 pages"
    if a.config in ("c3mask", "chunk"):
        bt = sl = None
    else:
        q, pool, bt, sl = build_paged(dev, lens, n_head, n_tok, kv, a.seed)
        out = torch.empty((len(lens), n_tok, n_head, 576), dtype=torch.float32, device=dev)
    kw = dict(dv=512, scale=scale, mask=mask, block_table=bt, seq_lens=sl, out=out, n_splits=a.splits, rows_per_wg=a.rows_per_wg,
              flags=(J.MLA_FLAG_UNIFORM_SPLITS if a.uniform_splits else 0) | (J.MLA_FLAG_BF16_DIRECT if a.bf16_direct else 0))
    if a.reuse_mask_extents:
        # the node of a layer after the first of a graph: the mask is the one whose extents the launch before left in the workspace
        assert mask is not None, "--reuse-mask-extents needs a masked config"
        ar0, _, keep0 = J.capi.make_args(q, pool, kvt, **kw)
        rc = lib.mla_attn_launch(C.byref(ar0), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
        assert rc == 0, rc
        torch.cuda.synchronize()
        kw["flags"] |= J.MLA_FLAG_MASK_EXTENTS_VALID
    # The cache is rotated between steps, as for the headline config: copies at different addresses, enough of them that a step
    # never finds its cells in the 256 MB Infinity Cache from the step before (a model's layers each have a cache of their own, so
    # that is what a real step sees); the prefill configs, whose row blocks re-read one cache inside a step, rotate too.
    pool_bytes = pool.numel() * pool.element_size()
    n_pools = max(a.pools, min(64, -(-(1 << 30) // pool_bytes)))
    pools = [pool] + [pool.clone() for _ in range(n_pools - 1)]
    ars = [J.capi.make_args(q, pl_, kvt, **kw) for pl_ in pools]
    ar, _, keep = ars[0]
    plan = J.plan(q, pool, kvt, **kw)
    stream = torch.cuda.current_stream(dev)
    st = C.c_void_p(stream.cuda_stream)
    step_no = [0]

    def run(fn, n, on=None):
        for _ in range(n):
            rc = fn(C.byref(ars[step_no[0] % n_pools][0]), on or st)
            step_no[0] += 1
            if rc != 0:
                raise RuntimeError("launch failed: %d" % rc)

    run(lib.mla_attn_launch, a.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run(lib.mla_attn_launch, a.steps)
    torch.cuda.synchronize()
    eager_ms = ms = (time.perf_counter() - t0) * 1e3 / a.steps
    if not a.eager:   # as for the headline config: the K steps replayed from one HIP graph
        side = torch.cuda.Stream(dev)
        graph = torch.cuda.CUDAGraph()
        sst = C.c_void_p(side.cuda_stream)
        with torch.cuda.stream(side):
            graph.capture_begin()
            run(lib.mla_attn_launch, a.steps, sst)
            graph.capture_end()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / a.steps
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    run(lib.mla_attn_launch_kernel, a.steps)
    e1.record(stream)
    torch.cuda.synchronize()
    kern_ms = e0.elapsed_time(e1) / a.steps
    if a.config in ("c4", "chunk"):
        n_old = 2048 if a.config == "c4" else n_old
        kv_bytes = sum(lens) * KV_ROW_BYTES
        flops = len(lens) * n_head * FLOP_PER_TOKEN_HEAD * (n_tok * n_old + n_tok * (n_tok + 1) // 2)
        roof = {"bound": "mfma", "achieved": flops / (kern_ms * 1e-3) / 1e12, "peak": 2500.0, "unit": "TFLOP/s"}
        metric, value, unit = "mla_prefill_attention_rate", flops / (ms * 1e-3) / 1e12, "TFLOP/s"
    else:
        kv_bytes = sum(lens) * (612 if kv == "q8_0" else KV_ROW_BYTES)
        flops = sum(lens) * n_head * FLOP_PER_TOKEN_HEAD
        roof = {"bound": "hbm", "achieved": kv_bytes / (kern_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s"}
        metric, value, unit = "mla_paged_decode_kv_read_bandwidth", kv_bytes / (ms * 1e-3) / 1e9, "GB/s"
    roof.update({"frac": roof["achieved"] / roof["peak"], "traffic": None, "kernel_us": {"mean": kern_ms * 1e3},
                 "mfma_tflops": flops / (kern_ms * 1e-3) / 1e12, "algorithmic_bytes_per_launch": kv_bytes})
    print(json.dumps({"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
                      "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
                      "dtype": "f16" if kv == "q8_0" else kv, "data": "synthetic",
                      "config": {"workload": name, "plan": plan, "kv_pools_rotated": n_pools}, "us_per_step": ms * 1e3, "eager_us_per_step": eager_ms * 1e3,
                      "launch": "eager" if a.eager else "hip graph replay of the K steps", "roofline": roof, "cpu_baseline": None}))


def cpu_baseline(q, pool, block_table, ctx, n_sample, scale, gpu_out):
    """ggml-cpu's flash_attn_ext on the host cores for the first n_sample sequences of the same workload:
    the reference's own compiled ggml when oracle/_ref is built (kind "reference"), else the C restatement ("port")."""
    import numpy as np
    import torch
    from oracle import oracle as O
    cores = min(os.cpu_count() or 1, 16)
    qs = q[:n_sample].cpu().numpy()
    ids = block_table[:n_sample].cpu().numpy().astype(np.int64)
    pool_pages = pool.view(torch.int16).reshape(-1, 128, 576)
    k = pool_pages[torch.from_numpy(ids).to(pool.device)].reshape(n_sample, ctx, 576).cpu().numpy().view(np.uint16)
    kind = "reference" if O.ref_available() else "port"

    def run():
        if kind == "reference":
            return O.ref_flash_attn_ext(qs, k, O.TYPE_BF16, scale=scale, n_threads=cores)[..., :512]
        return O.flash_attn_ext(qs, k, O.TYPE_BF16, dv=512, scale=scale, n_threads=cores)

    want = run()  # warm-up, also the parity check
    best = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        run()
        best = min(best, time.perf_counter() - t0)
    kv_bytes = n_sample * ctx * KV_ROW_BYTES
    got = gpu_out[:n_sample, :, :, :512].cpu().numpy()
    max_abs, rel_l2 = O.errors(got, want)
    return {
        "value": kv_bytes / best / 1e9, "unit": "GB/s", "cores": cores, "kind": kind,
        "sample": "%d of the workload's sequences (128 heads x %d keys each), OpenMP over rows, best of 3; %.1f ms" % (n_sample, ctx, best * 1e3),
        "us_per_step_equiv": best * 1e6 * (q.shape[0] / n_sample),
    }, {"max_abs": max_abs, "rel_l2": rel_l2, "vs": kind, "sequences": n_sample}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--heads", type=int, default=128)
    ap.add_argument("--ctx", type=int, default=8192)
    ap.add_argument("--pools", type=int, default=4, help="distinct KV pools rotated between steps")
    ap.add_argument("--front", choices=["batch", "separate"], default="batch", help="--config layer: the nodes ahead of the attention node in one dispatch (mla_front_batch_launch), or a launch each")
    ap.add_argument("--splits", type=int, default=0)
    ap.add_argument("--rows-per-wg", type=int, default=0)
    ap.add_argument("--cpu-seqs", type=int, default=32, help="sequences of the workload timed on the host cores (default: the whole step; 0 = skip)")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--tokens", type=int, default=32, help="query tokens of --config rope / absorb / unabsorb (32 = a decode step, 2048 = a prefill chunk)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="N",
                    help="also launch the library's plain copy kernel N times over one KV pool (known byte count) so that a "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run can be scaled")
    ap.add_argument("--kv", default="bf16", choices=["bf16", "f16", "q8_0"], help="storage type of the latent KV pool (the headline config is bf16; q8_0 only with --config kvwrite)")
    ap.add_argument("--reuse-mask-extents", action="store_true", help="masked configs: time the launch of a layer after the first of a graph, which finds the key extents of the shared mask in the workspace (MLA_FLAG_MASK_EXTENTS_VALID)")
    ap.add_argument("--cached", type=int, default=0, help="--config chunk: tokens already in the cache ahead of the chunk")
    ap.add_argument("--ragged", action="store_true", help="--config c3mask: sequence lengths uniform in [2048, 8192] instead of 8192")
    ap.add_argument("--uniform-splits", action="store_true", help="paged decode: equal KV splits per sequence (MLA_FLAG_UNIFORM_SPLITS) instead of the balanced schedule")
    ap.add_argument("--bf16-direct", action="store_true", help="bf16 KV: the hi + lo bf16 program (MLA_FLAG_BF16_DIRECT) instead of the default one that converts the tiles to f16 inside LDS")
    ap.add_argument("--eager", action="store_true", help="time the K steps as K eager launch sequences instead of one replay of a HIP graph that holds them")
    ap.add_argument("--config", default="c3", choices=["c2", "c3", "c3mask", "c4", "c5", "ragged", "chunk", "kvwrite", "rope", "absorb", "unabsorb", "layer"],
                    help="c3 (default) is the headline workload; the others time BASELINE's remaining GPU configs and the cache write for the profiles")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus %d is not supported (use --gpus 1)" % a.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import jittorinfer_amd as J
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = J.library()
    dev = torch.device("cuda:0")
    scale = 1.0 / (192.0 ** 0.5)
    if a.config == "kvwrite":
        kv_write_config(a, dev, lib, J)
        return
    if a.config in ("rope", "absorb", "unabsorb"):
        front_config(a, dev, lib, J)
        return
    if a.config == "layer":
        layer_config(a, dev, lib, J)
        return
    if a.config != "c3":
        other_config(a, dev, lib, J)
        return
    if a.kv == "q8_0":
        print("bench.py: --kv q8_0 goes with --config kvwrite or --config c5", file=sys.stderr)
        sys.exit(2)

    q, pools, block_table, seq_lens = build_workload(dev, a.batch, a.heads, a.ctx, a.pools, a.seed, a.kv)
    kv_type = J.MLA_TYPE_BF16 if a.kv == "bf16" else J.MLA_TYPE_F16
    out = torch.empty((a.batch, 1, a.heads, 576), dtype=torch.float32, device=dev)
    args = []
    keep = []
    for pool in pools:
        ar, _, k = J.capi.make_args(q, pool.view(torch.int16), kv_type, dv=512, scale=scale, block_table=block_table,
                                    seq_lens=seq_lens, out=out, n_splits=a.splits, rows_per_wg=a.rows_per_wg,
                                    flags=(J.MLA_FLAG_UNIFORM_SPLITS if a.uniform_splits else 0) | (J.MLA_FLAG_BF16_DIRECT if a.bf16_direct else 0))
        args.append(ar)
        keep.append(k)
    plan = J.plan(q, pools[0].view(torch.int16), kv_type, dv=512, scale=scale, block_table=block_table, seq_lens=seq_lens, out=out, n_splits=a.splits, rows_per_wg=a.rows_per_wg)
    stream = torch.cuda.current_stream(dev)
    st = C.c_void_p(stream.cuda_stream)

    def step(i, fn=lib.mla_attn_launch):
        rc = fn(C.byref(args[i % len(args)]), st)
        if rc != 0:
            raise RuntimeError("launch failed: %d" % rc)

    for i in range(a.warmup):
        step(i)
    torch.cuda.synchronize()

    # ---- timed region: exactly K steps, synchronised on both sides.  Eager: K calls of mla_attn_launch (three kernel
    # launches each).  Default: the same K calls captured once into a HIP graph (the library neither allocates nor
    # clears memory, so its launches can be captured) and replayed: what a serving loop does with a launch-bound step.
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(i)
    torch.cuda.synchronize()
    eager_ms_per_step = (time.perf_counter() - t0) * 1e3 / a.steps
    ms_per_step = eager_ms_per_step
    if not a.eager:
        side = torch.cuda.Stream(dev)
        graph = torch.cuda.CUDAGraph()
        sst = C.c_void_p(side.cuda_stream)
        with torch.cuda.stream(side):
            graph.capture_begin()
            for i in range(a.steps):
                rc = lib.mla_attn_launch(C.byref(args[i % len(args)]), sst)
                if rc != 0:
                    raise RuntimeError("launch failed during capture: %d" % rc)
            graph.capture_end()
        torch.cuda.synchronize()
        graph.replay()          # untimed: first replay uploads the graph
        torch.cuda.synchronize()
        # the K steps are timed several times over (each replay bracketed by a synchronize on both sides) until at least
        # 50 ms and 11 replays are on the clock; the reported step is the median replay, the spread is kept beside it
        replays = []
        while len(replays) < 11 or (sum(replays) * a.steps < 50e3 and len(replays) < 200):
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            replays.append((time.perf_counter() - t0) * 1e6 / a.steps)
        first_replay_us = replays[0]
        replays.sort()
        n = len(replays)
        ms_per_step = 0.5 * (replays[(n - 1) // 2] + replays[n // 2]) * 1e-3
        step_stats = {"median": ms_per_step * 1e3, "p10": replays[n // 10], "p90": replays[(9 * n) // 10], "first": first_replay_us, "replays_of_k_steps": n}
    else:
        step_stats = None

    # ---- the kernels that make up the node without the Q pre-pack: the split-K decode kernel and the combine pass, with a HIP
    # event on the launch stream between every two steps (the stream is in order: an interval is one launch's duration plus the
    # hand-over to the next); mean, median and spread all come from those K intervals.  Then the decode kernel alone the same
    # way, whole steps (pre-pack + decode + combine) the same way, and, labelled as what it is, K decode launches back to back
    # between one pair of events (a launch's first workgroups start while the last of the one before still run, so this is
    # the rate of a stream of launches, not the duration of one)
    def per_launch(fns):
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(a.steps + 1)]
        marks[0].record(stream)
        for i in range(a.steps):
            for fn in fns:
                step(i, fn)
            marks[i + 1].record(stream)
        torch.cuda.synchronize()
        us = sorted(marks[i].elapsed_time(marks[i + 1]) * 1e3 for i in range(a.steps))
        pick = lambda f: us[min(len(us) - 1, int(f * len(us)))]
        return {"mean": sum(us) / len(us), "median": 0.5 * (us[(len(us) - 1) // 2] + us[len(us) // 2]), "p10": pick(0.1), "p90": pick(0.9), "launches": len(us)}

    def back_to_back(fns):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(a.steps):
            for fn in fns:
                step(i, fn)
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / a.steps
    node_stats = per_launch([lib.mla_attn_launch_kernel, lib.mla_attn_launch_combine])   # the Q operand image in the workspace is the one the steps above wrote
    kern_stats = per_launch([lib.mla_attn_launch_kernel])
    kern_stats["back_to_back"] = back_to_back([lib.mla_attn_launch_kernel])
    step_stats_events = per_launch([lib.mla_attn_launch])
    node_ms, kern_ms, step_ms_events = node_stats["mean"] * 1e-3, kern_stats["mean"] * 1e-3, step_stats_events["mean"] * 1e-3

    kv_bytes = a.batch * a.ctx * KV_ROW_BYTES
    flops = a.batch * a.ctx * a.heads * FLOP_PER_TOKEN_HEAD
    value = kv_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = kv_bytes / (node_ms * 1e-3) / 1e9          # decode kernel + combine pass
    achieved_decode = kv_bytes / (kern_ms * 1e-3) / 1e9

    if a.copy_calibration > 0:
        dst_copy = torch.empty_like(pools[0])
        for _ in range(a.copy_calibration):
            J.hbm_copy(pools[0], dst_copy)
        torch.cuda.synchronize()
        del dst_copy

    # final output of the last step for the parity check
    step(0)
    torch.cuda.synchronize()
    cpu, parity = (None, None)
    if a.cpu_seqs > 0:
        cpu, parity = cpu_baseline(q, pools[0], block_table, a.ctx, min(a.cpu_seqs, a.batch), scale, out)

    # HBM bytes of one decode-kernel launch, from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) scaled by what the same
    # counters read for the library's copy kernel; figures and commands in profiles/mla_decode_kernel_c3_pmc.md
    traffic, traffic_source, traffic_decode = None, None, None
    measured_plan = {"variant": 2, "n_splits": 8, "balanced": 1, "n_workgroups": 256, "lds_bytes": 160864}   # the launch the constants below were taken on
    if a.batch == 32 and a.heads == 128 and a.ctx == 8192 and a.kv == "bf16":
        differs = {k: (plan.get(k), v) for k, v in measured_plan.items() if plan.get(k) != v}
        if differs:
            traffic_source = "not reported: the plan of this launch differs from the one profiles/mla_decode_kernel_c3_pmc.md was measured on: %s" % differs
        else:
            traffic_source = ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of the decode kernel and of the combine pass, scaled by the copy kernel's readings: "
                              "profiles/mla_decode_kernel_c3_pmc.md (constants of that profile, taken at commit %s on %s, not of this run)" % TRAFFIC_PROFILE_COMMIT)
            # KiB per dispatch, mean: decode kernel (fetch, write), combine pass (fetch, write)
            d_f, d_w, c_f, c_w = (150524, 34048, 16677, 8192) if a.bf16_direct else (150520, 34560, 16560, 8192)
            scale_f = 294912 / 147466.0   # the copy kernel reads 294 912 KiB and FETCH_SIZE reports 147 466
            traffic_decode = int(d_f * 1024 * scale_f + d_w * 1024)
            traffic = traffic_decode + int(c_f * 1024 * scale_f + c_w * 1024)
    res = {
        "metric": "mla_paged_decode_kv_read_bandwidth", "value": value, "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.kv, "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: paged MLA decode B=%d H=%d ctx=%d, bf16 latent KV 576/512, 128-token pages, shuffled block table" % (a.batch, a.heads, a.ctx),
                   "batch": a.batch, "heads": a.heads, "ctx": a.ctx, "kv_pools_rotated": a.pools, "plan": plan},
        "us_per_step": ms_per_step * 1e3,
        "launch": "eager" if a.eager else "hip graph replay of the K steps",
        "us_per_step_eager": eager_ms_per_step * 1e3,
        "us_per_step_events": step_stats_events,
        "us_per_step_spread": step_stats,
        "tokens_per_s": a.batch / (ms_per_step * 1e-3),
        "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBPS,
        "tflops": flops / (ms_per_step * 1e-3) / 1e12,
        "roofline": {"bound": "hbm", "kernel": "mla_decode_kernel<%s> + mla_attn_combine_kernel" % a.kv, "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic, "traffic_source": traffic_source,
                     "algorithmic_bytes_per_launch": kv_bytes, "kernels_us": node_stats,
                     "decode_kernel_alone": {"achieved": achieved_decode, "frac": achieved_decode / HBM_PEAK_GBPS, "kernel_us": kern_stats, "traffic": traffic_decode},
                     "mfma_tflops": flops / (node_ms * 1e-3) / 1e12},
        "cpu_baseline": cpu,
        "parity": parity,
    }
    print(json.dumps(res))


if __name__ == "__main__":
    main()

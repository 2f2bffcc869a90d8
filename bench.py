"""Decode-attention benchmark of the forest cascade path on one MI355X.

A step is one attention layer's decode call (shared-prefix items and per-sequence suffix
items in one launch, then the log-sum-exp merge) over the whole batch.  The forest
metadata is rebuilt once every ``--layers`` steps, the way a model forward shares one
build across its attention layers (Qwen3-4B: 36), and each layer reads its own KV cache
copy so no step finds its KV in a cache left by the previous one.

Prints one JSON line: step latency in microseconds, the share of the 8 TB/s HBM peak that
the unique KV bytes per step amount to, a roofline object for the attention kernel
(timed with events on the launch stream inside the timed region), the same shape through
the non-cascade kernel, and a CPU baseline (the oracle's flat attention on a sample).
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the attention kernel from the rocprofv3 FETCH_SIZE / WRITE_SIZE
# passes summarised in profiles/, keyed by (configuration, chunk_tokens, rows_per_item).
# Counters cannot be read from inside this process; other shapes report null.
MEASURED_TRAFFIC_BYTES = {(2, 1024, 32): 1_865_600_000}
# Share of the matrix-core cycles that were busy (SQ_VALU_MFMA_BUSY_CYCLES over cycles x SIMDs)
# in the counter passes of the same profile summary: the whole attention launch, and the
# shared-prefix pass launched on its own (every MFMA row a live query row).
MEASURED_MFMA_UTIL = {(2, 1024, 32): {"attention_launch": 0.074, "prefix_pass": 0.072, "source": "profiles/attend32_c2_qwen3_4b.md"}}
METRIC = "cascade decode-attn µs/step & % of HBM peak, Qwen3-4B shape 512 seqs"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=720)
    ap.add_argument("--warmup", type=int, default=72)
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1-5 (default 2: the Qwen3-4B decode step); 6 = the forest of 2 with the heads of Qwen3.5 (Hq 16 / Hkv 2 / D 256)")
    ap.add_argument("--shrink", type=int, default=1, help="the configuration with its group counts and lengths divided by this (to try the script out on a small batch; not a benchmark figure)")
    ap.add_argument("--device", default="cuda:0", help="device of the tensors (the tests that run this script against the CPU emulation of the kernels pass cpu; the library itself takes device memory only)")
    ap.add_argument("--layers", type=int, default=36, help="attention layers sharing one metadata build")
    ap.add_argument("--kv-copies", type=int, default=4, help="distinct KV caches cycled over the layers")
    ap.add_argument("--chunk", type=int, default=0, help="split-K chunk in tokens (0 = default of the configuration)")
    ap.add_argument("--rows", type=int, default=0, help="query rows per work item, 32 or 64 (0 = default)")
    ap.add_argument("--fp8-tile-buffers", type=int, default=0, choices=(0, 3), help="3: the attention kernel of an fp8 cache (--config 5) keeps three register tile buffers per wave instead of two")
    ap.add_argument("--kv-reread", action="store_true", help="keep the KV loads cacheable instead of streaming them (worth a try where a shared node fills more than one row tile, e.g. --config 3 --rows 32: its row tiles then read the same blocks at nearly the same time)")
    ap.add_argument("--time-every", type=int, default=0, help="time the attention launch of every n-th step with events (0 = every second step of a short run, about 24 launches of a long one; -1 = none; under rocprofv3 no launch is timed whatever this says)")
    ap.add_argument("--cpu-seqs", type=int, default=512, help="sequences in the CPU baseline sample (0 = skip)")
    ap.add_argument("--skip-noncascade", action="store_true")
    ap.add_argument("--split-passes", action="store_true", help="also time the shared-prefix pass and the suffix pass as launches of their own (and leave them in the trace for the profiler)")
    ap.add_argument("--calibrate", action="store_true", help="also run the library's plain copy kernel over 1 GiB (counter yardstick)")
    ap.add_argument("--query-runs", default="", metavar="NxL", help="instead of a decode configuration: N sequences that each bring a run of L query tokens (a prefill chunk), e.g. 4x2048")
    ap.add_argument("--context", type=int, default=0, help="tokens already cached in front of every query run")
    ap.add_argument("--append", default="", metavar="NxL", help="instead of a decode configuration: the cache writer and reader, N sequences that each append L tokens (512x1 = a decode step, 1x8192 = a prefill), with --context tokens cached in front")
    ap.add_argument("--split-train", default="", metavar="GxS", help="instead of a decode configuration: the trainer's split attention, forward + backward, over G prompt groups of S samples each, e.g. 8x8")
    return ap.parse_args()


def median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def run_steps(torch, ops, build, w, caches, md, out, lse, steps, layers, timed_events=None, time_every=1):
    """``steps`` layer calls; metadata refreshed at every ``layers``-th one.  ``timed_events``
    (a list of event pairs): the attention launch of every ``time_every``-th step records its
    own begin and end in the next pair, through the library's measurement hook, so the step
    is the same two launches either way and nothing else enters the stream."""
    hook = None
    if timed_events:
        from arctic_platform_amd import _lib

        hook = _lib.load_library().fca_time_next_attention
    used = 0
    for i in range(steps):
        cache = caches[i % len(caches)]
        if i % layers == 0:
            build()
        if hook is not None and i % time_every == 0 and used < len(timed_events):
            a, b = timed_events[used]
            used += 1
            hook(a.cuda_event, b.cuda_event)
        ops.forest_cascade_decode(w.q, cache, md, w.scale, w.k_scale, w.v_scale, out=out, return_lse=False)
    return used


def under_profiler():
    """rocprofv3 names its tool library in the environment of the program it starts."""
    return bool(os.environ.get("ROCP_TOOL_LIBRARIES"))


def time_steps(torch, ops, build, w, caches, md, out, lse, steps, warmup, layers, time_every=0):
    """Wall time of ``steps`` steps after ``warmup`` untimed ones, and the durations of the
    attention launches inside the timed region.  A launch that records events costs the step
    about 5 us (measured: 305.3 against 300.5 us per step with every launch timed), so by
    default (``time_every`` = 0) every second step of a short run is timed and about 24
    launches, evenly spread, of a long one."""
    if under_profiler():
        time_every = -1  # the profiler has its own hold on every dispatch: its trace has the durations
    if time_every == 0:
        time_every = max(2, steps // 24)
    # (negative: no launch is timed)
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range((steps + time_every - 1) // time_every if time_every > 0 else 0)]
    for a, b in pairs:  # a first record creates the underlying HIP events
        a.record()
        b.record()
    run_steps(torch, ops, build, w, caches, md, out, lse, warmup, layers)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    used = run_steps(torch, ops, build, w, caches, md, out, lse, steps, layers, pairs, time_every)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_us = [a.elapsed_time(b) * 1e3 for a, b in pairs[:used]]
    return wall, kernel_us


def cpu_baseline(torch, w, nseq, gpu_out=None):
    """The oracle's flat attention (fp32, every sequence gathers its own pages, no
    sharing exploited) on the first ``nseq`` sequences, scaled to the whole batch.  With
    ``gpu_out`` (the timed path's output rows of those sequences) the oracle's result also
    checks it, to the parity tolerance of the tests."""
    from oracle.attention import flat_decode_attention

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    nseq = min(nseq, w.num_seqs)
    seqs = list(range(nseq))
    need = sorted({int(b) for s in seqs for b in w.block_table[s, : (int(w.seq_lens[s]) + 15) // 16].tolist()})
    remap = torch.zeros(w.kv_cache.shape[1], dtype=torch.long)
    remap[need] = torch.arange(len(need))
    cache = w.kv_cache[:, torch.as_tensor(need, device=w.kv_cache.device)].cpu()
    table = remap[w.block_table[:nseq].cpu().long()].to(torch.int32)
    q, lens = w.q[:nseq].cpu(), w.seq_lens[:nseq].cpu()
    ks = None if w.k_scale is None else w.k_scale.cpu()
    vs = None if w.v_scale is None else w.v_scale.cpu()
    times = []
    for it in range(3):
        t0 = time.perf_counter()
        ref_out, _ = flat_decode_attention(q, cache, table, lens, w.scale, ks, vs, dtype=torch.float32)
        times.append(time.perf_counter() - t0)
    sample_s = median(times[1:]) if len(times) > 1 else times[0]
    scale_up = float(w.seq_lens.sum()) / float(lens.sum())
    # for context: the same sample through the CPU restatement of the cascade (shared nodes
    # read once for all their members, then the merge), discovery included
    from oracle.cascade import cascade_decode_attention

    t0 = time.perf_counter()
    cascade_decode_attention(q, cache, table, lens, w.scale, ks, vs, dtype=torch.float32)
    cascade_s = time.perf_counter() - t0
    err = None
    if gpu_out is not None:
        diff = (gpu_out.cpu().float() - ref_out.float()).abs()
        err = float(diff.max())
        assert bool((diff <= 2e-2 + 2e-2 * ref_out.float().abs()).all()), f"timed output differs from the oracle: max |err| {err}"
    return {
        "value": sample_s * scale_up * 1e6,
        "unit": "us/step",
        "cores": cores,
        "kind": "port",
        "sample": f"first {nseq} of {w.num_seqs} sequences ({int(lens.sum())} of {int(w.seq_lens.sum())} gathered tokens), "
        f"flat fp32 attention on torch-CPU, {sample_s:.2f} s measured, scaled by tokens x{scale_up:.2f}",
        "cascade_restatement_us": cascade_s * scale_up * 1e6,
        "max_abs_err_of_timed_output": err,
    }


MFMA_BF16_PEAK_TFLOPS = 2500.0


def main_query_runs(args):
    """Prefill-shaped work on the same kernels: every sequence brings a run of query tokens;
    one query row per token, the tokens of one cache block form a causal node.  A step is
    one layer's attention call over all rows; flops are counted causally."""
    import torch

    from arctic_platform_amd import ops
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.kv_layout import kv_cache_shape
    from oracle.attention import flat_decode_attention

    nseq, ql = (int(v) for v in args.query_runs.lower().split("x"))
    ctx, hq, hkv, d = args.context, 32, 8, 128
    dev = torch.device(args.device)
    gen = torch.Generator().manual_seed(4242)
    max_blocks = (ctx + ql + 15) // 16
    table = torch.randperm(nseq * max_blocks, generator=gen).to(torch.int32).view(nseq, max_blocks).to(dev)
    caches = [torch.randn(kv_cache_shape(nseq * max_blocks, 16, hkv, d), generator=gen).to(torch.bfloat16).to(dev)]
    caches += [caches[0].clone() for _ in range(max(1, args.kv_copies) - 1)]
    rows_total = nseq * ql
    q = torch.randn(rows_total, hq, d, generator=gen).to(torch.bfloat16).to(dev)
    seq = torch.arange(nseq, device=dev).repeat_interleave(ql)
    lens = (ctx + 1 + torch.arange(ql, device=dev).repeat(nseq)).to(torch.int32)
    row_table = seq.to(torch.int32)
    row_group = (seq * max_blocks + (lens - 1) // 16).to(torch.int32)
    chunk, rows = args.chunk or 1024, args.rows or 64
    kw = dict(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, chunk_tokens=chunk, rows_per_item=rows, row_table=row_table, row_group=row_group)
    md = build_forest_metadata(table, lens, **kw)
    torch.cuda.synchronize()
    md.check()
    out = torch.empty_like(q)
    scale = d**-0.5

    def step(i, events=None):
        cache = caches[i % len(caches)]
        if i % args.layers == 0:
            build_forest_metadata(table, lens, out=md, **kw)
            if events is not None:
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                ops.forest_pass(q, cache, md, scale)
                b.record()
                ops.merge_partials(md, q, out=out, return_lse=False)
                events.append((a, b))
                return
        ops.forest_cascade_decode(q, cache, md, scale, out=out, return_lse=False)

    steps, warmup = min(args.steps, 144), min(args.warmup, 36)
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    events = []
    t0 = time.perf_counter()
    for i in range(steps):
        step(i, events)
    torch.cuda.synchronize()
    step_us = (time.perf_counter() - t0) / steps * 1e6
    kern = sum(a.elapsed_time(b) * 1e3 for a, b in events) / len(events)
    fresh = None
    if ctx == 0:
        # what the adapter does for a step of fresh prompts: attention straight from the step's
        # K and V on the split-attention kernels, each prompt a group of its own (timing only:
        # random K and V of the same shape; checked against the oracle in the tests)
        from arctic_platform_amd.split_attention import SplitLayout, split_attention_forward

        layout = SplitLayout([(0, [ql])] * nseq, device=dev)
        kp, vp = (torch.randn(rows_total, hkv, d, generator=gen).to(torch.bfloat16).to(dev) for _ in range(2))
        out3 = torch.empty(rows_total, hq, d, dtype=torch.bfloat16, device=dev)
        for _ in range(3):
            split_attention_forward(q, kp, vp, layout, scale, out=out3)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(20):
            split_attention_forward(q, kp, vp, layout, scale, out=out3)
        b.record()
        torch.cuda.synchronize()
        fresh_us = a.elapsed_time(b) * 1e3 / 20
        fresh = {"us_per_step": round(fresh_us, 2), "tflops": round(4.0 * d * hq * float(lens.double().sum()) / fresh_us / 1e6, 1),
                 "what": "split_attention_forward on the step's packed K and V (operand images included)"}
    else:
        # what the adapter does for long chunks behind a cached context: K and V of context and
        # chunk gathered from the cache, then the split-attention forward for the chunk's rows
        from arctic_platform_amd.cache import gather_kv
        from arctic_platform_amd.split_attention import SplitLayout, split_attention_forward

        layout = SplitLayout([(ctx, [ql])] * nseq, device=dev, responses_only=True)
        req = torch.arange(nseq, device=dev).repeat_interleave(ctx + ql)
        pos = torch.arange(ctx + ql, device=dev).repeat(nseq)
        slots = table[req, pos // 16].to(torch.int64) * 16 + pos % 16
        out3 = torch.empty(rows_total, hq, d, dtype=torch.bfloat16, device=dev)

        def ctx_step():
            kk, vv = gather_kv(caches[0], slots, d)
            split_attention_forward(q, kk, vv, layout, scale, out=out3)

        for _ in range(3):
            ctx_step()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(20):
            ctx_step()
        b.record()
        torch.cuda.synchronize()
        fresh_us = a.elapsed_time(b) * 1e3 / 20
        ok = bool(((out3.float() - out.view(rows_total, hq, d).float()).abs() <= 2e-2 + 2e-2 * out.view(rows_total, hq, d).float().abs()).all())
        fresh = {"us_per_step": round(fresh_us, 2), "tflops": round(4.0 * d * hq * float(lens.double().sum()) / fresh_us / 1e6, 1),
                 "what": "K and V of context + chunk gathered from the cache, then split_attention_forward for the chunk's rows",
                 "agrees_with_query_run_path": ok}
    flops = 4.0 * d * hq * float(lens.double().sum())

    # CPU baseline and a parity spot check on a sample of rows
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    sample = list(range(0, rows_total, max(1, rows_total // 256)))[:256]
    idx = torch.tensor(sample)
    t0 = time.perf_counter()
    ref_out, _ = flat_decode_attention(q[idx.to(dev)].cpu(), caches[0].cpu(), table.cpu()[row_table.cpu()[idx].long()], lens.cpu()[idx], scale, dtype=torch.float32)
    cpu_s = time.perf_counter() - t0
    diff = (out[idx.to(dev)].cpu().float() - ref_out).abs()
    err = float(diff.max())
    assert bool((diff <= 2e-2 + 2e-2 * ref_out.abs()).all()), f"timed output differs from the oracle: max |err| {err}"
    scale_up = float(lens.double().sum()) / float(lens.cpu()[idx].double().sum())
    hdr = md.header()
    print(json.dumps({
        "metric": "query-run (prefill) attention µs/step, causal, Qwen3-4B heads",
        "value": round(step_us, 2), "unit": "us/step", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(step_us / 1e3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 MFMA / f32 accumulate", "data": "synthetic",
        "config": {"workload": f"{nseq} sequences x {ql} query tokens after {ctx} cached, Hq {hq} / Hkv {hkv} / D {d}, bf16, one causal node per cache block of a run",
                   "query_rows": rows_total, "chunk_tokens": chunk, "rows_per_item": rows, "work_items": hdr["items"],
                   "layers_per_metadata_build": args.layers, "causal_flops": flops},
        "roofline": {"kernel": "fca_attend64_kernel" if rows == 64 else "fca_attend32_kernel", "bound": "mfma",
                     "achieved": round(flops / kern / 1e6, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / kern / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None, "launches_timed": len(events)},
        "breakdown_us": {"attention_kernel": round(kern, 2)},
        "prompts_on_split_kernels": fresh,
        "cpu_baseline": {"value": cpu_s * scale_up * 1e6, "unit": "us/step", "cores": cores, "kind": "port",
                         "sample": f"{len(sample)} of {rows_total} query rows, flat fp32 attention on torch-CPU, {cpu_s:.2f} s measured, scaled by gathered tokens x{scale_up:.1f}"},
        "max_abs_err_vs_oracle_sample": err,
    }))


def main_append(args):
    """The KV-cache writer (fca_append_kv) and its way back (fca_gather_kv): N sequences append
    L tokens each into a paged cache with a random block table.  A step is one layer's append
    of the whole batch; bytes = what the call must move (K and V rows read, cache tiles
    written, and the other way round for the gather).  The yardstick is the library's plain
    copy kernel over the same number of bytes."""
    import torch

    from arctic_platform_amd import _lib
    from arctic_platform_amd.cache import append_kv, gather_kv
    from arctic_platform_amd.forest import _stream_ptr
    from arctic_platform_amd.kv_layout import kv_cache_shape
    from oracle.cache import append_kv_reference

    nseq, ql = (int(v) for v in args.append.lower().split("x"))
    ctx, hkv, d = args.context, 8, 128
    dev = torch.device(args.device)
    gen = torch.Generator().manual_seed(99)
    max_blocks = (ctx + ql + 15) // 16
    nblocks = nseq * max_blocks
    table = torch.randperm(nblocks, generator=gen).view(nseq, max_blocks)
    pos = ctx + torch.arange(ql).repeat(nseq)
    seq = torch.arange(nseq).repeat_interleave(ql)
    slots = (table[seq, pos // 16].to(torch.int64) * 16 + pos % 16).to(dev)
    t = nseq * ql
    key = torch.randn(t, hkv, d, generator=gen).to(torch.bfloat16).to(dev)
    value = torch.randn(t, hkv, d, generator=gen).to(torch.bfloat16).to(dev)
    lib = _lib.load_library()
    steps, warmup = min(args.steps, 200), min(args.warmup, 20)

    def timed(fn):
        for _ in range(warmup):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / steps

    out = {}
    for name, dtype in (("bf16", torch.bfloat16), ("fp8", torch.float8_e4m3fn)):
        cache = torch.zeros(kv_cache_shape(nblocks, 16, hkv, d), dtype=torch.bfloat16, device=dev).to(dtype)
        scales = None if dtype == torch.bfloat16 else (torch.full((hkv,), 0.05, device=dev), torch.full((hkv,), 0.04, device=dev))
        ks, vs = scales or (None, None)
        esz = cache.element_size()
        moved = 2 * t * hkv * d * (2 + esz)  # K and V: bf16 rows on one side, cache elements on the other
        us_a = timed(lambda: append_kv(key, value, cache, slots, ks, vs))
        rows = tuple(torch.empty_like(key) for _ in range(2))
        us_g = timed(lambda: gather_kv(cache, slots, d, ks, vs, out=rows))
        half = (moved // 2 + 15) // 16 * 16
        src, dst = torch.empty(half, dtype=torch.uint8, device=dev), torch.empty(half, dtype=torch.uint8, device=dev)
        us_c = timed(lambda: _lib.check(lib.fca_calibration_copy(src.data_ptr(), dst.data_ptr(), half, _stream_ptr(dev))))
        # the timed writer against the CPU restatement (plain loops) on a few of the blocks:
        # every token that lands in them is written, the blocks are compared byte for byte
        blocks = torch.unique(slots.cpu()[:: max(1, t // 6)] // 16)
        mask = torch.isin(slots.cpu() // 16, blocks)
        sel = mask.nonzero().squeeze(1)
        ref = append_kv_reference(
            torch.zeros(kv_cache_shape(nblocks, 16, hkv, d), dtype=torch.bfloat16).to(dtype), key.cpu()[sel], value.cpu()[sel], slots.cpu()[sel],
            None if ks is None else ks.cpu(), None if vs is None else vs.cpu(),
        )
        ok = bool(torch.equal(cache.cpu()[:, blocks].view(torch.uint8), ref[:, blocks].view(torch.uint8)))
        assert ok, f"{name}: the timed cache differs from the CPU restatement"
        got_k, got_v = (r.cpu()[sel] for r in rows)
        if dtype == torch.bfloat16:
            assert torch.equal(got_k, key.cpu()[sel]) and torch.equal(got_v, value.cpu()[sel]), "gather does not return what was appended"
        out[name] = {
            "append_us": round(us_a, 2), "append_gbs": round(moved / us_a / 1e3, 1),
            "gather_us": round(us_g, 2), "gather_gbs": round(moved / us_g / 1e3, 1),
            "copy_same_bytes_us": round(us_c, 2), "copy_gbs": round(2 * half / us_c / 1e3, 1),
            "bytes_moved": moved, "bit_exact_vs_cpu": ok,
        }
        del cache
    print(json.dumps({
        "metric": "KV-cache append µs/step (one layer, whole batch)", "value": out["bf16"]["append_us"], "unit": "us/step", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(out["bf16"]["append_us"] / 1e3, 5), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16 rows -> bf16 / fp8 e4m3 tiles", "data": "synthetic",
        "config": {"workload": f"{nseq} sequences x {ql} new tokens after {ctx} cached, Hkv {hkv} / D {d}, random block table", "tokens": t},
        "roofline": {"kernel": "fca_append_kernel", "bound": "hbm", "achieved": out["bf16"]["append_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(out["bf16"]["append_gbs"] / HBM_PEAK_GBS, 4), "traffic": None},
        "cache_io": out, "cpu_baseline": None,
    }))


def main_split_train(args):
    """The trainer's split attention over a deduplicated batch: G prompt groups, S samples
    each, prompts U[1024, 4096], responses U[1, 1024] tokens, Qwen3-4B heads.  A step is one
    layer's forward and backward.  Flops are the algorithmic ones of the visible (row, key)
    pairs: 4 D Hq per pair forward, 10 D Hq backward."""
    import random

    import torch

    from arctic_platform_amd.split_attention import SplitLayout, split_attention_backward, split_attention_forward
    from oracle.split_attention import split_attention as oracle_split

    ngroups, nsamples = (int(v) for v in args.split_train.lower().split("x"))
    hq, hkv, d = 32, 8, 128
    scale = d**-0.5
    rng = random.Random(1)
    groups = [(rng.randint(1024, 4096), [rng.randint(1, 1024) for _ in range(nsamples)]) for _ in range(ngroups)]

    def pairs_of(gs):
        return sum(p * (p + 1) // 2 + sum(r * p + r * (r + 1) // 2 for r in rs) for p, rs in gs)

    def tensors(gs, seed):
        gen = torch.Generator().manual_seed(seed)
        t = sum(p + sum(rs) for p, rs in gs)
        mk = lambda h: torch.randn(t, h, d, generator=gen).to(torch.bfloat16)
        return mk(hq), mk(hkv), mk(hkv), mk(hq)

    dev = torch.device(args.device)
    layout = SplitLayout(groups, device=dev)
    q, k, v, dout = (x.to(dev) for x in tensors(groups, 77))
    steps, warmup = min(args.steps, 20), min(args.warmup, 3)

    def fwd():
        return split_attention_forward(q, k, v, layout, scale)

    out, lse = fwd()

    def bwd():
        return split_attention_backward(dout, q, k, v, out, lse, layout, scale)

    def timed(fn, n):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / n

    for _ in range(warmup):
        fwd(), bwd()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fwd(), bwd()
    torch.cuda.synchronize()
    step_us = (time.perf_counter() - t0) / steps * 1e6
    fwd_us, bwd_us = timed(fwd, steps), timed(bwd, steps)
    pairs = pairs_of(groups)
    flops_f, flops_b = 4 * d * hq * pairs, 10 * d * hq * pairs

    # CPU baseline and check: the smallest group with two of its samples, through the oracle (fp32, autograd)
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    sp, srs = min(groups, key=lambda g: g[0] + sum(g[1]))
    sample = [(sp, srs[:2])]
    sq, sk, sv, sdo = tensors(sample, 78)
    sl = SplitLayout(sample, device=dev)
    g_out, g_lse = split_attention_forward(sq.to(dev), sk.to(dev), sv.to(dev), sl, scale)
    g_grads = split_attention_backward(sdo.to(dev), sq.to(dev), sk.to(dev), sv.to(dev), g_out, g_lse, sl, scale)
    t0 = time.perf_counter()
    rq, rk, rv = (x.float().requires_grad_() for x in (sq, sk, sv))
    r_out, _ = oracle_split(rq, rk, rv, sample, scale, dtype=torch.float32)
    r_out.backward(sdo.float())
    cpu_s = time.perf_counter() - t0
    errs = {}
    for name, got, ref, rel in (("out", g_out, r_out.detach(), 0.0), ("dq", g_grads[0], rq.grad, 1e-2), ("dk", g_grads[1], rk.grad, 1e-2), ("dv", g_grads[2], rv.grad, 1e-2)):
        diff = (got.cpu().float() - ref).abs()
        bound = (2e-2 if rel == 0.0 else rel * float(ref.abs().max())) + 2e-2 * ref.abs()
        assert bool((diff <= bound).all()), f"{name} differs from the oracle: max |err| {float(diff.max())}"
        errs[name] = float(diff.max())
    scale_up = pairs / pairs_of(sample)
    tfl = lambda f, us: round(f / us / 1e6, 1)
    print(json.dumps({
        "metric": "split attention (ZoRRo Train) forward + backward µs/step, Qwen3-4B heads",
        "value": round(step_us, 1), "unit": "us/step", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(step_us / 1e3, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 MFMA / f32 accumulate", "data": "synthetic",
        "config": {"workload": f"{ngroups} prompt groups x {nsamples} samples, prompt U[1024,4096], response U[1,1024], Hq {hq} / Hkv {hkv} / D {d}, bf16, deduplicated order",
                   "tokens": layout.num_tokens, "visible_pairs": pairs, "flops_forward": flops_f, "flops_backward": flops_b},
        "roofline": {"kernel": "split_query_kernel + split_key_kernel (forward, dq, dv, dk)", "bound": "mfma",
                     "achieved": tfl(flops_f + flops_b, fwd_us + bwd_us), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round((flops_f + flops_b) / (fwd_us + bwd_us) / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "forward_tflops": tfl(flops_f, fwd_us), "backward_tflops": tfl(flops_b, bwd_us)},
        "breakdown_us": {"forward": round(fwd_us, 1), "backward": round(bwd_us, 1)},
        "cpu_baseline": {"value": cpu_s * scale_up * 1e6, "unit": "us/step", "cores": cores, "kind": "port",
                         "sample": f"one group (prompt {sp}, responses {srs[:2]}) through the fp32 oracle with autograd on torch-CPU, {cpu_s:.2f} s measured, scaled by visible pairs x{scale_up:.1f}"},
        "max_abs_err_vs_oracle_sample": errs,
    }))


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path uses no collectives and the boxes have one GPU; run with --gpus 1")
    if args.query_runs:
        return main_query_runs(args)
    if args.split_train:
        return main_split_train(args)
    if args.append:
        return main_append(args)
    import torch

    from arctic_platform_amd import ops
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.workloads import make_config

    dev = torch.device(args.device)
    # configuration 1 is defined in fp32 (the CPU-runnable case) and runs on the all-fp32 path
    w = make_config(args.config, device=dev, shrink=args.shrink)
    fp32 = w.q.dtype == torch.float32
    # distinct copies at distinct addresses: same values, so every copy gives the same result
    caches = [w.kv_cache] + [w.kv_cache.clone() for _ in range(max(1, args.kv_copies) - 1)]
    chunk = args.chunk or (512 if w.head_dim == 256 else 1024)  # the adapter's defaults
    rows = args.rows or (64 if args.config == 3 else 32)
    kw = dict(num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, chunk_tokens=chunk, rows_per_item=rows)
    if args.kv_reread:
        kw["kv_reread"] = True
    if fp32:
        kw["partial_dtype"] = torch.float32
    out = torch.empty_like(w.q)

    md = build_forest_metadata(w.block_table, w.seq_lens, **kw)
    md.fp8_tile_buffers = args.fp8_tile_buffers
    torch.cuda.synchronize()
    md.check()
    hdr = md.header()
    unique_bytes = hdr["unique_tokens"] * w.kv_bytes_per_token
    assert unique_bytes == w.unique_kv_bytes, "builder and generator disagree on unique KV tokens"

    def build():
        build_forest_metadata(w.block_table, w.seq_lens, out=md, **kw)

    def refresh():
        # what a decode loop does at a scheduler step on a batch it has seen before: the
        # device checks that the rows still carry the forest and remakes leaves and work list
        build_forest_metadata(w.block_table, w.seq_lens, out=md, update=True, **kw)

    # builder and merge on their own, for the breakdown
    def ev_time(fn, n=20):
        fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(n):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b) * 1e3)
        return median(ts)

    build_us = ev_time(build)
    update_us = ev_time(refresh)
    # the merge reads what an attention pass wrote: one whole step first, then the merge on its own
    ops.forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale, out=out, return_lse=False)
    # (the fp32 path has no merge entry point of its own: it runs inside the step only)
    merge_us = None if fp32 else ev_time(lambda: ops.merge_partials(md, w.q, out=out, return_lse=False))

    split = None
    if args.split_passes:
        shared_tokens = sum(n["num_blocks"] * 16 for n in md.nodes())
        prefix_bytes = shared_tokens * w.kv_bytes_per_token
        tp = ev_time(lambda: ops.prefix_pass(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale))
        ts = ev_time(lambda: ops.suffix_pass(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale))
        split = {
            "prefix_pass_us": round(tp, 2),
            "prefix_unique_kv_bytes": prefix_bytes,
            "prefix_gbs": round(prefix_bytes / tp / 1e3, 1),
            "suffix_pass_us": round(ts, 2),
            "suffix_unique_kv_bytes": unique_bytes - prefix_bytes,
            "suffix_gbs": round((unique_bytes - prefix_bytes) / ts / 1e3, 1),
        }

    # The same batch through the same kernels with sharing off (every sequence reads its own
    # copy of the prefix: a plain paged decode attention), timed first so that the headline
    # below runs on a device that has been busy for a while.
    noncascade = None
    if not args.skip_noncascade:
        noncascade = {}
        nc = build_forest_metadata(w.block_table, w.seq_lens, cascade=False, **kw)
        torch.cuda.synchronize()

        def nc_build():
            build_forest_metadata(w.block_table, w.seq_lens, cascade=False, out=nc, **kw)

        nsteps = max(args.layers, args.steps // 4)
        nwall, _ = time_steps(torch, ops, nc_build, w, caches, nc, out, None, nsteps, args.layers, args.layers, -1)
        nc_us = nwall / nsteps * 1e6
        noncascade["noncascade"] = {
            "us_per_step": round(nc_us, 2),
            "order": "natural (the samples of a group are adjacent rows)",
            "gbs_on_flat_bytes": round(w.flat_kv_bytes / (nc_us * 1e-6) / 1e9, 1),
        }
        # same batch with the rows of each group spread across the batch
        perm = torch.arange(w.num_seqs, device=dev).view(-1, 8).t().reshape(-1) if w.num_seqs % 8 == 0 else None
        if perm is not None:
            bt2, sl2 = w.block_table[perm].contiguous(), w.seq_lens[perm].contiguous()
            nc2 = build_forest_metadata(bt2, sl2, cascade=False, **kw)

            def nc2_build():
                build_forest_metadata(bt2, sl2, cascade=False, out=nc2, **kw)

            import dataclasses

            w2 = dataclasses.replace(w, q=w.q[perm].contiguous(), block_table=bt2, seq_lens=sl2)
            nwall2, _ = time_steps(torch, ops, nc2_build, w2, caches, nc2, out, None, nsteps, args.layers, args.layers, -1)
            nc2_us = nwall2 / nsteps * 1e6
            noncascade["noncascade_interleaved"] = {
                "us_per_step": round(nc2_us, 2),
                "order": "group-interleaved (row i of every group, then row i+1, ...)",
            }
            del nc2
        del nc

    wall, kern_us = time_steps(torch, ops, refresh, w, caches, md, out, None, args.steps, args.warmup, args.layers, args.time_every)
    step_us = wall / args.steps * 1e6
    checked_rows = out[: max(0, min(args.cpu_seqs, w.num_seqs))].clone()  # compared with the oracle below
    kern = sum(kern_us) / len(kern_us) if kern_us else None

    result = {
        "metric": METRIC,
        "value": round(step_us, 2),
        "unit": "us/step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_us / 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if fp32 else "fp8 KV / bf16 MFMA / f32 accumulate" if args.config == 5 else "bf16 MFMA / f32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": w.name + (f", every count and length divided by {args.shrink}" if args.shrink > 1 else ""),
            "seed": 1000 + args.config,
            "num_seqs": w.num_seqs,
            "unique_kv_bytes": unique_bytes,
            "flat_kv_bytes": w.flat_kv_bytes,
            "layers_per_metadata_refresh": args.layers,
            "metadata_refresh": "fca_update_metadata (fingerprint check, leaves and work list remade); a full build is timed in breakdown_us",
            "kv_cache_copies": len(caches),
            "chunk_tokens": chunk,
            "rows_per_item": rows,
            "fp8_tile_buffers": args.fp8_tile_buffers or None,
            "work_items": hdr["items"],
            "shared_nodes": hdr["shared_nodes"],
        },
        "pct_hbm_peak_unique_bytes": round(unique_bytes / (step_us * 1e-6) / 1e9 / HBM_PEAK_GBS * 100, 2),
        "breakdown_us": {
            "attention_kernel": round(kern, 2) if kern else None,
            "merge_kernel": round(merge_us, 2) if merge_us is not None else None,
            "metadata_builder": round(build_us, 2),
            "metadata_update": round(update_us, 2),
            "metadata_per_step": round(update_us / args.layers, 2),
        },
        "roofline": {
            "kernel": "fca_attend_f32_kernel" if fp32 else "fca_attend64_kernel" if rows > 32 or w.head_dim == 256 else "fca_attend32_kernel",
            "bound": "hbm",
            "achieved": round(unique_bytes / (kern * 1e-6) / 1e9, 1) if kern else None,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(unique_bytes / (kern * 1e-6) / 1e9 / HBM_PEAK_GBS, 4) if kern else None,
            "traffic": MEASURED_TRAFFIC_BYTES.get((args.config, chunk, rows)) if args.shrink == 1 else None,
            "launches_timed": len(kern_us),  # 0 under rocprofv3: the trace has the durations
            "launch_us_mean": round(kern, 2) if kern else None,
            "launch_us_min": round(min(kern_us), 2) if kern_us else None,
            "launch_us_max": round(max(kern_us), 2) if kern_us else None,
        },
    }

    result["mfma_util"] = MEASURED_MFMA_UTIL.get((args.config, chunk, rows)) if args.shrink == 1 else None
    if split is not None:
        result["split_passes"] = split

    if args.calibrate:
        from arctic_platform_amd import _lib
        from arctic_platform_amd.forest import _stream_ptr

        src = torch.ones(1 << 28, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(_lib.load_library().fca_calibration_copy(src.data_ptr(), dst.data_ptr(), src.numel() * 4, _stream_ptr(dev)))
        torch.cuda.synchronize()
        result["calibration_copy_bytes"] = src.numel() * 4
        del src, dst

    if noncascade is not None:
        for key, entry in noncascade.items():
            entry["speedup_of_cascade"] = round(entry["us_per_step"] / step_us, 3)
            result[key] = entry

    if args.cpu_seqs > 0:
        result["cpu_baseline"] = cpu_baseline(torch, w, args.cpu_seqs, checked_rows)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()

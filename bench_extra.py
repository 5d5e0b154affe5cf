"""Secondary bench workloads (`bench.py --workload ...`): MLA decode at 64K context and chunked GQA prefill.
Same one-JSON-line contract as the default workload."""
from __future__ import annotations

import ctypes as C
import json
import os
import time

import numpy as np

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA peak
MLA_64K_TRAFFIC_BYTES = 210674278  # mla_partial_ws on seed 2's config 4: 177.0 MB read (cache rows: 172.0 MB) + 33.7 MB of split records written
HBM_PEAK_GBPS = 8000.0


def _event_ms(fn, steps):
    import torch

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def _wall_ms(fn, steps):
    """Wall clock per call over exactly `steps` calls, after 0.1 s of untimed calls: the device needs some milliseconds of
    work to return to its running clocks after the idle stretch a graph capture leaves."""
    import torch

    started = time.perf_counter()
    while time.perf_counter() - started < 0.1:
        fn()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def run_mla_decode(args):
    """benchmark configuration 3 (counted from 0): B=4, 128 heads, latent 512 (Q8g64, bf16 scales) + rope 64 (bf16), ctx 65,536,
    bf16 queries, softmax scale 1/sqrt(192); W_kv_b ~ N(0, 1/512) in bf16; 64-token pages in a random permutation."""
    import torch

    import oracle as O
    from zllm_amd import capi, ops

    dev = "cuda"
    batch, heads, nope, rope, value, latent, bt, ctx = 4, 128, 128, 64, 128, 512, 64, 65536
    lens = [ctx] * batch
    ops.init(0)
    rng = np.random.default_rng(args.seed)
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed)
    need_blocks = batch * ctx // bt
    pool_blocks = max(need_blocks * 8, need_blocks + 1)
    rows = pool_blocks * bt
    codes = torch.empty((rows, latent), dtype=torch.int8, device=dev)
    scales = torch.empty((rows, latent // 64), dtype=torch.int16, device=dev)
    rope_cache = torch.empty((rows, rope), dtype=torch.int16, device=dev)
    ids = rng.choice(pool_blocks, size=need_blocks, replace=False).astype(np.uint32).reshape(batch, -1)
    tables = torch.from_numpy(ids.view(np.int32)).to(dev)
    for b in range(batch):
        for pos in range(0, ctx, 8192):
            lat = torch.randn((8192, latent), generator=gen, device=dev)
            kr = torch.randn((8192, rope), generator=gen, device=dev)
            ops.mla_append(lat, kr, codes, scales, rope_cache, tables[b], pos, bt)
    q = torch.randn((batch, heads * (nope + rope)), generator=gen, device=dev).to(torch.bfloat16)
    kv_b = (torch.randn((heads * (nope + value), latent), generator=gen, device=dev) / np.sqrt(latent)).to(torch.bfloat16)
    lens_dev = torch.tensor(lens, dtype=torch.int32, device=dev)
    call, out, workspace = ops.mla_decode_args(q, kv_b, codes, scales, rope_cache, tables, lens_dev, heads, nope + rope, nope + value,
                                               latent, rope, bt, ctx, out_dtype=torch.float32, out_compact=True)
    lib = capi.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def run(mask):
        def fn():
            call.stage_mask = mask
            capi.check(lib.zllm_attn_mla_decode(C.byref(call), stream))
        return fn

    for _ in range(args.warmup):
        run(0)()
    ms_eager = _wall_ms(run(0), args.steps)
    # The decode step is replayed from a HIP graph, as the reference replays its decode launches
    # (src/kernel/rocm/hip/graph.rs): same kernels, same arguments, without per-launch host overhead.  One graph holds
    # `per_graph` consecutive calls, the way a model step holds one attention call per layer.
    per_graph = max(g for g in range(1, 17) if args.steps % g == 0)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(0)()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        capture_stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        for _ in range(per_graph):
            call.stage_mask = 0
            capi.check(lib.zllm_attn_mla_decode(C.byref(call), capture_stream))
    replays = args.steps // per_graph
    for _ in range(max(1, args.warmup // per_graph)):
        graph.replay()
    ms_step = _wall_ms(graph.replay, replays) / per_graph
    ms_events = _event_ms(graph.replay, replays) / per_graph
    stage_ms = {name: _event_ms(run(mask), args.steps) for name, mask in
                (("absorb", capi.MLA_ABSORB), ("partial", capi.MLA_PARTIAL), ("merge_project", capi.MLA_MERGE | capi.MLA_PROJECT),
                 # the second split-KV kernel (ZLLM_MLA_WIDE_TILES), not the default: timed beside it
                 ("partial_wide_tiles", capi.MLA_PARTIAL | capi.MLA_WIDE_TILES))}
    singles = sorted(_event_ms(run(capi.MLA_PARTIAL), 1) for _ in range(max(args.steps, 100)))
    run(0)()
    torch.cuda.synchronize()
    flops = sum(lens) * heads * (2 * (latent + rope) + 2 * latent)  # QK^T over 576 + PV over 512, multiply-add = 2
    kv_bytes = sum(lens) * (latent + latent // 64 * 2 + rope * 2)   # 656 B/token
    tflops_call = flops / (ms_step * 1e-3) / 1e12
    achieved = flops / (stage_ms["partial"] * 1e-3) / 1e12
    record = {
        "metric": "MLA decode attn TFLOP/s (% of bf16 MFMA peak) + tokens/s at 64K ctx, 1 GPU",
        "value": round(tflops_call, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "C4 absorbed MLA decode, B=4, 128 heads, latent 512 Q8g64 + rope 64 bf16, ctx 65536, 64-token pages",
                   "algorithmic_flops_per_call": flops, "kv_bytes_per_call": kv_bytes, "seed": args.seed,
                   "q_head_dim": nope + rope, "kv_head_dim": nope + value},
        "pct_of_mfma_peak": round(100.0 * tflops_call / MFMA_BF16_PEAK_TFLOPS, 2),
        "tokens_per_s": round(batch / (ms_step * 1e-3), 1),
        "effective_kv_gbps": round(kv_bytes / (ms_step * 1e-3) / 1e9, 1),
        "ms_per_step_events": round(ms_events, 5), "ms_per_step_eager": round(ms_eager, 5),
        "launch": f"hipGraph replay, {per_graph} decode calls (absorb + partial + merge/project each) per graph; 0.1 s of untimed replays before the timed ones",
        "stage_ms": {k: round(v, 5) for k, v in stage_ms.items()},
        "roofline": {"bound": "mfma", "kernel": "mla_partial", "achieved": round(achieved, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": MLA_64K_TRAFFIC_BYTES if args.seed == 2 else None,
                     "traffic_source": "profiles/mla_partial_ws__mla_decode_64k.md: rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this workload, scaled by a 1 GiB copy; "
                                       "not read in this run" if args.seed == 2 else None,
                     "kernel_ms": round(stage_ms["partial"], 5), "kernel_ms_single_launch_median": round(singles[len(singles) // 2], 5),
                     "kernel_ms_single_launch_min": round(singles[0], 5),
                     "second_kernel_wide_tiles": {"kernel_ms": round(stage_ms["partial_wide_tiles"], 5),
                                                  "frac": round(flops / (stage_ms["partial_wide_tiles"] * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}},
    }
    if not args.no_cpu_baseline:
        # CPU oracle (port of mla_attention_absorbed_q8_history) on a bounded sample: sequence 0, the first 8 heads,
        # the first `sample_ctx` tokens of context.
        sample_heads, sample_ctx = 8, getattr(args, "oracle_sample_ctx", 16384)
        threads = O.set_threads(min(len(os.sched_getaffinity(0)), 16))
        h_codes = ops.gather_rows(codes, tables[0], 0, sample_ctx, latent, bt).cpu().numpy()
        h_scales = ops.gather_rows(scales, tables[0], 0, sample_ctx, latent // 64 * 2, bt).cpu().numpy().view(np.uint16)
        h_rope = ops.gather_rows(rope_cache, tables[0], 0, sample_ctx, rope * 2, bt).cpu().numpy().view(np.uint16)
        spec = O.MlaSpec(latent, rope, sample_heads * (nope + rope), sample_heads * (nope + value), sample_heads)
        q_bits = q[0].view(torch.int16).cpu().numpy().view(np.uint16)[: sample_heads * (nope + rope)].reshape(1, -1)
        w = kv_b.float().cpu().numpy()[: sample_heads * (nope + value)]
        t0 = time.perf_counter()
        rc, _, out_f, _ = O.mla_absorbed_q8_history(spec, q_bits, 1, sample_ctx - 1, h_codes, h_scales, 64, h_rope, sample_ctx, w)
        seconds = time.perf_counter() - t0
        assert rc == 0
        cpu_flops = sample_ctx * sample_heads * (2 * (latent + rope) + 2 * latent)
        record["cpu_baseline"] = {"value": round(cpu_flops / seconds / 1e12, 6), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                                  "sample": f"sequence 0, heads 0..{sample_heads - 1}, first {sample_ctx} tokens; {seconds:.2f}s "
                                            f"(one task per head, so {min(threads, sample_heads)} cores busy)"}
        # parity of the same slice on the device (separate small call)
        small = ops.mla_decode(q[0:1, : sample_heads * (nope + rope)].contiguous(), kv_b[: sample_heads * (nope + value)].contiguous(),
                               codes, scales, rope_cache, tables[0:1].contiguous(), torch.tensor([sample_ctx], dtype=torch.int32, device=dev),
                               sample_heads, nope + rope, nope + value, latent, rope, bt, sample_ctx)
        record["parity_vs_oracle_max_abs"] = float(np.abs(small.cpu().numpy().ravel() - out_f).max())
    return record


def run_mla_prefill(args):
    """Chunked MLA prefill: one sequence, a 512-row chunk appended to a 16,384-token prefix (causal inside the chunk),
    128 heads, latent 512 Q8g64 + rope 64 bf16, 64-token pages in a random permutation, bf16 queries and bf16 output.
    Every chunk row runs as one query row of the split-KV kernels over the same pages."""
    import torch

    import oracle as O
    from zllm_amd import capi, ops

    dev = "cuda"
    heads, nope, rope, value, latent, bt, prefix, rows = 128, 128, 64, 128, 512, 64, 16384, 512
    ctx = prefix + rows
    ops.init(0)
    rng = np.random.default_rng(args.seed)
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed)
    need_blocks = (ctx + bt - 1) // bt
    pool_blocks = need_blocks * 8
    pool_rows = pool_blocks * bt
    codes = torch.empty((pool_rows, latent), dtype=torch.int8, device=dev)
    scales = torch.empty((pool_rows, latent // 64), dtype=torch.int16, device=dev)
    rope_cache = torch.empty((pool_rows, rope), dtype=torch.int16, device=dev)
    ids = rng.choice(pool_blocks, size=need_blocks, replace=False).astype(np.uint32).reshape(1, -1)
    tables = torch.from_numpy(ids.view(np.int32)).to(dev)
    for pos in range(0, ctx, 2048):
        n = min(2048, ctx - pos)
        ops.mla_append(torch.randn((n, latent), generator=gen, device=dev), torch.randn((n, rope), generator=gen, device=dev), codes, scales,
                       rope_cache, tables[0], pos, bt)
    q = torch.randn((rows, heads * (nope + rope)), generator=gen, device=dev).to(torch.bfloat16)
    kv_b = (torch.randn((heads * (nope + value), latent), generator=gen, device=dev) / np.sqrt(latent)).to(torch.bfloat16)
    lens_dev = torch.tensor([ctx], dtype=torch.int32, device=dev)
    call, out, workspace = ops.mla_decode_args(q, kv_b, codes, scales, rope_cache, tables, lens_dev, heads, nope + rope, nope + value, latent,
                                               rope, bt, ctx, out_dtype=torch.bfloat16, out_compact=True, query_rows=rows)
    lib = capi.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def run(mask):
        def fn():
            call.stage_mask = mask
            capi.check(lib.zllm_attn_mla_decode(C.byref(call), stream))
        return fn

    steps, warmup = max(1, args.steps // 10), max(1, args.warmup // 10)
    for _ in range(warmup):
        run(0)()
    ms_step = _event_ms(run(0), steps)
    stage_ms = {name: _event_ms(run(mask), steps) for name, mask in
                (("absorb", capi.MLA_ABSORB), ("partial", capi.MLA_PARTIAL), ("merge_project", capi.MLA_MERGE | capi.MLA_PROJECT))}
    run(0)()
    torch.cuda.synchronize()
    pairs = rows * prefix + rows * (rows + 1) // 2
    flops = pairs * heads * (2 * (latent + rope) + 2 * latent)
    tflops = flops / (ms_step * 1e-3) / 1e12
    achieved = flops / (stage_ms["partial"] * 1e-3) / 1e12
    record = {
        "metric": "MLA chunked prefill attn TFLOP/s (% of bf16 MFMA peak), 1 GPU", "value": round(tflops, 1), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"absorbed MLA prefill chunk, B=1, {rows} rows on a {prefix}-token prefix, 128 heads, latent 512 Q8g64 + rope 64 bf16, 64-token pages",
                   "algorithmic_flops_per_call": flops, "seed": args.seed, "workspace_bytes": int(workspace.numel())},
        "pct_of_mfma_peak": round(100.0 * tflops / MFMA_BF16_PEAK_TFLOPS, 2),
        "tokens_per_s": round(rows / (ms_step * 1e-3), 1),
        "stage_ms": {k: round(v, 5) for k, v in stage_ms.items()},
        "roofline": {"bound": "mfma", "kernel": "mla_partial_ws", "achieved": round(achieved, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None, "kernel_ms": round(stage_ms["partial"], 5)},
    }
    if not args.no_cpu_baseline:
        # CPU oracle on a bounded sample: the last four chunk rows, heads 0..3, over the whole history
        sample_rows, sample_heads = 4, 4
        threads = O.set_threads(min(len(os.sched_getaffinity(0)), 16))
        h_codes = ops.gather_rows(codes, tables[0], 0, ctx, latent, bt).cpu().numpy()
        h_scales = ops.gather_rows(scales, tables[0], 0, ctx, latent // 64 * 2, bt).cpu().numpy().view(np.uint16)
        h_rope = ops.gather_rows(rope_cache, tables[0], 0, ctx, rope * 2, bt).cpu().numpy().view(np.uint16)
        spec = O.MlaSpec(latent, rope, sample_heads * (nope + rope), sample_heads * (nope + value), sample_heads)
        q_bits = q[rows - sample_rows:].view(torch.int16).cpu().numpy().view(np.uint16)[:, : sample_heads * (nope + rope)]
        w = kv_b.float().cpu().numpy()[: sample_heads * (nope + value)]
        t0 = time.perf_counter()
        rc, _, out_f, _ = O.mla_absorbed_q8_history(spec, np.ascontiguousarray(q_bits), sample_rows, ctx - sample_rows, h_codes, h_scales, 64, h_rope,
                                                    ctx, w)
        seconds = time.perf_counter() - t0
        assert rc == 0
        cpu_flops = sample_rows * ctx * sample_heads * (2 * (latent + rope) + 2 * latent)
        record["cpu_baseline"] = {"value": round(cpu_flops / seconds / 1e12, 6), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                                  "sample": f"last {sample_rows} chunk rows, heads 0..{sample_heads - 1}, {ctx} tokens; {seconds:.2f}s"}
        got = out[rows - sample_rows:].float().cpu().numpy().reshape(sample_rows, heads, value)[:, :sample_heads].reshape(-1)
        excess = np.abs(got - out_f) - np.abs(out_f) * 2.0 ** -7  # bf16 output: beyond one bf16 step of the oracle's unrounded value
        record["parity_vs_oracle_max_abs_beyond_bf16_step"] = float(max(excess.max(), 0.0))
    return record


def run_gqa_decode_f16(args):
    """C3: f16 KV cache, B=4, 16q/8kv, d=256, ctx 8192, soft-cap 50; the full layer and the sliding layer (window 1024) are
    timed as two calls of the same entry point.  `value` is the full layer (268 MB of KV per call)."""
    import torch

    import oracle as O
    from zllm_amd import capi, ops

    dev = torch.device("cuda:0")
    batch, hq, hkv, d, ctx, bt, window, softcap = 4, 16, 8, 256, 8192, 16, 1024, 50.0
    scale = 1.0 / 16.0  # 1/sqrt(256)
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    blocks_per_seq = ctx // bt
    pool_blocks = batch * blocks_per_seq * 8  # pages scattered over an 8x larger pool (~2 GiB per plane)
    rows = pool_blocks * bt
    k_plane = torch.empty((rows, hkv * d), dtype=torch.float16, device=dev)
    v_plane = torch.empty((rows, hkv * d), dtype=torch.float16, device=dev)
    perm = torch.randperm(pool_blocks, generator=gen, device=dev)[: batch * blocks_per_seq].to(torch.int32)
    tables = perm.view(batch, blocks_per_seq).contiguous()
    for b in range(batch):
        idx = (tables[b].long()[:, None] * bt + torch.arange(bt, device=dev)[None, :]).reshape(-1)
        k_plane[idx] = torch.randn((ctx, hkv * d), generator=gen, device=dev, dtype=torch.float32).to(torch.float16)
        v_plane[idx] = torch.randn((ctx, hkv * d), generator=gen, device=dev, dtype=torch.float32).to(torch.float16)
    q = torch.randn((batch, hq * d), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    lens = [ctx] * batch
    lens_dev = torch.tensor(lens, dtype=torch.int32, device=dev)
    first_dev = torch.tensor([ctx - window] * batch, dtype=torch.int32, device=dev)
    lib = capi.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    results = {}
    outs = {}
    for name, first, visible in (("full", None, ctx), ("window", first_dev, window)):
        call, out, workspace = ops.gqa_decode_args(q, k_plane, None, v_plane, None, tables, lens_dev, hq, hkv, d, bt, scale, ctx,
                                                   first_visible=first, softcap=softcap, kv_format=capi.KV_F16,
                                                   total_kv_tokens=visible * batch)

        def launch(stages, call=call):
            def fn():
                call.stages = stages
                capi.check(lib.zllm_attn_gqa_decode(C.byref(call), stream))
            return fn

        for _ in range(args.warmup):
            launch(capi.STAGE_ALL)()
        per_graph = max(g for g in range(1, 17) if args.steps % g == 0)
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            launch(capi.STAGE_ALL)()
        torch.cuda.current_stream().wait_stream(side)
        with torch.cuda.graph(graph):
            cap = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            for _ in range(per_graph):
                call.stages = capi.STAGE_ALL
                capi.check(lib.zllm_attn_gqa_decode(C.byref(call), cap))
        replays = args.steps // per_graph
        graph.replay()
        ms_step = _wall_ms(graph.replay, replays) / per_graph
        ms_partial = _event_ms(launch(capi.STAGE_PARTIAL), args.steps)
        launch(capi.STAGE_ALL)()
        torch.cuda.synchronize()
        kv_bytes = batch * visible * 2 * hkv * d * 2  # K + V, f16
        results[name] = {"ms_per_step": ms_step, "kernel_ms": ms_partial, "kv_bytes": kv_bytes}
        outs[name] = (out.clone(), call, workspace)
    full, win = results["full"], results["window"]
    gbps = full["kv_bytes"] / (full["ms_per_step"] * 1e-3) / 1e9
    achieved = full["kv_bytes"] / (full["kernel_ms"] * 1e-3) / 1e9
    record = {
        "metric": "f16-KV GQA decode attn effective KV GB/s (% of HBM peak) at 8K ctx, 1 GPU", "value": round(gbps, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(full["ms_per_step"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "C3 f16-KV GQA decode, B=4, 16q/8kv, d=256, ctx 8192, soft-cap 50, score_scale 1/16, 16-token pages; "
                               "full layer (value) and sliding layer (window 1024)",
                   "kv_bytes_per_call": full["kv_bytes"], "window_kv_bytes_per_call": win["kv_bytes"], "seed": args.seed},
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "tokens_per_s": round(batch / (full["ms_per_step"] * 1e-3), 1),
        "window_layer": {"ms_per_step": round(win["ms_per_step"], 5), "kernel_ms": round(win["kernel_ms"], 5),
                         "effective_kv_gbps": round(win["kv_bytes"] / (win["ms_per_step"] * 1e-3) / 1e9, 1),
                         "kernel_gbps": round(win["kv_bytes"] / (win["kernel_ms"] * 1e-3) / 1e9, 1)},
        "roofline": {"bound": "hbm", "kernel": "gqa_decode_f16_partial", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel_ms": round(full["kernel_ms"], 5)},
    }
    if not args.no_cpu_baseline:
        # CPU oracle on a bounded sample: sequence 0, all heads, both layer kinds
        threads = O.set_threads(min(len(os.sched_getaffinity(0)), 16))
        k_rows = ops.gather_rows(k_plane.view(torch.uint8), tables[0], 0, ctx, hkv * d * 2, bt).cpu().numpy().view(np.uint16)
        v_rows = ops.gather_rows(v_plane.view(torch.uint8), tables[0], 0, ctx, hkv * d * 2, bt).cpu().numpy().view(np.uint16)
        k_f32 = O.f16_to_f32(k_rows).reshape(ctx, hkv * d)
        v_f32 = O.f16_to_f32(v_rows).reshape(ctx, hkv * d)
        q_f32 = q[0:1].float().cpu().numpy()
        worst = 0.0
        seconds = 0.0
        for name, win_size in (("full", 0), ("window", window)):
            start, end = O.key_range(win_size, ctx - 1, ctx)
            t0 = time.perf_counter()
            rc, want = O.gqa_prefill_at_visible(q_f32, k_f32[start:end], v_f32[start:end], start, end, ctx - 1, hq, hkv, d,
                                                window=win_size, score_scale=scale, softcap=softcap)
            if name == "full":
                seconds = time.perf_counter() - t0
            assert rc == 0
            worst = max(worst, float(np.abs(outs[name][0][0].cpu().numpy().ravel() - want.ravel()).max()))
        record["cpu_baseline"] = {"value": round(ctx * 2 * hkv * d * 2 / seconds / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
                                  "sample": f"sequence 0 of the full layer ({ctx} keys, {hq} heads) on dequantised f32 K/V; {seconds:.2f}s"}
        record["parity_vs_oracle_max_abs"] = worst
    return record


def workload_record(args):
    """The JSON record of one secondary workload."""
    if args.workload == "mla_decode_64k":
        return run_mla_decode(args)
    if args.workload == "mla_prefill_chunk":
        return run_mla_prefill(args)
    if args.workload == "gqa_decode_f16_window":
        return run_gqa_decode_f16(args)
    import bench_prefill

    if args.workload == "gqa_prefill_chunk":
        return bench_prefill.run(args)
    if args.workload == "gqa_prefill_f16":
        return bench_prefill.run_f16(args)
    raise SystemExit(f"unknown workload {args.workload}")


def run(args):
    print(json.dumps(workload_record(args)))

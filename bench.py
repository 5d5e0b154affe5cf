#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

Default workload = benchmark configuration 1 (counted from 0): Qwen3-style Q8g64 GQA decode, batch 8, 64 query heads /
8 KV heads, head_dim 128, every sequence at 32,768 tokens (the "32K ctx" case the metric is quoted
on), 16-token pages scattered over a large pool, bf16 queries, K/V ~ N(0,1) with 1 % outlier
channels x8.  One "step" = one decode attention call (split-KV partial + LSE merge) over the batch.

Prints ONE JSON line.  `value` = effective KV GB/s of the whole call (KV codes + scales inside the
visible window, each counted once; inputs resident in HBM).  `roofline` prices the dominant kernel
(the split-KV partial kernel) alone, timed with HIP events on the launch stream.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E peak
# HBM bytes one launch of the partial kernel moves on the default workload: rocprofv3 FETCH_SIZE and WRITE_SIZE
# per dispatch, each scaled by what the same counter reads for a 1 GiB device copy (FETCH_SIZE x 2.0,
# WRITE_SIZE x 1.0); the runs and their numbers are in profiles/gqa_decode_q8_dma128__gqa_decode_32k.md.
GQA_32K_TRAFFIC_BYTES = 564179558
GQA_RAGGED_TRAFFIC_BYTES = 246880256  # seed 2's draw: profiles/gqa_decode_q8_dma128__gqa_decode_ragged.md
METRIC = "decode attn effective KV GB/s (% of HBM peak) + tokens/s at 32K ctx, 1 GPU"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="gqa_decode_32k",
                    choices=["gqa_decode_32k", "gqa_decode_ragged", "gqa_decode_c1", "mla_decode_64k", "mla_prefill_chunk", "gqa_prefill_chunk", "gqa_prefill_f16", "gqa_decode_f16_window", "copy_calibration", "append_prologue"])
    ap.add_argument("--pool-gib", type=float, default=256.0, help="address span of the paged pool (all four planes); clipped to 90 %% of free HBM")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true", help="default workload only: leave out the other configurations' entries")
    ap.add_argument("--seed", type=int, default=2)
    return ap.parse_args()


_PROBE = None


def probe_lib():
    """libbench_probe.so: plain-read measurement kernels (bench_probe.hip), outside the attention library."""
    global _PROBE
    if _PROBE is None:
        path = os.path.join(ROOT, "libbench_probe.so")
        if not os.path.exists(path):
            from zllm_amd.build import build_bench_probe

            build_bench_probe()
        lib = C.CDLL(path)
        lib.bench_probe_stream_read.restype = C.c_int
        lib.bench_probe_stream_read.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]
        lib.bench_probe_paged_read.restype = C.c_int
        lib.bench_probe_paged_read.argtypes = [C.c_void_p] * 5 + [C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        lib.bench_probe_paged_read_lds.restype = C.c_int
        lib.bench_probe_paged_read_lds.argtypes = lib.bench_probe_paged_read.argtypes
        _PROBE = lib
    return _PROBE


def stream_read_probe(buffer, sink):
    import torch

    rc = probe_lib().bench_probe_stream_read(buffer.data_ptr(), buffer.numel() * buffer.element_size(), sink.data_ptr(),
                                             torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc


def paged_read_probe(planes, table_flat, workgroups, pages_in_flight, sink, through_lds=False):
    import torch

    lib = probe_lib()
    rc = (lib.bench_probe_paged_read_lds if through_lds else lib.bench_probe_paged_read)(planes["k_codes"].data_ptr(), planes["v_codes"].data_ptr(), planes["k_scales"].data_ptr(),
                                            planes["v_scales"].data_ptr(), table_flat.data_ptr(), table_flat.numel(), workgroups, pages_in_flight,
                                            sink.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc


def event_time_ms(fn, steps):
    """Average duration per call of `fn` over `steps` back-to-back launches, by HIP events on the stream."""
    import torch

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def probe_times(fn, launches, kv_bytes):
    """A read probe timed both ways the decode kernel is: `kernel_ms` = one event pair around `launches` back-to-back
    launches (what roofline.kernel_ms is), and the median / minimum of single launches."""
    for _ in range(10):
        fn()
    mean = event_time_ms(fn, launches)
    med, low = event_times_ms(fn, launches)
    return {"kernel_ms": round(mean, 5), "kernel_ms_median": round(med, 5), "kernel_ms_min": round(low, 5),
            "gbps": round(kv_bytes / (mean * 1e-3) / 1e9, 1), "gbps_median": round(kv_bytes / (med * 1e-3) / 1e9, 1)}


def event_times_ms(fn, launches):
    """Per-launch durations (one HIP event pair around each of `launches` back-to-back launches): median and minimum, the
    reference's bench idiom (src/kernel/rocm/hip/attention/paged_mla.rs:6742-6759)."""
    import torch

    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(launches)]
    torch.cuda.synchronize()
    for start, stop in pairs:
        start.record()
        fn()
        stop.record()
    torch.cuda.synchronize()
    times = sorted(start.elapsed_time(stop) for start, stop in pairs)
    return times[len(times) // 2], times[0]


CLOCK_SETTLE_S = 0.1


def settle_clocks(fn, seconds=CLOCK_SETTLE_S):
    """Untimed calls of `fn` for `seconds`: after the idle stretch a graph capture or host-side set-up leaves, the
    device takes some milliseconds of work to return to its running clocks (measured: the first 25 ms region after a
    capture reads 3 to 11 % slow, every later one agrees with the event timeline)."""
    import torch

    started = time.perf_counter()
    while time.perf_counter() - started < seconds:
        fn()
        torch.cuda.synchronize()


def wall_time_ms(fn, steps, regions=1):
    """Wall clock per call over exactly `steps` calls, bracketed by synchronize, after settle_clocks.  With `regions` > 1 the
    region of `steps` calls is timed that many times back to back and the median region is returned (with the shortest and
    the longest one beside it)."""
    import torch

    settle_clocks(fn)
    times = []
    for _ in range(regions):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3 / steps)
    times.sort()
    if regions == 1:
        return times[0]
    return times[len(times) // 2], times[0], times[-1]


# ------------------------------------------------------------------------------------------- GQA decode
def build_gqa_pool(args, lens, hq, hkv, d, block_tokens):
    """Fill a paged Q8g64 pool on the device: K/V ~ N(0,1), 1 % outlier channels x8, quantized by the library's
    own append kernel (bit-exact with the oracle's quantizer), pages drawn without replacement from the pool."""
    import torch

    from zllm_amd import capi, ops

    dev = "cuda"
    cols = hkv * d
    groups = cols // 64
    bytes_per_row = 2 * (cols + groups * 2)
    free, _ = torch.cuda.mem_get_info()
    span = min(int(args.pool_gib * (1 << 30)), int(free * 0.90))
    need_blocks = sum((l + block_tokens - 1) // block_tokens for l in lens)
    pool_blocks = max(span // (bytes_per_row * block_tokens), need_blocks + 1)
    pool_rows = pool_blocks * block_tokens
    planes = dict(
        k_codes=torch.empty((pool_rows, cols), dtype=torch.int8, device=dev),
        k_scales=torch.empty((pool_rows, groups), dtype=torch.int16, device=dev),
        v_codes=torch.empty((pool_rows, cols), dtype=torch.int8, device=dev),
        v_scales=torch.empty((pool_rows, groups), dtype=torch.int16, device=dev),
    )
    rng = np.random.default_rng(args.seed)
    ids = rng.choice(pool_blocks, size=need_blocks, replace=False).astype(np.uint32)
    stride = max((l + block_tokens - 1) // block_tokens for l in lens)
    tables = np.zeros((len(lens), stride), dtype=np.uint32)
    at = 0
    for b, l in enumerate(lens):
        n = (l + block_tokens - 1) // block_tokens
        tables[b, :n] = ids[at:at + n]
        at += n
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed)
    gain = torch.ones(cols, device=dev)
    gain[torch.from_numpy(rng.choice(cols, size=max(1, cols // 100), replace=False)).to(dev)] = 8.0
    tables_dev = torch.from_numpy(tables.view(np.int32)).to(dev)
    step = 4096
    for b, l in enumerate(lens):
        for pos in range(0, l, step):
            n = min(step, l - pos)
            k = torch.randn((n, cols), generator=gen, device=dev) * gain
            v = torch.randn((n, cols), generator=gen, device=dev) * gain
            ops.q8g64_append(k, planes["k_codes"], planes["k_scales"], tables_dev[b], pos, block_tokens, capi.QUANT_METAL_GQA)
            ops.q8g64_append(v, planes["v_codes"], planes["v_scales"], tables_dev[b], pos, block_tokens, capi.QUANT_METAL_GQA)
    q = torch.randn((len(lens), hq * d), generator=gen, device=dev).to(torch.bfloat16)
    torch.cuda.synchronize()
    span_bytes = int(ids.max()) * block_tokens * cols
    return planes, tables, tables_dev, q, dict(pool_rows=pool_rows, pool_blocks=pool_blocks,
                                               pool_bytes=pool_rows * bytes_per_row, max_code_offset=span_bytes)


def gqa_cpu_baseline(planes, tables_dev, lens, q, hq, hkv, d, block_tokens, scale, budget_s=10.0):
    """The CPU oracle over the whole batch in the two modes the reference's CPU code has, each repeated until about
    `budget_s` seconds of CPU work are spent: `value` = dequantize the Q8g64 rows to f32, then causal_head_range per
    (token, head) task (what its CpuKvCache holds and runs); `direct_q8` = attention straight over the Q8 rows, values
    formed from the codes on the fly (the way its absorbed MLA path reads the Q8 latent)."""
    import oracle as O
    from zllm_amd import ops

    cols = hkv * d
    threads = O.set_threads(min(len(os.sched_getaffinity(0)), 16))
    host = []
    for b, l in enumerate(lens):
        rows = {}
        for name, width in (("k_codes", cols), ("k_scales", cols // 64 * 2), ("v_codes", cols), ("v_scales", cols // 64 * 2)):
            rows[name] = ops.gather_rows(planes[name], tables_dev[b], 0, l, width, block_tokens).cpu().numpy()
        host.append(rows)
    q_host = q.float().cpu().numpy()
    total_bytes = sum(lens) * 2 * (cols + cols // 64 * 2)
    outs = np.zeros((len(lens), hq * d), dtype=np.float32)
    passes, t_deq, t_att = [], 0.0, 0.0
    started = time.perf_counter()
    while time.perf_counter() - started < budget_s or not passes:
        p_deq = p_att = 0.0
        for b, l in enumerate(lens):
            t0 = time.perf_counter()
            k = O.gather_dequant_rows(O.FMT_Q8, host[b]["k_codes"].view(np.int8), host[b]["k_scales"].view(np.uint16), O.SCALE_F16,
                                      None, block_tokens, 0, l, cols)
            v = O.gather_dequant_rows(O.FMT_Q8, host[b]["v_codes"].view(np.int8), host[b]["v_scales"].view(np.uint16), O.SCALE_F16,
                                      None, block_tokens, 0, l, cols)
            t1 = time.perf_counter()
            rc, out = O.gqa_prefill_at_visible(q_host[b:b + 1], k, v, 0, l, l - 1, hq, hkv, d, score_scale=scale)
            t2 = time.perf_counter()
            assert rc == 0
            outs[b] = out[0]
            p_deq += t1 - t0
            p_att += t2 - t1
        passes.append(p_deq + p_att)
        t_deq += p_deq
        t_att += p_att
    median = float(np.median(passes))
    n = len(passes)
    direct_passes = []
    direct_out = np.zeros_like(outs)
    started = time.perf_counter()
    while time.perf_counter() - started < budget_s or not direct_passes:
        t0 = time.perf_counter()
        for b, l in enumerate(lens):
            rc, out = O.gqa_decode_q8_direct(q_host[b], host[b]["k_codes"], host[b]["k_scales"].view(np.uint16), host[b]["v_codes"],
                                             host[b]["v_scales"].view(np.uint16), O.SCALE_F16, 0, l, hq, hkv, d, scale)
            assert rc == 0
            direct_out[b] = out
        direct_passes.append(time.perf_counter() - t0)
    direct_median = float(np.median(direct_passes))
    return dict(value=round(total_bytes / median / 1e9, 3), unit="GB/s", cores=threads, kind="port",
                sample=f"whole batch ({len(lens)} sequences, all heads), {n} passes in {sum(passes):.1f}s, median pass {median:.3f}s; "
                       f"per pass: dequantize {t_deq / n:.3f}s + f32 attention {t_att / n:.3f}s",
                direct_q8=dict(value=round(total_bytes / direct_median / 1e9, 3), unit="GB/s", cores=threads,
                               sample=f"same batch, attention straight over the Q8g64 rows: {len(direct_passes)} passes, median pass {direct_median:.3f}s",
                               max_abs_vs_dequantize_mode=float(np.abs(direct_out - outs).max()))), outs


def run_gqa_decode(args, ragged, config1=False):
    import torch

    from zllm_amd import capi, ops

    hq, hkv, d, bt, batch = (16, 4, 128, 16, 1) if config1 else (64, 8, 128, 16, 8)
    rng = np.random.default_rng(args.seed)
    lens = [int(x) for x in rng.integers(1024, 32769, size=batch)] if ragged else [4096 if config1 else 32768] * batch
    scale = 1.0 / float(np.sqrt(d))
    ops.init(0)
    planes, tables, tables_dev, q, pool = build_gqa_pool(args, lens, hq, hkv, d, bt)
    lens_dev = torch.tensor(lens, dtype=torch.int32, device="cuda")
    call_args, out, workspace = ops.gqa_decode_args(q, planes["k_codes"], planes["k_scales"], planes["v_codes"], planes["v_scales"],
                                                    tables_dev, lens_dev, hq, hkv, d, bt, scale, max(lens),
                                                    kv_format=capi.KV_Q8G64, scale_dtype=capi.SCALE_F16, total_kv_tokens=sum(lens))
    lib = capi.load()

    def launch(stages):
        call_args.stages = stages
        capi.check(lib.zllm_attn_gqa_decode(C.byref(call_args), C.c_void_p(torch.cuda.current_stream().cuda_stream)))

    def full():
        launch(capi.STAGE_ALL)

    def partial_only():
        launch(capi.STAGE_PARTIAL)

    for _ in range(args.warmup):
        full()
    ms_eager = wall_time_ms(full, args.steps)
    # The decode step is replayed from a HIP graph, as the reference replays its decode launches
    # (src/kernel/rocm/hip/graph.rs): same kernels, same arguments, without per-launch host overhead.
    # One graph holds `per_graph` consecutive decode calls, the way a model step holds one attention call per
    # layer; `steps` calls are timed as steps / per_graph replays.
    per_graph = max(g for g in range(1, 17) if args.steps % g == 0)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        full()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        for _ in range(per_graph):
            full()
    replays = args.steps // per_graph
    for _ in range(max(1, args.warmup // per_graph)):
        graph.replay()
    # exactly `steps` calls make one timed region; the region is repeated and the median region is the step time
    regions = 11
    ms_step, ms_step_min, ms_step_max = (t / per_graph for t in wall_time_ms(graph.replay, replays, regions=regions))
    ms_events = event_time_ms(graph.replay, replays) / per_graph
    settle_clocks(partial_only)
    ms_partial = event_time_ms(partial_only, args.steps)  # one event pair around `steps` back-to-back launches
    ms_partial_median, ms_partial_min = event_times_ms(partial_only, max(args.steps, 100))
    out.zero_()
    graph.replay()
    torch.cuda.synchronize()

    bytes_per_token = 2 * (hkv * d + 2 * hkv * d // 64)  # 2,112 B: K+V codes + 16-bit scales
    kv_bytes = sum(lens) * bytes_per_token
    gbps = kv_bytes / (ms_step * 1e-3) / 1e9
    # the kernel figure is the median of per-launch event pairs (a mean over eager launches carries their launch gaps)
    achieved = kv_bytes / (ms_partial * 1e-3) / 1e9
    record = {
        "metric": METRIC, "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8+bf16", "data": "synthetic",
        "config": {"workload": ("C1 Q8g64 GQA decode, B=1, 16q/4kv, d=128, L=4096, 16-token pages (the reference's CPU-runnable case: latency-bound on a GPU)"
                                if config1 else "C2 Q8g64 GQA decode, B=8, 64q/8kv, d=128, " + ("ragged L~U[1024,32768]" if ragged else "all L=32768")
                                + ", 16-token pages"),
                   "kv_lens": lens, "kv_bytes_per_call": kv_bytes, "bytes_per_token": bytes_per_token, "seed": args.seed,
                   "pool_bytes": pool["pool_bytes"], "pool_blocks": pool["pool_blocks"], "max_code_plane_offset": pool["max_code_offset"],
                   "q_dtype": "bf16", "scale_dtype": "f16", "kv_arithmetic": "K.Q on int8 MFMA (K codes raw, Q as three 8-bit digits); P.V on bf16 MFMA (V codes exact in bf16); f32 accumulate"},
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "tokens_per_s": round(batch / (ms_step * 1e-3), 1),
        "ms_per_step_events": round(ms_events, 5),
        "ms_per_step_eager_launch": round(ms_eager, 5),
        "ms_per_step_regions": {"count": regions, "median": round(ms_step, 5), "min": round(ms_step_min, 5), "max": round(ms_step_max, 5)},
        "launch": f"hipGraph replay, {per_graph} decode calls (partial + merge each) per graph; {CLOCK_SETTLE_S} s of untimed replays, then {regions} "
                  f"regions of exactly {args.steps} steps each, bracketed by synchronize: ms_per_step is the median region",
        "roofline": {"bound": "hbm", "kernel": "gqa_decode_q8_dma128", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": None if config1 or args.seed != 2 else GQA_RAGGED_TRAFFIC_BYTES if ragged else GQA_32K_TRAFFIC_BYTES,
                     "traffic_source": None if config1 or args.seed != 2 else
                     f"profiles/gqa_decode_q8_dma128__gqa_decode_{'ragged' if ragged else '32k'}.md: rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this workload, "
                     "scaled by a 1 GiB copy; not read in this run",
                     "kernel_ms": round(ms_partial, 5), "kernel_ms_single_launch_median": round(ms_partial_median, 5),
                     "kernel_ms_single_launch_min": round(ms_partial_min, 5)},
    }
    if not config1:
        # what a kernel that only reads the same number of bytes reaches, timed the same way in the same process
        probe_src = torch.empty(kv_bytes // 16 * 16, dtype=torch.uint8, device="cuda").random_(0, 255)
        probe_sink = torch.full((1,), 7, dtype=torch.int32, device="cuda")
        record["roofline"]["plain_read_of_same_bytes"] = probe_times(lambda: stream_read_probe(probe_src, probe_sink), 100, probe_src.numel())
        del probe_src
        if not ragged:
            # the decode kernel's own access pattern without its arithmetic: same pages, same 128-byte lines per wave
            flat = tables_dev.reshape(-1).contiguous()
            paged = {}
            for in_flight in (1, 2, 4, 8):  # pages (33 KB each) a workgroup requests before it waits
                paged[f"{in_flight}_pages_in_flight"] = probe_times(lambda: paged_read_probe(planes, flat, 256, in_flight, probe_sink), 100, kv_bytes)
            for in_flight in (1, 2, 4):  # the same walk with the decode kernel's transport (global -> LDS loads)
                paged[f"{in_flight}_pages_in_flight_through_lds"] = probe_times(
                    lambda: paged_read_probe(planes, flat, 256, in_flight, probe_sink, through_lds=True), 100, kv_bytes)
            record["roofline"]["paged_read_of_same_pages"] = paged
    if not args.no_cpu_baseline:
        cpu, cpu_out = gqa_cpu_baseline(planes, tables_dev, lens, q, hq, hkv, d, bt, scale)
        record["cpu_baseline"] = cpu
        record["parity_vs_oracle_max_abs"] = float(np.abs(out.cpu().numpy() - cpu_out).max())
    elif getattr(args, "oracle_sequences", 0):
        # parity only (no CPU timing): the oracle on the first sequences of the batch
        n = args.oracle_sequences
        _, cpu_out = gqa_cpu_baseline(planes, tables_dev[:n], lens[:n], q[:n], hq, hkv, d, bt, scale, budget_s=0.0)
        record["parity_vs_oracle_max_abs"] = float(np.abs(out[:n].cpu().numpy() - cpu_out).max())
        record["parity_sample"] = f"first {n} sequences, all heads"
    return record


def run_append_prologue(args):
    """The steps in front of the attention call on every chunk of a prefill: the quantizing page appends and the fused
    prologue (per-head RMSNorm + RoPE, Q out, K/V into the pages), at chunk sizes, as bytes moved per second.  `value` is
    the prologue of a 2,048-row chunk (64 query / 8 KV heads, head_dim 128, bf16 in, bf16 Q out)."""
    import torch

    from zllm_amd import capi, ops

    ops.init(0)
    rng = np.random.default_rng(args.seed)
    dev = "cuda"
    bt = 16
    results = {}
    launches = max(10, min(args.steps, 50))

    def timed(fn):
        for _ in range(3):
            fn()
        settle_clocks(fn, 0.05)
        return event_time_ms(fn, launches)

    for rows in (2048, 8192):
        cols = 1024
        pool = (rows + bt - 1) // bt * 2 + 64
        table = torch.from_numpy(rng.choice(pool, size=(rows + bt - 1) // bt + 1, replace=False).astype(np.int32)).to(dev)
        codes = torch.zeros((pool * bt, cols), dtype=torch.int8, device=dev)
        scales = torch.zeros((pool * bt, cols // 64), dtype=torch.int16, device=dev)
        src = torch.randn((rows, cols), device=dev).to(torch.bfloat16)
        ms = timed(lambda: ops.q8g64_append(src, codes, scales, table, 0, bt, capi.QUANT_METAL_GQA))
        moved = rows * cols * 2 + rows * cols + rows * cols // 64 * 2
        results[f"q8g64_append_{rows}_rows_bf16"] = {"ms": round(ms, 5), "bytes": moved, "gbps": round(moved / ms / 1e6, 1)}
        cache = torch.zeros((pool * bt, cols), dtype=torch.float16, device=dev)
        ms = timed(lambda: ops.half_append(src, cache, table, 0, bt))
        moved = rows * cols * 4
        results[f"half_append_{rows}_rows_bf16"] = {"ms": round(ms, 5), "bytes": moved, "gbps": round(moved / ms / 1e6, 1)}
        latent = torch.randn((rows, 512), device=dev).to(torch.bfloat16)
        k_rope = torch.randn((rows, 64), device=dev).to(torch.bfloat16)
        pool64 = (rows + 63) // 64 * 2 + 8
        table64 = torch.from_numpy(rng.choice(pool64, size=(rows + 63) // 64 + 1, replace=False).astype(np.int32)).to(dev)
        lc = torch.zeros((pool64 * 64, 512), dtype=torch.int8, device=dev)
        ls = torch.zeros((pool64 * 64, 8), dtype=torch.int16, device=dev)
        rc = torch.zeros((pool64 * 64, 64), dtype=torch.int16, device=dev)
        latent_f32, rope_f32 = latent.float(), k_rope.float()
        ms = timed(lambda: ops.mla_append(latent_f32, rope_f32, lc, ls, rc, table64, 0, 64))
        moved = rows * (576 * 4 + 512 + 16 + 128)
        results[f"mla_append_{rows}_rows_f32"] = {"ms": round(ms, 5), "bytes": moved, "gbps": round(moved / ms / 1e6, 1)}
        hq, hkv, d = 64, 8, 128
        q = torch.randn((rows, hq * d), device=dev).to(torch.bfloat16)
        k = torch.randn((rows, hkv * d), device=dev).to(torch.bfloat16)
        v = torch.randn((rows, hkv * d), device=dev).to(torch.bfloat16)
        qn, kn = torch.ones(d, device=dev), torch.ones(d, device=dev)
        cos, sin = torch.ones((rows + 8, d // 2), device=dev), torch.zeros((rows + 8, d // 2), device=dev)
        v_codes, v_scales = torch.zeros_like(codes), torch.zeros_like(scales)
        ms = timed(lambda: ops.gqa_prologue(q, k, v, qn, kn, cos, sin, codes, scales, v_codes, v_scales, table, 0, hq, hkv, d, d, bt,
                                            q_out_dtype=torch.bfloat16))
        moved = rows * (hq * d * 2 * 2 + 2 * hkv * d * 2 + 2 * hkv * d + 2 * (hkv * d // 64) * 2 + d * 4)
        results[f"gqa_prologue_{rows}_rows_bf16"] = {"ms": round(ms, 5), "bytes": moved, "gbps": round(moved / ms / 1e6, 1)}
    head = results["gqa_prologue_2048_rows_bf16"]
    return ({"metric": "pre-attention prologue of a 2,048-row chunk, bytes moved per second", "value": head["gbps"], "unit": "GB/s",
                      "n_gpus": 1, "steps": launches, "warmup": 3, "ms_per_step": head["ms"], "higher_is_better": True, "dtype": "f32",
                      "data": "synthetic", "config": {"workload": "page appends and fused prologue at chunk sizes", **results},
                      "roofline": {"bound": "hbm", "kernel": "gqa_prologue_kernel", "achieved": head["gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                   "frac": round(head["gbps"] / HBM_PEAK_GBPS, 4), "traffic": None}})


def run_copy_calibration(args):
    """A plain device-to-device copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE counters of the
    attention kernels are scaled by (the counters do not report bytes one-to-one on this GPU)."""
    import torch

    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(args.warmup):
        dst.copy_(src)
    ms = event_time_ms(lambda: dst.copy_(src), args.steps)
    return {"metric": "device copy (counter calibration)", "value": round(2 * n / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
            "config": {"workload": "torch uint8 copy_", "bytes_read": n, "bytes_written": n}}


def other_configs(args):
    """The other benchmark configurations in the same process, each replayed or launched at least 100 times and checked
    against the oracle on a slice: the ragged draw of config 2, config 4 (MLA decode at 64K, the MFMA-bound one), config 5
    (the prefill chunk) and config 3 (f16 cache at head_dim 256, a full and a sliding-window layer).  Keys per entry: ms_per_step, value + unit, roofline {kernel, achieved, peak, frac, kernel_ms},
    parity_vs_oracle_max_abs."""
    import copy

    import torch

    import bench_extra

    def brief(record):
        keep = ("ms_per_step", "value", "unit", "steps", "pct_of_hbm_peak", "pct_of_mfma_peak", "tokens_per_s", "stage_ms", "parity_vs_oracle_max_abs",
                "parity_sample", "ms_per_step_regions", "window_layer")
        out = {k: record[k] for k in keep if k in record}
        out["workload"] = record["config"]["workload"]
        out["roofline"] = {k: v for k, v in record["roofline"].items() if k in ("bound", "kernel", "achieved", "peak", "unit", "frac", "kernel_ms",
                                                                                 "kernel_ms_single_launch_median", "kernel_ms_single_launch_min",
                                                                                 "second_kernel_wide_tiles", "traffic", "traffic_source")}
        if "cpu_baseline" in record:
            out["cpu_baseline"] = {k: record["cpu_baseline"][k] for k in ("value", "unit", "cores", "kind", "sample")}
        return out

    results = {}
    sub = copy.copy(args)
    sub.steps, sub.warmup = max(args.steps, 100), max(args.warmup, 10)
    sub.no_cpu_baseline, sub.oracle_sequences = True, 2
    results["gqa_decode_ragged"] = brief(run_gqa_decode(sub, ragged=True))
    torch.cuda.empty_cache()
    sub = copy.copy(args)
    sub.steps, sub.warmup = max(args.steps, 100), max(args.warmup, 10)
    sub.no_cpu_baseline, sub.oracle_sample_ctx, sub.workload = False, 4096, "mla_decode_64k"
    results["mla_decode_64k"] = brief(bench_extra.workload_record(sub))
    torch.cuda.empty_cache()
    sub = copy.copy(args)
    sub.steps, sub.warmup = 100, 5
    sub.no_cpu_baseline, sub.workload = False, "gqa_prefill_chunk"
    results["gqa_prefill_chunk"] = brief(bench_extra.workload_record(sub))
    torch.cuda.empty_cache()
    sub = copy.copy(args)
    sub.steps, sub.warmup = max(args.steps, 100), max(args.warmup, 10)
    sub.no_cpu_baseline, sub.workload = False, "gqa_decode_f16_window"
    results["gqa_decode_f16_window"] = brief(bench_extra.workload_record(sub))
    torch.cuda.empty_cache()
    return results


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build targets one MI355X; --gpus must be 1 (multi-GPU sharding is design-only)", file=sys.stderr)
        sys.exit(2)
    if args.workload == "gqa_decode_32k":
        import torch

        record = run_gqa_decode(args, ragged=False)
        if not args.no_other_configs:
            torch.cuda.empty_cache()
            record["other_configs"] = other_configs(args)
    elif args.workload == "gqa_decode_ragged":
        record = run_gqa_decode(args, ragged=True)
    elif args.workload == "gqa_decode_c1":
        record = run_gqa_decode(args, ragged=False, config1=True)
    elif args.workload == "copy_calibration":
        record = run_copy_calibration(args)
    elif args.workload == "append_prologue":
        record = run_append_prologue(args)
    else:
        import bench_extra

        record = bench_extra.workload_record(args)
    print(json.dumps(record))


if __name__ == "__main__":
    main()

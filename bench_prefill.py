"""bench.py --workload gqa_prefill_chunk: benchmark configuration 4 (counted from 0) — a 2,048-row chunk appended to a 50,000-token
Q8g64 prefix, 64q/8kv, d=128, bf16 Q/K/V, 16-token pages; the chunk's K/V are quantized into fresh pages inside the
timed step (append + attention), as the path does per chunk."""
from __future__ import annotations

import ctypes as C
import json
import os
import time

import numpy as np

from bench_extra import MFMA_BF16_PEAK_TFLOPS, _event_ms, _wall_ms


def run(args):
    import torch

    import oracle as O
    from zllm_amd import capi, ops

    dev = "cuda"
    hq, hkv, d, bt, prefix, chunk = 64, 8, 128, 16, 50000, 2048
    total = prefix + chunk
    cols = hkv * d
    ops.init(0)
    rng = np.random.default_rng(args.seed)
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed)
    need = (total + bt - 1) // bt
    pool_blocks = need * 16
    rows = pool_blocks * bt
    planes = dict(k_codes=torch.empty((rows, cols), dtype=torch.int8, device=dev), k_scales=torch.empty((rows, cols // 64), dtype=torch.int16, device=dev),
                  v_codes=torch.empty((rows, cols), dtype=torch.int8, device=dev), v_scales=torch.empty((rows, cols // 64), dtype=torch.int16, device=dev))
    table = torch.from_numpy(rng.choice(pool_blocks, size=need, replace=False).astype(np.uint32).view(np.int32)).to(dev)
    for pos in range(0, prefix, 5000):
        n = min(5000, prefix - pos)
        k = torch.randn((n, cols), generator=gen, device=dev).to(torch.bfloat16)
        v = torch.randn((n, cols), generator=gen, device=dev).to(torch.bfloat16)
        ops.q8g64_append(k, planes["k_codes"], planes["k_scales"], table, pos, bt, capi.QUANT_METAL_GQA)
        ops.q8g64_append(v, planes["v_codes"], planes["v_scales"], table, pos, bt, capi.QUANT_METAL_GQA)
    q = torch.randn((chunk, hq * d), generator=gen, device=dev).to(torch.bfloat16)
    kc = torch.randn((chunk, cols), generator=gen, device=dev).to(torch.bfloat16)
    vc = torch.randn((chunk, cols), generator=gen, device=dev).to(torch.bfloat16)
    scale = 1.0 / float(np.sqrt(d))
    out = torch.empty((chunk, hq * d), dtype=torch.float32, device=dev)

    def attend():
        return ops.gqa_prefill_chunk(q, planes["k_codes"], planes["k_scales"], planes["v_codes"], planes["v_scales"], table, prefix,
                                     hq, hkv, d, bt, scale)

    def step():
        ops.q8g64_append(kc, planes["k_codes"], planes["k_scales"], table, prefix, bt, capi.QUANT_METAL_GQA)
        ops.q8g64_append(vc, planes["v_codes"], planes["v_scales"], table, prefix, bt, capi.QUANT_METAL_GQA)
        return attend()

    for _ in range(args.warmup):
        step()
    ms_step = _wall_ms(step, args.steps)
    ms_attn = _event_ms(attend, args.steps)
    result = step()
    torch.cuda.synchronize()
    pairs = chunk * prefix + chunk * (chunk + 1) // 2
    flops = 4 * d * hq * pairs  # QK^T + PV, multiply-add = 2
    tflops = flops / (ms_step * 1e-3) / 1e12
    achieved = flops / (ms_attn * 1e-3) / 1e12
    record = {
        "metric": "chunked-prefill GQA attn TFLOP/s (% of bf16 MFMA peak), 2048-row chunk on a 50K prefix, 1 GPU",
        "value": round(tflops, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "C5 chunked prefill GQA, B=1, 2048-row chunk on a 50,000-token Q8g64 prefix, 64q/8kv, d=128, 16-token pages",
                   "algorithmic_flops_per_call": flops, "causal_pairs_per_head": pairs, "seed": args.seed},
        "pct_of_mfma_peak": round(100.0 * tflops / MFMA_BF16_PEAK_TFLOPS, 2),
        "prefill_tokens_per_s": round(chunk / (ms_step * 1e-3), 1),
        "roofline": {"bound": "mfma", "kernel": "gqa_prefill_q8", "achieved": round(achieved, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None, "kernel_ms": round(ms_attn, 4)},
    }
    if not args.no_cpu_baseline:
        # CPU oracle on a bounded sample: the LAST 16 rows of the chunk, all 64 heads, against the full 52,048-token cache
        sample = 16
        threads = O.set_threads(min(len(os.sched_getaffinity(0)), 16))
        host = {n: ops.gather_rows(planes[n], table, 0, total, planes[n].shape[1] * planes[n].element_size(), bt).cpu().numpy() for n in planes}
        t0 = time.perf_counter()
        kd = O.gather_dequant_rows(O.FMT_Q8, host["k_codes"].view(np.int8), host["k_scales"].view(np.uint16), O.SCALE_F16, None, bt, 0, total, cols)
        vd = O.gather_dequant_rows(O.FMT_Q8, host["v_codes"].view(np.int8), host["v_scales"].view(np.uint16), O.SCALE_F16, None, bt, 0, total, cols)
        t1 = time.perf_counter()
        qs = q[chunk - sample:].float().cpu().numpy()
        rc, want = O.gqa_prefill_at_visible(qs, kd, vd, 0, total, total - sample, hq, hkv, d, score_scale=scale)
        t2 = time.perf_counter()
        assert rc == 0
        cpu_pairs = sum(total - sample + r + 1 for r in range(sample))
        record["cpu_baseline"] = {"value": round(4 * d * hq * cpu_pairs / (t2 - t1) / 1e12, 5), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                                  "sample": f"last {sample} rows of the chunk, all heads, full cache; attention {t2 - t1:.2f}s (+ dequantize {t1 - t0:.2f}s, not counted)"}
        record["parity_vs_oracle_max_abs"] = float(np.abs(result[chunk - sample:].cpu().numpy() - want).max())
    return record


def run_f16(args):
    """bench.py --workload gqa_prefill_f16: the prefill of benchmark configuration 2's model family (counted from 0) -- f16 K/V, 16 query
    heads / 8 KV heads, head_dim 256, soft-cap 50 -- as one 2,048-row chunk on a 6,144-token prefix (context 8,192), global causal layer
    (`value`) and the 1,024-token sliding-window layer beside it."""
    import torch

    import oracle as O
    from zllm_amd import capi, ops

    dev = "cuda"
    hq, hkv, d, bt, prefix, chunk, window, softcap = 16, 8, 256, 16, 6144, 2048, 1024, 50.0
    total = prefix + chunk
    cols = hkv * d
    ops.init(0)
    rng = np.random.default_rng(args.seed)
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed)
    need = (total + bt - 1) // bt
    pool_blocks = need * 16
    k_plane = torch.zeros((pool_blocks * bt, cols), dtype=torch.float16, device=dev)
    v_plane = torch.zeros((pool_blocks * bt, cols), dtype=torch.float16, device=dev)
    table = torch.from_numpy(rng.choice(pool_blocks, size=need, replace=False).astype(np.uint32).view(np.int32)).to(dev)
    k = torch.randn((total, cols), generator=gen, device=dev)
    v = torch.randn((total, cols), generator=gen, device=dev)
    ops.half_append(k, k_plane, table, 0, bt)
    ops.half_append(v, v_plane, table, 0, bt)
    q = torch.randn((chunk, hq * d), generator=gen, device=dev).to(torch.bfloat16)
    scale = 1.0 / float(np.sqrt(d))

    def attend(win):
        return lambda: ops.gqa_prefill_chunk(q, k_plane, None, v_plane, None, table, prefix, hq, hkv, d, bt, scale, window=win, softcap=softcap,
                                             kv_format=capi.KV_F16)

    results = {}
    for name, win in (("global", 0), ("sliding", window)):
        for _ in range(args.warmup):
            attend(win)()
        ms = _event_ms(attend(win), args.steps)
        pairs = sum(min(prefix + r + 1, win) if win else prefix + r + 1 for r in range(chunk))
        flops = 4 * d * hq * pairs
        results[name] = {"ms_per_step": ms, "pairs": pairs, "flops": flops, "tflops": flops / (ms * 1e-3) / 1e12}
    result = attend(0)()
    torch.cuda.synchronize()
    g = results["global"]
    record = {
        "metric": "f16-KV chunked-prefill GQA attn TFLOP/s (% of f16 MFMA peak), 2048-row chunk at 8K ctx, 1 GPU",
        "value": round(g["tflops"], 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(g["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "f16-KV chunked prefill GQA, B=1, 2048-row chunk on a 6,144-token prefix, 16q/8kv, d=256, soft-cap 50, 16-token pages",
                   "algorithmic_flops_per_call": g["flops"], "causal_pairs_per_head": g["pairs"], "seed": args.seed},
        "pct_of_mfma_peak": round(100.0 * g["tflops"] / MFMA_BF16_PEAK_TFLOPS, 2),
        "prefill_tokens_per_s": round(chunk / (g["ms_per_step"] * 1e-3), 1),
        "window_layer": {"ms_per_step": round(results["sliding"]["ms_per_step"], 4), "tflops": round(results["sliding"]["tflops"], 1)},
        "roofline": {"bound": "mfma", "kernel": "gqa_prefill_tiles", "achieved": round(g["tflops"], 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(g["tflops"] / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None, "kernel_ms": round(g["ms_per_step"], 4)},
    }
    if not args.no_cpu_baseline:
        sample = 16
        threads = O.set_threads(min(len(os.sched_getaffinity(0)), 16))
        kd = ops.gather_rows(k_plane, table, 0, total, cols * 2, bt).view(torch.float16).float().cpu().numpy()
        vd = ops.gather_rows(v_plane, table, 0, total, cols * 2, bt).view(torch.float16).float().cpu().numpy()
        qs = q[chunk - sample:].float().cpu().numpy()
        t1 = time.perf_counter()
        rc, want = O.gqa_prefill_at_visible(qs, kd, vd, 0, total, total - sample, hq, hkv, d, score_scale=scale, softcap=softcap)
        t2 = time.perf_counter()
        assert rc == 0
        cpu_pairs = sum(total - sample + r + 1 for r in range(sample))
        record["cpu_baseline"] = {"value": round(4 * d * hq * cpu_pairs / (t2 - t1) / 1e12, 5), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                                  "sample": f"last {sample} rows of the chunk, all heads, full cache; attention {t2 - t1:.2f}s"}
        record["parity_vs_oracle_max_abs"] = float(np.abs(result[chunk - sample:].cpu().numpy() - want).max())
    return record

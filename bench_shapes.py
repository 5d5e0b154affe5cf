"""Shape sweeps beside bench.py: the same entry points as the headline workloads over the shapes a serving stack
produces -- batches that do not divide the CU count, multi-GB batches, one or two KV heads (a GPU's share under tensor
parallelism), one sequence alone on the GPU, short chunks over long prefixes and first chunks at position 0, MLA decode
batches and one-sequence MLA decode at the reference test's head shape.  One JSON line per case.  These are the cases
the split planner, the items-per-workgroup rule, the wide split merges, the few-rows route, half-size row tiles and KV
splits of the chunk kernels, and the matrix-core and narrow MLA stages exist for; run it after touching any of them.

    python bench_shapes.py [--suite gqa_decode|gqa_heads|prefill_chunks|mla_batches|all] [--pool-gib 40]
"""
import argparse
import ctypes as C
import json
import sys

import numpy as np


def _time_us(fn, launches=30):
    import bench

    for _ in range(3):
        fn()
    bench.settle_clocks(fn, 0.05)
    return bench.event_time_ms(fn, launches) * 1e3


def gqa_decode_cases(args, geometries, shapes):
    import torch

    import bench
    from zllm_amd import capi, ops

    lib = capi.load()
    for hq, hkv, d in geometries:
        batch_max = max(b for b, _ in shapes)
        len_max = max(l for _, l in shapes)
        build = argparse.Namespace(pool_gib=args.pool_gib, seed=2)
        planes, tables, tables_dev, q, pool = bench.build_gqa_pool(build, [len_max] * batch_max, hq, hkv, d, 16)
        for batch, length in shapes:
            lens = torch.tensor([length] * batch, dtype=torch.int32, device="cuda")
            call, out, ws = ops.gqa_decode_args(q[:batch].contiguous(), planes["k_codes"], planes["k_scales"], planes["v_codes"], planes["v_scales"],
                                                tables_dev[:batch].contiguous(), lens, hq, hkv, d, 16, 1.0 / float(np.sqrt(d)), length,
                                                scale_dtype=capi.SCALE_F16, total_kv_tokens=batch * length)

            def launch(stages):
                def fn():
                    call.stages = stages
                    capi.check(lib.zllm_attn_gqa_decode(C.byref(call), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
                return fn

            kernel_us, call_us = _time_us(launch(capi.STAGE_PARTIAL)), _time_us(launch(capi.STAGE_ALL))
            chunk, chunks = C.c_uint32(), C.c_uint32()
            lib.zllm_attn_gqa_decode_split_plan(C.byref(call), C.byref(chunk), C.byref(chunks))
            kv_bytes = batch * length * 2 * (hkv * d + 2 * hkv * d // 64)
            print(json.dumps({"suite": "gqa_decode", "heads": f"{hq}q/{hkv}kv", "head_dim": d, "batch": batch, "kv_len": length,
                              "kv_mb": round(kv_bytes / 1e6, 1), "split_plan": f"{chunk.value} tokens x {chunks.value}",
                              "partial_us": round(kernel_us, 1), "call_us": round(call_us, 1),
                              "partial_gbps": round(kv_bytes / kernel_us / 1e3), "call_gbps": round(kv_bytes / call_us / 1e3)}), flush=True)
        del planes
        torch.cuda.empty_cache()


def prefill_chunk_cases(args):
    import torch

    from zllm_amd import capi, ops

    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    rng = np.random.default_rng(3)
    hq, hkv, d, bt = 32, 8, 128, 16
    prefix_max, chunk_max = 32768, 2048
    total, cols = prefix_max + chunk_max, hkv * d
    need = (total + bt - 1) // bt
    pool = need * 2
    planes = {n: torch.empty((pool * bt, cols if n[1] == "c" else cols // 64), dtype=torch.int8 if n[1] == "c" else torch.int16, device="cuda")
              for n in ("kc", "ks", "vc", "vs")}
    table = torch.from_numpy(rng.choice(pool, size=need, replace=False).astype(np.uint32).view(np.int32)).to("cuda")
    for name in ("k", "v"):
        rows = torch.randn((total, cols), generator=gen, device="cuda").to(torch.bfloat16)
        ops.q8g64_append(rows, planes[name + "c"], planes[name + "s"], table, 0, bt, capi.QUANT_METAL_GQA)
    lib = capi.load()
    for prefix in (0, 2048, 32768):  # position 0: a prompt's first chunk, whose row tiles' ranges grow from nothing
        for chunk in (1, 2, 4, 8, 64, 256, 512, 2048) if prefix else (128, 512, 2048):
            q = torch.randn((chunk, hq * d), generator=gen, device="cuda").to(torch.bfloat16)
            times = {}
            for label, workspace in (("with_workspace", True), ("without_workspace", False)):
                call, out, scratch = ops.gqa_prefill_chunk_args(q, planes["kc"], planes["ks"], planes["vc"], planes["vs"], table, prefix, hq, hkv,
                                                                d, bt, 1.0 / float(np.sqrt(d)), workspace=workspace)
                times[label] = _time_us(lambda: capi.check(lib.zllm_attn_gqa_prefill_chunk(C.byref(call), C.c_void_p(torch.cuda.current_stream().cuda_stream))),
                                        launches=5)
            pairs = sum(prefix + r + 1 for r in range(chunk))
            flops = 4 * d * hq * pairs
            print(json.dumps({"suite": "prefill_chunks", "heads": f"{hq}q/{hkv}kv", "head_dim": d, "prefix": prefix, "chunk_rows": chunk,
                              "kv_splits_us": round(times["with_workspace"], 1), "unsplit_us": round(times["without_workspace"], 1),
                              "kv_splits_tflops": round(flops / times["with_workspace"] / 1e6, 1)}), flush=True)


def mla_batch_cases(args):
    import torch

    from zllm_amd import capi, ops

    rope, latent, bt = 64, 512, 64
    ops.init(0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(2)
    rng = np.random.default_rng(2)
    pool = 8 * 131072 // bt * 2
    codes = torch.randint(-127, 127, (pool * bt, latent), dtype=torch.int8, device="cuda")
    scales = torch.full((pool * bt, latent // 64), 0x3C00, dtype=torch.int16, device="cuda")
    rope_cache = torch.zeros((pool * bt, rope), dtype=torch.int16, device="cuda")
    lib = capi.load()
    # 128 heads over batch sizes; then one sequence of 32 and 64 heads at long contexts, the shape of the reference's own
    # split-decode latency test (src/kernel/rocm/hip/attention/paged_mla.rs:6243-6253: a GPU's half of the heads)
    shapes = [(128, batch, ctx, 128, 128) for batch in (1, 3, 4, 13, 16, 32, 64) for ctx in (2048, 16384)]
    shapes += [(heads, 1, ctx, 192, 256) for heads in (32, 64) for ctx in (2048, 16384, 131072)]  # q_head 256, kv_head 448
    for heads, batch, ctx, nope, value in shapes:
        kv_b = (torch.randn((heads * (nope + value), latent), generator=gen, device="cuda") / np.sqrt(latent)).to(torch.bfloat16)
        need = batch * ctx // bt
        tables = torch.from_numpy(rng.choice(pool, size=need, replace=False).astype(np.uint32).reshape(batch, -1).view(np.int32)).to("cuda")
        q = torch.randn((batch, heads * (nope + rope)), generator=gen, device="cuda").to(torch.bfloat16)
        lens = torch.tensor([ctx] * batch, dtype=torch.int32, device="cuda")
        call, out, ws = ops.mla_decode_args(q, kv_b, codes, scales, rope_cache, tables, lens, heads, nope + rope, nope + value, latent, rope, bt, ctx)

        def launch(mask):
            def fn():
                call.stage_mask = mask
                capi.check(lib.zllm_attn_mla_decode(C.byref(call), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
            return fn

        stage = {name: round(_time_us(launch(mask), launches=20), 1) for name, mask in (("absorb", 1), ("partial", 2), ("merge_project", 12), ("call", 0))}
        flops = batch * ctx * heads * (2 * 576 + 2 * 512)
        print(json.dumps({"suite": "mla_batches", "batch": batch, "heads": heads, "q_head_dim": nope + rope, "kv_head_dim": nope + value, "ctx": ctx, "stage_us": stage,
                          "call_tflops": round(flops / stage["call"] / 1e6, 1)}), flush=True)
    # one long sequence among short ones, with and without the token-count hint
    heads, nope, value = 128, 128, 128
    kv_b = (torch.randn((heads * (nope + value), latent), generator=gen, device="cuda") / np.sqrt(latent)).to(torch.bfloat16)
    batch, lens_host = 32, [65536] + [2048] * 31
    need = sum(l // bt for l in lens_host)
    ids = rng.choice(pool, size=need, replace=False).astype(np.uint32)
    tables_host = np.zeros((batch, 65536 // bt), dtype=np.uint32)
    at = 0
    for b, l in enumerate(lens_host):
        tables_host[b, : l // bt] = ids[at: at + l // bt]
        at += l // bt
    tables = torch.from_numpy(tables_host.view(np.int32)).to("cuda")
    q = torch.randn((batch, heads * (nope + rope)), generator=gen, device="cuda").to(torch.bfloat16)
    lens = torch.tensor(lens_host, dtype=torch.int32, device="cuda")
    for label, hint in (("without_hint", 0), ("with_hint", sum(lens_host))):
        call, out, ws = ops.mla_decode_args(q, kv_b, codes, scales, rope_cache, tables, lens, heads, nope + rope, nope + value, latent, rope, bt,
                                            65536, total_ctx_tokens=hint)

        def whole():
            capi.check(lib.zllm_attn_mla_decode(C.byref(call), C.c_void_p(torch.cuda.current_stream().cuda_stream)))

        print(json.dumps({"suite": "mla_batches", "batch": batch, "ctx": "65536 + 31 x 2048", "plan": label, "call_us": round(_time_us(whole, launches=10), 1),
                          "workspace_mb": round(ws.numel() / 1e6, 1)}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--suite", default="all", choices=["gqa_decode", "gqa_heads", "prefill_chunks", "mla_batches", "all"])
    ap.add_argument("--pool-gib", type=float, default=40.0)
    args = ap.parse_args()
    from zllm_amd import ops

    ops.init(0)
    if args.suite in ("gqa_decode", "all"):
        gqa_decode_cases(args, [(64, 8, 128)], [(8, 32768), (12, 32768), (5, 65536), (16, 65536), (24, 2048), (3, 8192), (128, 1024), (512, 2048)])
    if args.suite in ("gqa_heads", "all"):
        gqa_decode_cases(args, [(32, 4, 128), (16, 2, 128), (8, 1, 128), (8, 1, 64), (4, 1, 256)], [(8, 32768), (32, 8192)])
        # one sequence alone on the GPU: the reference's embedded engine decodes one request at a time, and its standard
        # model has 16 query / 2 KV heads of 256 (src/runtime/ornith/mod.rs:709-720)
        gqa_decode_cases(args, [(16, 2, 256), (64, 8, 128)], [(1, 32768), (1, 131072)])
    if args.suite in ("prefill_chunks", "all"):
        prefill_chunk_cases(args)
    if args.suite in ("mla_batches", "all"):
        mla_batch_cases(args)


if __name__ == "__main__":
    sys.exit(main())

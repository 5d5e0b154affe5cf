"""Explicit per-row visible ranges (`visible_starts` + `visible_ends` of zllm_attn_gqa_prefill_chunk) against the CPU oracle of
`attention::block::attention_f32` (src/attention/block.rs:67-119): BlockAttentionSpec::visible, its varlen form (isolated
segments, src/attention/block.rs:41-63) and asymmetric windows, over Q8g64 and f16 caches, through every route of the entry
point (the chunk kernels, with and without KV splits, and rows run as decode items)."""
import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, draw_tables, to_torch_bf16, upload

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def varlen_ranges(query_offsets, kv_offsets):
    """BlockAttentionSpec::varlen: every query row of segment i sees the KV rows of segment i."""
    ranges = []
    for (q0, q1), (k0, k1) in zip(zip(query_offsets[:-1], query_offsets[1:]), zip(kv_offsets[:-1], kv_offsets[1:])):
        ranges += [(k0, k1)] * (q1 - q0)
    return np.asarray(ranges, dtype=np.uint32)


def run_block(seed, q_rows, kv_rows, hq, hkv, d, visible, kv="q8", q_kind="bf16", block_tokens=16, workspace=True, scale=None, layout="random"):
    from zllm_amd import capi, ops

    rng = np.random.default_rng(seed)
    cols = hkv * d
    cache_rows = max(kv_rows, q_rows)  # the entry point's bound on what it may read is position + rows
    position = cache_rows - q_rows
    tables, pool_blocks = draw_tables(rng, [cache_rows], block_tokens, layout=layout)
    pool = pool_blocks * block_tokens
    k = rng.standard_normal((kv_rows, cols)).astype(np.float32)
    v = rng.standard_normal((kv_rows, cols)).astype(np.float32)
    q = rng.standard_normal((q_rows, hq * d)).astype(np.float32)
    q_bits = O.f32_to_bf16(q)
    if q_kind == "bf16":
        q = O.bf16_to_f32(q_bits)
    scale = scale or 1.0 / np.sqrt(d)
    if kv == "q8":
        planes = {n: np.zeros((pool, cols if "codes" in n else cols // 64), dtype=np.int8 if "codes" in n else np.uint16)
                  for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
        O.q8g64_append_paged(O.RULE_METAL_GQA, k, planes["k_codes"], planes["k_scales"], tables[0], 0, block_tokens)
        O.q8g64_append_paged(O.RULE_METAL_GQA, v, planes["v_codes"], planes["v_scales"], tables[0], 0, block_tokens)
        kd = O.gather_dequant_rows(O.FMT_Q8, planes["k_codes"], planes["k_scales"], O.SCALE_F16, tables[0], block_tokens, 0, kv_rows, cols)
        vd = O.gather_dequant_rows(O.FMT_Q8, planes["v_codes"], planes["v_scales"], O.SCALE_F16, tables[0], block_tokens, 0, kv_rows, cols)
        dev = [upload(planes[n]) for n in ("k_codes", "k_scales", "v_codes", "v_scales")]
        fmt = capi.KV_Q8G64
    else:
        kc = np.zeros((pool, cols), dtype=np.uint16)
        vc = np.zeros((pool, cols), dtype=np.uint16)
        O.half_append_paged(1, k, kc, tables[0], 0, block_tokens)
        O.half_append_paged(1, v, vc, tables[0], 0, block_tokens)
        kd, vd = k.astype(np.float16).astype(np.float32), v.astype(np.float16).astype(np.float32)
        dev = [upload(kc).view(torch.float16), None, upload(vc).view(torch.float16), None]
        fmt = capi.KV_F16
    visible = np.ascontiguousarray(visible, dtype=np.uint32)
    q_dev = to_torch_bf16(q_bits, "cuda") if q_kind == "bf16" else upload(q)
    out = ops.gqa_prefill_chunk(q_dev, dev[0], dev[1], dev[2], dev[3], upload(tables[0]), position, hq, hkv, d, block_tokens, scale,
                                kv_format=fmt, visible_starts=upload(visible[:, 0].copy()), visible_ends=upload(visible[:, 1].copy()),
                                workspace=workspace)
    torch.cuda.synchronize()
    rc, want = O.block_attention(q, kd, vd, hq, hkv, d, scale, visible)
    assert rc == 0
    return out.cpu().numpy(), want


def test_reference_vectors():
    """src/attention/block.rs:125-141: zero queries, so every row is the mean of the values it sees -- [4, 4, 30] for the
    varlen offsets Q [0, 2, 3] / KV [0, 3, 5] over values 2 4 6 20 40, and [4, 8] for the ranges 0..2 and 1..3 over 2 6 10."""
    from zllm_amd import ops

    d, bt = 128, 16
    for values, visible, want in (([2.0, 4.0, 6.0, 20.0, 40.0], varlen_ranges([0, 2, 3], [0, 3, 5]), [4.0, 4.0, 30.0]),
                                  ([2.0, 6.0, 10.0], np.array([[0, 2], [1, 3]], dtype=np.uint32), [4.0, 8.0])):
        kv_rows, q_rows = len(values), len(want)
        v = np.zeros((kv_rows, d), dtype=np.float32)
        v[:, 0] = values
        planes = {n: np.zeros((bt, d if "codes" in n else d // 64), dtype=np.int8 if "codes" in n else np.uint16)
                  for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
        table = np.array([0], dtype=np.uint32)
        O.q8g64_append_paged(O.RULE_METAL_GQA, np.zeros_like(v), planes["k_codes"], planes["k_scales"], table, 0, bt)
        O.q8g64_append_paged(O.RULE_METAL_GQA, v, planes["v_codes"], planes["v_scales"], table, 0, bt)
        q = torch.zeros((q_rows, d), dtype=torch.float32, device="cuda")
        out = ops.gqa_prefill_chunk(q, upload(planes["k_codes"]), upload(planes["k_scales"]), upload(planes["v_codes"]), upload(planes["v_scales"]),
                                    upload(table), kv_rows - q_rows, 1, 1, d, bt, 1.0, visible_starts=upload(visible[:, 0].copy()),
                                    visible_ends=upload(visible[:, 1].copy()))
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        np.testing.assert_allclose(got[:, 0], want, rtol=2e-3)
        assert (got[:, 1:] == 0).all()


@pytest.mark.parametrize("kv,d,hq,hkv,q_kind,block_tokens", [("q8", 128, 16, 4, "bf16", 16), ("q8", 128, 8, 2, "f32", 64), ("q8", 64, 8, 2, "bf16", 16),
                                                             ("q8", 256, 8, 2, "bf16", 16), ("f16", 128, 8, 2, "bf16", 16), ("f16", 256, 16, 8, "f32", 16)])
def test_varlen_segments(kv, d, hq, hkv, q_kind, block_tokens):
    """Isolated sequences packed into one call: query segments of 1 to 300 rows against KV segments of other lengths."""
    q_off = [0, 1, 40, 340, 357]
    kv_off = [0, 700, 733, 1500, 1501]
    visible = varlen_ranges(q_off, kv_off)
    out, want = run_block(10 + d + hq, q_off[-1], kv_off[-1], hq, hkv, d, visible, kv=kv, q_kind=q_kind, block_tokens=block_tokens)
    assert_attention_close(out, want, f"varlen {kv} d={d}")


@pytest.mark.parametrize("workspace", [True, False])
def test_random_ranges_and_fewer_keys_than_rows(workspace):
    """Arbitrary [start, end) per row (not monotone, not causal), one-key rows, and a call with more query rows than cache
    rows; with the workspace a short chunk is cut into KV splits, without it the chunk kernel walks the ranges unsplit."""
    rng = np.random.default_rng(77)
    q_rows, kv_rows = 48, 5000
    starts = rng.integers(0, kv_rows - 1, size=q_rows)
    ends = np.minimum(starts + rng.integers(1, 3000, size=q_rows), kv_rows)
    starts[5], ends[5] = 4321, 4322
    visible = np.stack([starts, ends], axis=1)
    out, want = run_block(78, q_rows, kv_rows, 16, 4, 128, visible, workspace=workspace)
    assert_attention_close(out, want, "random ranges")
    q_rows, kv_rows = 300, 70
    starts = rng.integers(0, kv_rows - 1, size=q_rows)
    ends = np.minimum(starts + rng.integers(1, 70, size=q_rows), kv_rows)
    out, want = run_block(79, q_rows, kv_rows, 8, 2, 128, np.stack([starts, ends], axis=1), workspace=workspace)
    assert_attention_close(out, want, "more rows than keys")


def test_few_rows_over_a_long_range_run_as_decode_items():
    """Two rows over 20,000 keys: with the workspace the rows become items of the split-KV decode kernels."""
    visible = np.array([[100, 19000], [7, 20000]], dtype=np.uint32)
    out, want = run_block(80, 2, 20000, 32, 8, 128, visible)
    assert_attention_close(out, want, "decode items with explicit ranges")


def test_an_empty_range_gives_a_zero_row_and_bad_arguments_are_refused():
    from zllm_amd import capi, ops

    visible = np.array([[10, 10], [0, 50], [60, 20]], dtype=np.uint32)  # the reference refuses empty ranges; the device zeroes the row
    rng = np.random.default_rng(81)
    cols = 2 * 128
    k = rng.standard_normal((64, cols)).astype(np.float32)
    planes = {n: np.zeros((64, cols if "codes" in n else cols // 64), dtype=np.int8 if "codes" in n else np.uint16)
              for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
    O.q8g64_append_paged(O.RULE_METAL_GQA, k, planes["k_codes"], planes["k_scales"], None, 0, 16)
    O.q8g64_append_paged(O.RULE_METAL_GQA, k, planes["v_codes"], planes["v_scales"], None, 0, 16)
    q = torch.randn((3, 8 * 128), device="cuda").to(torch.bfloat16)
    dev = [upload(planes[n]) for n in ("k_codes", "k_scales", "v_codes", "v_scales")]
    got = ops.gqa_prefill_chunk(q, *dev, None, 61, 8, 2, 128, 16, 0.09, visible_starts=upload(visible[:, 0].copy()),
                                visible_ends=upload(visible[:, 1].copy())).cpu().numpy()
    assert not got[0].any() and not got[2].any() and got[1].any()
    with pytest.raises(capi.ZllmAttnError, match="visible_starts"):
        ops.gqa_prefill_chunk(q, *dev, None, 61, 8, 2, 128, 16, 0.09, visible_starts=upload(visible[:, 0].copy()))
    with pytest.raises(capi.ZllmAttnError, match="visible_starts"):
        ops.gqa_prefill_chunk(q, *dev, None, 61, 8, 2, 128, 16, 0.09, window=8, visible_starts=upload(visible[:, 0].copy()),
                              visible_ends=upload(visible[:, 1].copy()))

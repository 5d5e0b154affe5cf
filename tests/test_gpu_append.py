"""Bit-exact parity of the page appends and the row gather with the CPU oracle (through the C ABI)."""
import numpy as np
import pytest

import oracle as O
from tests.cases import draw_tables, upload

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def _planes(rows, cols, sdt):
    codes = torch.zeros((rows, cols), dtype=torch.int8, device="cuda")
    scales = torch.zeros((rows, cols // 64), dtype=torch.float32 if sdt == O.SCALE_F32 else torch.int16, device="cuda")
    return codes, scales


@pytest.mark.parametrize("rule", [O.RULE_ROCM_MLA, O.RULE_METAL_GQA, O.RULE_CUDA_GQA])
@pytest.mark.parametrize("block_tokens,layout", [(16, "random"), (64, "reversed"), (1, "random"), (4, "identity"), (128, "random")])
def test_q8g64_append_bit_exact(rule, block_tokens, layout):
    from zllm_amd import ops

    rng = np.random.default_rng(100 + rule * 10 + block_tokens)
    cols, total = 1024, 203
    sdt = {0: O.SCALE_BF16, 1: O.SCALE_F16, 2: O.SCALE_F32}[rule]
    tables, pool_blocks = draw_tables(rng, [total], block_tokens, layout=layout)
    rows = pool_blocks * block_tokens
    x = rng.standard_normal((total, cols)).astype(np.float32)
    x[:, rng.choice(cols, 10, replace=False)] *= 8.0
    x[5, 64:128] = 0.0  # all-zero group -> scale 1.0
    x[7, :64] = 1e-30  # tiny magnitudes
    x[9, 128:192] *= 1e4
    ref_codes = np.zeros((rows, cols), dtype=np.int8)
    ref_scales = np.zeros((rows, cols // 64), dtype=np.float32 if sdt == O.SCALE_F32 else np.uint16)
    codes, scales = _planes(rows, cols, sdt)
    table = upload(tables[0])
    # two appends: [0, 150) then [150, total) -> the second must land at absolute rows
    for start, stop in ((0, 150), (150, total)):
        O.q8g64_append_paged(rule, x[start:stop], ref_codes, ref_scales, tables[0], start, block_tokens)
        ops.q8g64_append(upload(x[start:stop]), codes, scales, table, start, block_tokens, rule)
    torch.cuda.synchronize()
    got_scales = scales.cpu().numpy().view(ref_scales.dtype)
    assert np.array_equal(got_scales, ref_scales), "scale bits differ"
    assert np.array_equal(codes.cpu().numpy(), ref_codes), "codes differ"


@pytest.mark.parametrize("src", ["bf16", "f16"])
def test_q8g64_append_half_sources(src):
    from zllm_amd import ops

    rng = np.random.default_rng(7)
    x32 = rng.standard_normal((40, 512)).astype(np.float32)
    if src == "bf16":
        xb = O.bf16_to_f32(O.f32_to_bf16(x32))
        dev = upload(O.f32_to_bf16(x32)).view(torch.bfloat16)
    else:
        xb = x32.astype(np.float16).astype(np.float32)
        dev = upload(x32.astype(np.float16))
    ref_codes = np.zeros((48, 512), dtype=np.int8)
    ref_scales = np.zeros((48, 8), dtype=np.uint16)
    O.q8g64_append_paged(O.RULE_METAL_GQA, xb, ref_codes, ref_scales, None, 3, 16)
    codes, scales = _planes(48, 512, O.SCALE_F16)
    ops.q8g64_append(dev, codes, scales, None, 3, 16, O.RULE_METAL_GQA)
    torch.cuda.synchronize()
    assert np.array_equal(codes.cpu().numpy(), ref_codes)
    assert np.array_equal(scales.cpu().numpy().view(np.uint16), ref_scales)


def test_q8g64_append_position_from_device_memory():
    """Graph-replay form: the row comes from positions[0] on the device (source.hip:787-807)."""
    from zllm_amd import ops

    rng = np.random.default_rng(8)
    x = rng.standard_normal((1, 256)).astype(np.float32)
    ref_codes = np.zeros((64, 256), dtype=np.int8)
    ref_scales = np.zeros((64, 4), dtype=np.uint16)
    O.q8g64_append_paged(O.RULE_METAL_GQA, x, ref_codes, ref_scales, None, 37, 16)
    codes, scales = _planes(64, 256, O.SCALE_F16)
    positions = upload(np.array([37, 0], dtype=np.uint32))
    ops.q8g64_append(upload(x), codes, scales, None, 0, 16, O.RULE_METAL_GQA, positions=positions)
    torch.cuda.synchronize()
    assert np.array_equal(codes.cpu().numpy(), ref_codes)
    assert np.array_equal(scales.cpu().numpy().view(np.uint16), ref_scales)


def test_ring_append_and_gather():
    from zllm_amd import ops

    rng = np.random.default_rng(9)
    cap, cols, total = 32, 256, 75
    x = rng.standard_normal((total, cols)).astype(np.float32)
    ref = np.zeros((cap, cols), dtype=np.uint16)
    O.half_append_paged(1, x, ref, None, 0, 16, ring_capacity=cap)
    cache = torch.zeros((cap, cols), dtype=torch.float16, device="cuda")
    # a chunk longer than the ring writes only its surviving tail (HybridGqaCacheLayout::write_plan)
    for pos, cnt in ((0, 50), (50, 25)):
        plan = O.ring_write_plan(cap, 1 << 20, pos, cnt)
        src = x[pos + plan["source_start"]: pos + cnt]
        assert len(src) == plan["token_count"] <= cap
        ops.half_append(upload(src), cache, None, pos + plan["source_start"], 16, ring_capacity=cap)
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy().view(np.uint16), ref)
    got = ops.gather_rows(cache, None, total - cap, cap, cols * 2, 16, ring_capacity=cap).cpu().numpy()
    want = O.gather_rows_bytes(ref, None, 16, total - cap, cap, cols * 2, ring_capacity=cap)
    assert np.array_equal(got, want)
    assert np.array_equal(got.view(np.float16).reshape(cap, cols), x[total - cap:].astype(np.float16))


@pytest.mark.parametrize("block_tokens,row_bytes", [(16, 1024), (16, 32), (64, 656), (4, 6), (128, 130)])
def test_gather_rows_bit_exact(block_tokens, row_bytes):
    from zllm_amd import ops

    rng = np.random.default_rng(block_tokens + row_bytes)
    total = 333
    tables, pool_blocks = draw_tables(rng, [total], block_tokens)
    plane = rng.integers(0, 256, size=(pool_blocks * block_tokens, row_bytes), dtype=np.uint8)
    got = ops.gather_rows(upload(plane), upload(tables[0]), 5, total - 5, row_bytes, block_tokens).cpu().numpy()
    want = O.gather_rows_bytes(plane, tables[0], block_tokens, 5, total - 5, row_bytes)
    assert np.array_equal(got, want)
    # identity table == no table
    got2 = ops.gather_rows(upload(plane), None, 5, 100, row_bytes, block_tokens).cpu().numpy()
    assert np.array_equal(got2, plane[5:105])


@pytest.mark.parametrize("layout,rotary_dim", [(1, 64), (0, 64), (1, 32), (1, 0)])
def test_mla_append_bit_exact(layout, rotary_dim):
    """Latent Q8 (bf16 scale, rounded-scale codes) + rotated bf16 rope in one launch."""
    from zllm_amd import ops

    rng = np.random.default_rng(50 + layout + rotary_dim)
    rows, latent_cols, rope_cols, block, position = 37, 512, 64, 16, 21
    tables, pool_blocks = draw_tables(rng, [position + rows], block)
    latent = rng.standard_normal((rows, latent_cols)).astype(np.float32)
    k_rope = rng.standard_normal((rows, rope_cols)).astype(np.float32)
    half = max(rotary_dim // 2, 1)
    angles = rng.uniform(0, 6.28, size=(position + rows + 3, half)).astype(np.float32)
    cos, sin = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
    pool = pool_blocks * block
    ref_codes = np.zeros((pool, latent_cols), dtype=np.int8)
    ref_scales = np.zeros((pool, latent_cols // 64), dtype=np.uint16)
    ref_rope = np.zeros((pool, rope_cols), dtype=np.uint16)
    O.q8g64_append_paged(O.RULE_ROCM_MLA, latent, ref_codes, ref_scales, tables[0], position, block)
    rotated = k_rope
    if rotary_dim:
        # oracle layout 0 = SplitHalf, 1 = Interleaved; ABI 1 = split-half, 0 = interleaved
        rc, rotated = O.rope_apply(k_rope, 1, rotary_dim, position + 2, cos, sin, layout=0 if layout == 1 else 1, placement=1)
        assert rc == 0
    O.half_append_paged(0, rotated, ref_rope, tables[0], position, block)
    codes = torch.zeros((pool, latent_cols), dtype=torch.int8, device="cuda")
    scales = torch.zeros((pool, latent_cols // 64), dtype=torch.int16, device="cuda")
    rope_cache = torch.zeros((pool, rope_cols), dtype=torch.int16, device="cuda")
    ops.mla_append(upload(latent), upload(k_rope), codes, scales, rope_cache, upload(tables[0]), position, block,
                   cos=upload(cos) if rotary_dim else None, sin=upload(sin) if rotary_dim else None,
                   rotary_dim=rotary_dim, rotary_layout=layout, rope_position=position + 2)
    torch.cuda.synchronize()
    assert np.array_equal(codes.cpu().numpy(), ref_codes)
    assert np.array_equal(scales.cpu().numpy().view(np.uint16), ref_scales)
    assert np.array_equal(rope_cache.cpu().numpy().view(np.uint16), ref_rope)


@pytest.mark.parametrize("layout,rotary_dim,rows", [(1, 64, 1), (0, 64, 1), (1, 32, 5), (1, 0, 3)])
def test_mla_append_positions_from_device_memory(layout, rotary_dim, rows):
    """Graph-replay form of the fused MLA append (paged_cache_append_mla_f32_q8_bf16_indirect, paged_mla/source.hip:787-807,
    launcher paged_mla.rs:960-1036): the cache row comes from positions[0] and the rope-table row from positions[1], both
    in device memory; the host-side numbers of the argument block are deliberately wrong and must not be used."""
    from zllm_amd import ops

    rng = np.random.default_rng(900 + layout + rotary_dim + rows)
    latent_cols, rope_cols, block = 512, 64, 16
    pool_rows = 160
    tables, pool_blocks = draw_tables(rng, [pool_rows], block)
    pool = pool_blocks * block
    half = max(rotary_dim // 2, 1)
    angles = rng.uniform(0, 6.28, size=(pool_rows + 16, half)).astype(np.float32)
    cos, sin = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
    ref_codes = np.zeros((pool, latent_cols), dtype=np.int8)
    ref_scales = np.zeros((pool, latent_cols // 64), dtype=np.uint16)
    ref_rope = np.zeros((pool, rope_cols), dtype=np.uint16)
    codes = torch.zeros((pool, latent_cols), dtype=torch.int8, device="cuda")
    scales = torch.zeros((pool, latent_cols // 64), dtype=torch.int16, device="cuda")
    rope_cache = torch.zeros((pool, rope_cols), dtype=torch.int16, device="cuda")
    table = upload(tables[0])
    positions = torch.zeros(2, dtype=torch.int32, device="cuda")
    dev_cos, dev_sin = (upload(cos), upload(sin)) if rotary_dim else (None, None)
    # three appends through one argument shape; only the device words move (a page boundary is crossed on the way)
    for position, rope_position in ((13, 13), (13 + rows, 20), (47, 3)):
        latent = rng.standard_normal((rows, latent_cols)).astype(np.float32)
        k_rope = rng.standard_normal((rows, rope_cols)).astype(np.float32)
        O.q8g64_append_paged(O.RULE_ROCM_MLA, latent, ref_codes, ref_scales, tables[0], position, block)
        rotated = k_rope
        if rotary_dim:
            rc, rotated = O.rope_apply(k_rope, 1, rotary_dim, rope_position, cos, sin, layout=0 if layout == 1 else 1, placement=1)
            assert rc == 0
        O.half_append_paged(0, rotated, ref_rope, tables[0], position, block)
        positions.copy_(upload(np.array([position, rope_position], dtype=np.uint32)).view(torch.int32))
        ops.mla_append(upload(latent), upload(k_rope), codes, scales, rope_cache, table, 99, block, cos=dev_cos, sin=dev_sin,
                       rotary_dim=rotary_dim, rotary_layout=layout, rope_position=77, positions=positions)
    torch.cuda.synchronize()
    assert np.array_equal(codes.cpu().numpy(), ref_codes), "codes differ"
    assert np.array_equal(scales.cpu().numpy().view(np.uint16), ref_scales), "scale bits differ"
    assert np.array_equal(rope_cache.cpu().numpy().view(np.uint16), ref_rope), "rope bits differ"

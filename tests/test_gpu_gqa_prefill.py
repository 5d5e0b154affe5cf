"""Parity of chunked-prefill GQA attention (new chunk quantized into fresh pages, then attended causally against the
Q8g64 prefix) with the CPU oracle `prefill_attention_at_visible_with_dot_f32` (src/attention/gqa.rs:243-282)."""
import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, draw_tables, to_torch_bf16, upload

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def run_case(seed, prefix, chunk, hq, hkv, window=0, softcap=0.0, block_tokens=16, rule=O.RULE_METAL_GQA, q_bf16=True,
             out_dtype=None, scale=None, outliers=False, gate_cols=0, q_gain=1.0, k_gain=1.0, v_gain=1.0, oracle_segments=None,
             d=128, visible_ends=None, workspace=True):
    from zllm_amd import capi, ops

    out_dtype = out_dtype or torch.float32
    rng = np.random.default_rng(seed)
    cols = hkv * d
    total = prefix + chunk
    tables, pool_blocks = draw_tables(rng, [total], block_tokens)
    rows = pool_blocks * block_tokens
    sdt = {O.RULE_METAL_GQA: O.SCALE_F16, O.RULE_ROCM_MLA: O.SCALE_BF16, O.RULE_CUDA_GQA: O.SCALE_F32}[rule]
    gain = np.ones(cols, dtype=np.float32)
    if outliers:  # 1 % of the channels carry values eight times larger
        gain[rng.choice(cols, size=max(1, cols // 100), replace=False)] = 8.0
    # q_gain / k_gain / v_gain: a factor, or one factor per token (rows of the chunk for q), for the magnitude tests
    k = rng.standard_normal((total, cols)).astype(np.float32) * gain * np.reshape(np.asarray(k_gain, dtype=np.float32), (-1, 1))
    v = rng.standard_normal((total, cols)).astype(np.float32) * gain * np.reshape(np.asarray(v_gain, dtype=np.float32), (-1, 1))
    # the chunk's K/V arrive as bf16 activations
    k[prefix:] = O.bf16_to_f32(O.f32_to_bf16(k[prefix:]))
    v[prefix:] = O.bf16_to_f32(O.f32_to_bf16(v[prefix:]))
    planes = {n: np.zeros((rows, cols if "codes" in n else cols // 64),
                          dtype=np.int8 if "codes" in n else (np.float32 if rule == O.RULE_CUDA_GQA else np.uint16))
              for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
    # prefix already cached (oracle quantizer); host copy of the full cache for the oracle
    O.q8g64_append_paged(rule, k, planes["k_codes"], planes["k_scales"], tables[0], 0, block_tokens)
    O.q8g64_append_paged(rule, v, planes["v_codes"], planes["v_scales"], tables[0], 0, block_tokens)
    dev = {n: upload(a) for n, a in planes.items()}
    table = upload(tables[0])
    # wipe the chunk's pages on the device, then let the library quantize the new rows into them
    first_new_block = prefix // block_tokens
    for n in dev:
        for blk in tables[0][first_new_block + (1 if prefix % block_tokens else 0):]:
            dev[n][int(blk) * block_tokens:(int(blk) + 1) * block_tokens] = 0
    kc = to_torch_bf16(O.f32_to_bf16(k[prefix:]), "cuda")
    vc = to_torch_bf16(O.f32_to_bf16(v[prefix:]), "cuda")
    ops.q8g64_append(kc, dev["k_codes"], dev["k_scales"], table, prefix, block_tokens, rule)
    ops.q8g64_append(vc, dev["v_codes"], dev["v_scales"], table, prefix, block_tokens, rule)
    torch.cuda.synchronize()
    for n in dev:  # appended bytes == oracle bytes on every row the sequence owns
        got = ops.gather_rows(dev[n], table, 0, total, planes[n].shape[1] * planes[n].itemsize, block_tokens).cpu().numpy()
        want = O.gather_rows_bytes(planes[n], tables[0], block_tokens, 0, total, planes[n].shape[1] * planes[n].itemsize)
        assert np.array_equal(got, want), n
    q = rng.standard_normal((chunk, hq * d)).astype(np.float32) * np.reshape(np.asarray(q_gain, dtype=np.float32), (-1, 1))
    q_bits = O.f32_to_bf16(q)
    q = O.bf16_to_f32(q_bits) if q_bf16 else q
    scale = scale or 1.0 / np.sqrt(d)
    gate = (rng.standard_normal((chunk, gate_cols)) * 3).astype(np.float32) if gate_cols else None
    out = ops.gqa_prefill_chunk(to_torch_bf16(q_bits, "cuda") if q_bf16 else upload(q), dev["k_codes"], dev["k_scales"], dev["v_codes"],
                                dev["v_scales"], table, prefix, hq, hkv, d, block_tokens, scale, window=window, softcap=softcap,
                                scale_dtype=sdt, out_dtype=out_dtype, gate=None if gate is None else upload(gate),
                                visible_ends=None if visible_ends is None else upload(np.asarray(visible_ends, dtype=np.uint32)),
                                workspace=workspace)
    torch.cuda.synchronize()
    kd = O.gather_dequant_rows(O.FMT_Q8, planes["k_codes"], planes["k_scales"], sdt, tables[0], block_tokens, 0, total, cols)
    vd = O.gather_dequant_rows(O.FMT_Q8, planes["v_codes"], planes["v_scales"], sdt, tables[0], block_tokens, 0, total, cols)
    if oracle_segments is not None:
        # the oracle on a few runs of chunk rows only (a full-size chunk is hours of scalar work): rows [r0, r0 + n) are a
        # chunk of their own appended at prefix + r0; key_range caps every row at its own position
        parts = []
        for r0, n in oracle_segments:
            rc, part = O.gqa_prefill_at_visible(q[r0:r0 + n], kd, vd, 0, total, prefix + r0, hq, hkv, d, window=window, score_scale=scale,
                                                softcap=softcap)
            assert rc == 0
            parts.append(part)
        return out, np.concatenate(parts)
    rc, want = O.gqa_prefill_at_visible(q, kd, vd, 0, total, prefix, hq, hkv, d, window=window, score_scale=scale, softcap=softcap,
                                        visible_ends=None if visible_ends is None else np.asarray(visible_ends, dtype=np.uint32))
    assert rc == 0
    if gate is not None:
        rc, want = O.sigmoid_gate(want, gate)
        assert rc == 0
    return out, want


@pytest.mark.parametrize("d,prefix,chunk,hq,hkv,window,softcap,extra", [
    (128, 5000, 24, 16, 2, 0, 0.0, ""), (128, 3000, 300, 8, 2, 700, 0.0, ""), (128, 2500, 70, 32, 4, 0, 30.0, "gate"),
    (128, 4000, 33, 8, 1, 0, 0.0, "bf16out"), (128, 2000, 90, 8, 2, 0, 0.0, "ends"), (64, 3000, 20, 8, 2, 0, 0.0, ""),
    (256, 3000, 20, 8, 2, 500, 0.0, ""), (128, 2600, 40, 16, 4, 0, 0.0, "f32scales"),
    # more than 64 splits a row and few rows: the records go through the wide split merge
    (128, 24000, 8, 16, 2, 0, 0.0, "gate"), (128, 20000, 12, 32, 4, 0, 0.0, "bf16out")])
def test_prefill_kv_splits_and_the_unsplit_kernel_agree(d, prefix, chunk, hq, hkv, window, softcap, extra):
    """A short chunk over a long prefix is cut into KV splits when the caller brings the workspace for their records (parts
    of a row tile's visible range, merged like a decode call's splits) and runs unsplit without one: both against the oracle.
    Covered: row tiles whose range is shorter than the longest (parts beyond their own count stay empty), windows, the soft
    cap, gates, bf16 output, explicit visible ends, f32 scales, head_dim 64 / 256 and outlier channels (the V window of a
    split differs from its neighbours')."""
    kw = dict(window=window, softcap=softcap, outliers=True, d=d)
    if extra == "gate":
        kw["gate_cols"] = hq * d
    if extra == "bf16out":
        kw["out_dtype"] = torch.bfloat16
    if extra == "ends":
        ends = np.arange(prefix + 1, prefix + chunk + 1, dtype=np.uint32)
        ends[10:40] = prefix + 40  # a block of rows that reads to the end of the block
        kw["visible_ends"] = ends
    if extra == "f32scales":
        kw["rule"] = O.RULE_CUDA_GQA
    from zllm_amd import capi
    import ctypes as C

    probe = capi.GqaPrefillArgs()
    probe.rows, probe.position, probe.window, probe.num_heads, probe.num_kv_heads, probe.head_dim = chunk, prefix, window, hq, hkv, d
    probe.block_tokens, probe.score_scale, probe.kv_format = 16, 0.1, capi.KV_Q8G64
    probe.scale_dtype = capi.SCALE_F32 if extra == "f32scales" else capi.SCALE_F16
    probe.q_dtype = capi.DTYPE_BF16
    assert capi.load().zllm_attn_gqa_prefill_workspace_bytes(C.byref(probe)) > 0, "this shape is meant to be split"
    tol = 2.0 ** -8 if extra == "bf16out" else 0.0
    for workspace in (True, False):
        out, want = run_case(77 + d + chunk, prefix, chunk, hq, hkv, workspace=workspace, **kw)
        got = out.float().cpu().numpy()
        if tol:
            assert np.abs(got - want).max() <= 2e-3 + tol * max(1.0, float(np.abs(want).max()))
        else:
            assert_attention_close(got, want, f"d={d} prefix={prefix} chunk={chunk} {hq}/{hkv} {extra} workspace={workspace}")


@pytest.mark.parametrize("d,prefix,chunk,hq,hkv,window,extra", [
    (128, 20000, 1, 32, 8, 0, ""), (128, 5000, 4, 16, 2, 0, "gate"), (128, 3000, 2, 8, 2, 700, "bf16out"),
    (128, 900, 8, 8, 2, 0, "ends"), (256, 6000, 3, 8, 2, 0, ""), (64, 2000, 5, 8, 2, 0, "")])
def test_prefill_few_rows_run_as_decode_items(d, prefix, chunk, hq, hkv, window, extra):
    """A chunk of a few rows is a decode step in all but name (the reference decodes through this entry with one row,
    src/backend/rocm/attention.rs:2202-2231): with the workspace the call asks for, its rows run as items of the decode
    kernels; without one, through the chunk kernel.  Both against the oracle, with a gate, a window, explicit visible ends
    and bf16 output."""
    kw = dict(window=window, outliers=True, d=d)
    if extra == "gate":
        kw["gate_cols"] = hq * d
    if extra == "bf16out":
        kw["out_dtype"] = torch.bfloat16
    if extra == "ends":
        kw["visible_ends"] = np.array([prefix + 4] * 4 + [0] + [prefix + chunk] * (chunk - 5), dtype=np.uint32)
    tol = 2.0 ** -8 if extra == "bf16out" else 0.0
    for workspace in (True, False):
        out, want = run_case(31 + d + chunk, prefix, chunk, hq, hkv, workspace=workspace, **kw)
        got = out.float().cpu().numpy()
        assert np.abs(got - want).max() <= 2e-3 + tol * max(1.0, float(np.abs(want).max())), (workspace, np.abs(got - want).max())


@pytest.mark.parametrize("prefix,chunk,hq,hkv,extra", [(0, 300, 8, 2, ""), (17, 700, 16, 2, "gate"), (0, 1024, 8, 2, "bf16out"),
                                                    (40, 200, 32, 4, "softcap"), (0, 33, 8, 1, "")])
def test_prefill_first_chunks_on_half_size_row_tiles(prefix, chunk, hq, hkv, extra):
    """A chunk much longer than what lies before it -- a prompt's first chunk -- runs row tiles of 128 (row, head) pairs,
    handed out longest range first, with or without KV splits on top: against the oracle, with and without a workspace."""
    kw = dict(outliers=True)
    if extra == "gate":
        kw["gate_cols"] = hq * 128
    if extra == "bf16out":
        kw["out_dtype"] = torch.bfloat16
    if extra == "softcap":
        kw["softcap"] = 30.0
    tol = 2.0 ** -8 if extra == "bf16out" else 0.0
    for workspace in (True, False):
        out, want = run_case(61 + chunk, prefix, chunk, hq, hkv, workspace=workspace, **kw)
        got = out.float().cpu().numpy()
        assert np.abs(got - want).max() <= 2e-3 + tol * max(1.0, float(np.abs(want).max())), (workspace, np.abs(got - want).max())


def test_prefill_f16_kv_splits():
    for workspace in (True, False):
        got, want = run_f16_case(5, 256, 4000, 24, 8, 2, softcap=50.0, q_kind="bf16", workspace=workspace)
        assert_attention_close(got, want, f"f16 split workspace={workspace}")
        got, want = run_f16_case(6, 128, 3000, 100, 8, 2, window=600, q_kind="f16", workspace=workspace)
        assert_attention_close(got, want, f"f16 d=128 split workspace={workspace}")


@pytest.mark.parametrize("gate_cols", [8 * 128, 1])
def test_prefill_output_gate(gate_cols):
    """out * sigmoid(gate), one gate per element or per row (src/attention/hybrid.rs:79, src/backend/cpu/context.rs:419-432)."""
    out, want = run_case(31 + gate_cols, 200, 70, 8, 2, gate_cols=gate_cols)
    assert_attention_close(out.cpu().numpy(), want, f"gate_cols={gate_cols}")


@pytest.mark.parametrize("prefix,chunk,hq,hkv", [(1000, 200, 64, 8), (0, 77, 8, 2), (333, 1, 16, 4), (50, 300, 8, 8), (700, 65, 12, 3),
                                                  (129, 40, 32, 1)])
def test_prefill_chunk_matches_oracle(prefix, chunk, hq, hkv):
    out, want = run_case(prefix + chunk, prefix, chunk, hq, hkv)
    print("prefill", prefix, chunk, hq, hkv, assert_attention_close(out.cpu().numpy(), want, f"prefix={prefix} chunk={chunk} {hq}/{hkv}"))


def test_prefill_config5_shape_at_oracle_size():
    """Benchmark config 5 geometry (64q/8kv, d=128, bf16 activations, 16-token pages, chunk into fresh pages) with a
    3,000-token prefix and a 256-row chunk, which the CPU oracle finishes in seconds."""
    out, want = run_case(5, 3000, 256, 64, 8)
    print("config5-small", assert_attention_close(out.cpu().numpy(), want, "config 5 (small)"))


@pytest.mark.parametrize("scale", [None, 1.0])
def test_prefill_long_prefix_with_outlier_channels(scale):
    """Far into a long prefix no single probability weighs much against the running sum and the kernel drops
    the low-order half of P'; with score_scale 1.0 attention is peaked and it must keep it.  Outlier channels
    make |v| large, which is where a lost low-order term would show against the absolute tolerance."""
    out, want = run_case(90, 8000, 64, 16, 2, outliers=True, scale=scale)
    print("long prefix", scale, assert_attention_close(out.cpu().numpy(), want, f"long prefix, scale={scale}"))


@pytest.mark.parametrize("window", [1, 64, 500])
def test_prefill_sliding_window(window):
    out, want = run_case(60 + window, 900, 150, 16, 4, window=window)
    assert_attention_close(out.cpu().numpy(), want, f"window={window}")


def test_prefill_softcap_pages_and_outputs():
    out, want = run_case(71, 400, 100, 16, 8, softcap=30.0, block_tokens=64, rule=O.RULE_ROCM_MLA, scale=0.3)
    assert_attention_close(out.cpu().numpy(), want, "softcap + bf16 scales + 64-token pages")
    out, want = run_case(72, 200, 50, 8, 2, block_tokens=1, q_bf16=False)
    assert_attention_close(out.cpu().numpy(), want, "1-token pages, f32 queries")
    out, want = run_case(73, 200, 50, 8, 2, out_dtype=torch.bfloat16)
    got = out.float().cpu().numpy()
    assert np.abs(got - want).max() <= np.abs(want).max() * 2.0 ** -8 + 2e-3


def _close_at_scale(out, want, what):
    """The 2e-3 / 1e-2 bounds, with the absolute one taken relative to the largest expected magnitude."""
    got = out.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all(), what
    top = float(np.abs(want).max())
    assert top > 0
    return assert_attention_close(got / top, np.asarray(want, dtype=np.float64) / top, what)


@pytest.mark.parametrize("rule,exponent", [(O.RULE_ROCM_MLA, 40), (O.RULE_ROCM_MLA, -40), (O.RULE_METAL_GQA, 11), (O.RULE_METAL_GQA, -12)])
def test_prefill_value_magnitudes(rule, exponent):
    """V scales far from 1 (the kernel carries P' = p * v_scale as f16 and must keep it in range), uniformly and
    with the large values first or last in the sequence (the range the kernel tracks grows while it runs)."""
    total = 600 + 90
    flat = float(2.0 ** exponent)
    print("uniform", _close_at_scale(*run_case(41, 600, 90, 8, 2, rule=rule, v_gain=flat), f"v * 2^{exponent}"))
    first = np.ones(total, dtype=np.float32)
    first[:40] = 2.0 ** abs(exponent)
    print("large first", _close_at_scale(*run_case(42, 600, 90, 8, 2, rule=rule, v_gain=first), "large values first"))
    last = np.ones(total, dtype=np.float32)
    last[500:] = 2.0 ** abs(exponent)
    print("large last", _close_at_scale(*run_case(43, 600, 90, 8, 2, rule=rule, v_gain=last), "large values last"))
    # a single large row in the middle of the prefix, small ones around it
    spike = np.full(total, 2.0 ** -abs(exponent) if rule == O.RULE_ROCM_MLA else 2.0 ** -6, dtype=np.float32)
    spike[333] = 1.0
    print("spike", _close_at_scale(*run_case(44, 600, 90, 8, 2, rule=rule, v_gain=spike), "one large row"))


@pytest.mark.parametrize("q_exp,k_exp", [(12, -12), (-14, 14), (20, 0), (0, -20), (-9, -9)])
def test_prefill_query_and_key_magnitudes(q_exp, k_exp):
    """Queries and keys far from unit magnitude with the score scale compensating: the kernel multiplies its query
    tile by a power of two before rounding it to f16 and folds the inverse into the exponent's argument."""
    scale = float(2.0 ** -(q_exp + k_exp)) / np.sqrt(128)
    out, want = run_case(50 + q_exp, 500, 70, 8, 2, rule=O.RULE_ROCM_MLA, q_gain=2.0 ** q_exp, k_gain=2.0 ** k_exp, scale=scale, q_bf16=False)
    print("q/k magnitudes", q_exp, k_exp, assert_attention_close(out.cpu().numpy(), want, f"q 2^{q_exp}, k 2^{k_exp}"))
    # one row of the chunk much larger than its neighbours inside the same wave's tile (bf16 queries: its scores have a
    # standard deviation near 180, so any rounding of the operands would move the output)
    rows = np.ones(70, dtype=np.float32)
    rows[7] = 2.0 ** 10
    out, want = run_case(60 + q_exp, 300, 70, 8, 2, q_gain=rows, scale=1.0 / 64)
    print("one large query row", assert_attention_close(out.cpu().numpy(), want, "one large query row"))


def test_prefill_rejects_unsupported_shapes():
    from zllm_amd import capi, ops

    z = torch.zeros((16, 96), dtype=torch.int8, device="cuda")
    s = torch.zeros((16, 2), dtype=torch.int16, device="cuda")
    q = torch.zeros((1, 96), dtype=torch.float32, device="cuda")
    with pytest.raises(capi.ZllmAttnError, match="head_dim 64 / 128 / 192 / 256"):
        ops.gqa_prefill_chunk(q, z, s, z, s, None, 0, 1, 1, 96, 16, 1.0)
    with pytest.raises(capi.ZllmAttnError, match="128 / 256 over an f16 cache"):
        ops.gqa_prefill_chunk(q, z, None, z, None, None, 0, 1, 1, 64, 16, 1.0, kv_format=capi.KV_F16)
    table = torch.zeros(2, dtype=torch.int32, device="cuda")  # two pages of 16 tokens cannot hold 40 + 8 tokens
    q8 = torch.zeros((8, 128), dtype=torch.float32, device="cuda")
    with pytest.raises(capi.ZllmAttnError, match="cannot cover"):
        ops.gqa_prefill_chunk(q8, z, s, z, s, table, 40, 1, 1, 128, 16, 1.0)


def test_prefill_config5_full_size():
    """Benchmark config 5 at its own size: a 2,048-row chunk on a 50,000-token prefix, 64q/8kv, d = 128, bf16 activations,
    16-token pages, the chunk quantized into fresh pages by the library.  The oracle runs on the first, a middle and the
    last eight chunk rows of the full call's output."""
    segments = [(0, 8), (1020, 8), (2040, 8)]
    out, want = run_case(5, 50000, 2048, 64, 8, oracle_segments=segments)
    got = np.concatenate([out[r0:r0 + n].cpu().numpy() for r0, n in segments])
    print("config5 full", assert_attention_close(got, want, "config 5 full size"))


# ---- explicit visible ends (multimodal blocks) --------------------------------------------------------------------

def _block_ends(prefix, chunk, block):
    """Rows of a visual block read to the end of their block: visible end of row r = end of r's block (absolute)."""
    return [min(prefix + (r // block + 1) * block, prefix + chunk) for r in range(chunk)]


@pytest.mark.parametrize("prefix,chunk,hq,hkv,block,window", [(0, 3, 2, 1, 3, 0), (200, 96, 16, 4, 24, 0), (1000, 300, 64, 8, 77, 0),
                                                              (500, 130, 8, 2, 40, 64)])
def test_prefill_visible_ends(prefix, chunk, hq, hkv, block, window):
    """key_range_with_visible_end (src/attention/gqa.rs:65-68): a row sees up to max(its own position + 1, its visible
    end), the left edge still follows its window.  The first case is the shape of the reference's visual-block vector
    (src/kernel/cpu/gqa.rs:33-69: three rows that all see the whole block)."""
    ends = _block_ends(prefix, chunk, block)
    out, want = run_case(prefix + chunk + block, prefix, chunk, hq, hkv, window=window, visible_ends=ends)
    assert_attention_close(out.cpu().numpy(), want, f"visible ends block={block}")
    # not the causal result: the ends must have been used
    _, causal = run_case(prefix + chunk + block, prefix, chunk, hq, hkv, window=window)
    assert np.abs(causal - want).max() > 1e-3


def test_prefill_visible_ends_reference_vector():
    """The reference's own known answer (src/kernel/cpu/gqa.rs:33-69): zero queries, three rows that each see the
    whole three-token block -> every row is the mean of the three values."""
    from zllm_amd import capi, ops

    d, bt = 128, 16
    v = np.zeros((3, d), dtype=np.float32)
    v[:, 0] = [3.0, 6.0, 9.0]  # mean 6 in every row: the [6, 6, 6] of the reference's test
    k = np.zeros((3, d), dtype=np.float32)
    planes = {n: np.zeros((bt, d if "codes" in n else d // 64), dtype=np.int8 if "codes" in n else np.uint16)
              for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
    table = np.array([0], dtype=np.uint32)
    O.q8g64_append_paged(O.RULE_METAL_GQA, k, planes["k_codes"], planes["k_scales"], table, 0, bt)
    O.q8g64_append_paged(O.RULE_METAL_GQA, v, planes["v_codes"], planes["v_scales"], table, 0, bt)
    q = torch.zeros((3, d), dtype=torch.float32, device="cuda")
    out = ops.gqa_prefill_chunk(q, upload(planes["k_codes"]), upload(planes["k_scales"]), upload(planes["v_codes"]), upload(planes["v_scales"]),
                                upload(table), 0, 1, 1, d, bt, 1.0, visible_ends=upload(np.array([3, 3, 3], dtype=np.uint32)))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    np.testing.assert_allclose(got[:, 0], [6.0, 6.0, 6.0], rtol=2e-3)
    assert (got[:, 1:] == 0).all()


# ---- other geometries: every chunk row as one item of the split-KV decode kernels ------------------------------------

@pytest.mark.parametrize("d,prefix,chunk,hq,hkv,window,block_tokens", [(64, 300, 70, 8, 2, 0, 16), (256, 500, 40, 16, 8, 0, 16),
                                                                       (256, 700, 33, 4, 1, 128, 64), (64, 0, 50, 4, 4, 0, 4)])
def test_prefill_head_dim_64_and_256(d, prefix, chunk, hq, hkv, window, block_tokens):
    out, want = run_case(d + prefix, prefix, chunk, hq, hkv, window=window, d=d, block_tokens=block_tokens)
    print("prefill d", d, assert_attention_close(out.cpu().numpy(), want, f"head_dim={d}"))


def test_prefill_head_dim_256_visible_ends_gate_and_bf16_out():
    ends = _block_ends(100, 48, 16)
    out, want = run_case(256, 100, 48, 8, 2, d=256, visible_ends=ends, out_dtype=torch.bfloat16)
    got = out.float().cpu().numpy()
    assert np.abs(got - want).max() <= 2e-3 + np.abs(want).max() * 2.0 ** -8
    out, want = run_case(257, 100, 48, 8, 2, d=256, gate_cols=1)
    assert_attention_close(out.cpu().numpy(), want, "head_dim 256 gated")


def run_f16_case(seed, d, prefix, chunk, hq, hkv, window=0, softcap=0.0, block_tokens=16, q_kind="f32", gain=1.0, visible_ends=None,
                 gate_cols=0, out_dtype=None, scale=None, workspace=True):
    """A chunk over an f16 cache: rows written by the oracle's f16 append into a pool whose other rows hold f16 NaN, queries
    as f32 / bf16 / f16; returns (device output as f32 numpy, oracle output)."""
    from zllm_amd import capi, ops

    out_dtype = out_dtype or torch.float32
    rng = np.random.default_rng(seed)
    total = prefix + chunk
    cols = hkv * d
    tables, pool_blocks = draw_tables(rng, [total], block_tokens)
    k = rng.standard_normal((total, cols)).astype(np.float32) * gain
    v = rng.standard_normal((total, cols)).astype(np.float32) * gain
    planes = {n: np.full((pool_blocks * block_tokens, cols), 0x7e00, dtype=np.uint16) for n in ("k", "v")}
    O.half_append_paged(1, k, planes["k"], tables[0], 0, block_tokens)
    O.half_append_paged(1, v, planes["v"], tables[0], 0, block_tokens)
    q = rng.standard_normal((chunk, hq * d)).astype(np.float32)
    if q_kind == "bf16":
        q = O.bf16_to_f32(O.f32_to_bf16(q))
        q_dev = to_torch_bf16(O.f32_to_bf16(q), "cuda")
    elif q_kind == "f16":
        q = q.astype(np.float16).astype(np.float32)
        q_dev = upload(q).to(torch.float16)
    else:
        q_dev = upload(q)
    scale = scale or 1.0 / np.sqrt(d)
    gate = (rng.standard_normal((chunk, gate_cols)) * 3).astype(np.float32) if gate_cols else None
    out = ops.gqa_prefill_chunk(q_dev, upload(planes["k"]), None, upload(planes["v"]), None, upload(tables[0]), prefix, hq, hkv, d, block_tokens,
                                scale, window=window, softcap=softcap, kv_format=capi.KV_F16, out_dtype=out_dtype,
                                gate=None if gate is None else upload(gate), visible_ends=None if visible_ends is None else upload(visible_ends),
                                workspace=workspace)
    torch.cuda.synchronize()
    kd = O.gather_dequant_rows(O.FMT_F16, planes["k"], None, 0, tables[0], block_tokens, 0, total, cols)
    vd = O.gather_dequant_rows(O.FMT_F16, planes["v"], None, 0, tables[0], block_tokens, 0, total, cols)
    rc, want = O.gqa_prefill_at_visible(q, kd, vd, 0, total, prefix, hq, hkv, d, window=window, score_scale=scale, softcap=softcap,
                                        visible_ends=visible_ends)
    assert rc == 0
    if gate is not None:
        rc, want = O.sigmoid_gate(want.reshape(chunk, -1), gate)
        assert rc == 0
    return out.float().cpu().numpy(), want


@pytest.mark.parametrize("d,prefix,chunk,window,softcap", [(256, 900, 64, 0, 50.0), (256, 1500, 40, 1024, 50.0), (128, 300, 100, 0, 0.0)])
def test_prefill_f16_kv(d, prefix, chunk, window, softcap):
    """Chunked prefill over an f16 cache (the config-3 model family prefills too): head_dim 128 and 256 run a matrix-core
    kernel of their own; the soft cap is the family's 50."""
    for q_kind in ("bf16", "f32"):  # bf16 activations run the tile kernel, f32 queries the decode kernels' route
        out, want = run_f16_case(d + prefix, d, prefix, chunk, 16, 8, window=window, softcap=softcap, q_kind=q_kind)
        print("prefill f16", d, q_kind, assert_attention_close(out, want, f"f16 KV prefill d={d} q={q_kind}"))


@pytest.mark.parametrize("d,prefix,chunk,hq,hkv,window,softcap,block_tokens,q_kind",
                         [(128, 0, 1, 4, 4, 0, 0.0, 16, "f32"), (256, 0, 300, 16, 8, 0, 50.0, 16, "bf16"), (128, 2000, 130, 48, 3, 0, 0.0, 64, "bf16"),
                          (256, 1100, 70, 3, 1, 1, 0.0, 1, "f16"), (128, 777, 33, 64, 4, 100, 30.0, 48, "f32"), (256, 640, 129, 128, 1, 0, 0.0, 4, "bf16"),
                          (128, 31, 2, 2, 2, 40, 0.0, 16, "f16"), (256, 2047, 65, 32, 8, 1024, 50.0, 16, "bf16")])
def test_prefill_f16_kv_shapes(d, prefix, chunk, hq, hkv, window, softcap, block_tokens, q_kind):
    """The f16 chunk kernel over group sizes 1 to 128 (one workgroup holds 256 (row, head) pairs at head_dim 128 and 128 at
    256), pages of 1 to 64 tokens, windows down to one token, chunks that start the sequence, every query type."""
    out, want = run_f16_case(1000 + prefix + chunk, d, prefix, chunk, hq, hkv, window=window, softcap=softcap, block_tokens=block_tokens, q_kind=q_kind)
    print("prefill f16 shapes", assert_attention_close(out, want, f"f16 KV prefill d={d} {hq}/{hkv} prefix={prefix} chunk={chunk}"))


@pytest.mark.parametrize("d,out_dtype", [(128, torch.bfloat16), (256, torch.float16), (256, torch.float32)])
def test_prefill_f16_kv_visible_ends_gate_and_output_types(d, out_dtype):
    prefix, chunk, hq, hkv, block = 500, 90, 16, 4, 24
    ends = np.array([min(prefix + chunk, prefix + ((r // block) + 1) * block) if r % 5 else 0 for r in range(chunk)], dtype=np.uint32)
    out, want = run_f16_case(2000 + d, d, prefix, chunk, hq, hkv, visible_ends=ends, gate_cols=hq * d, out_dtype=out_dtype, gain=2.0)
    step = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[out_dtype]
    top = max(1.0, float(np.abs(want).max()))
    assert np.abs(out.astype(np.float64) - want).max() / top <= 2e-3 + step


def test_prefill_f16_kv_magnitudes():
    """Keys and values at 2^6 and 2^-6 of unit scale with the score scale compensating: the query tile's power of two and the
    2^8 carried by the probabilities keep f16 in range either way."""
    for gain in (64.0, 1.0 / 64.0):
        out, want = run_f16_case(3000, 256, 700, 50, 16, 8, gain=gain, scale=1.0 / (np.sqrt(256.0) * gain))
        top = max(1e-30, float(np.abs(want).max()))
        assert np.abs(out.astype(np.float64) - want).max() / top <= 2e-3, gain


def test_prefill_f16_kv_soft_cap_limit():
    """An ever larger cap recovers the uncapped result (the caps models use take a cheaper tanh whose error grows with the
    cap; large caps must not)."""
    plain, want = run_f16_case(5000, 256, 400, 30, 16, 8)
    capped, _ = run_f16_case(5000, 256, 400, 30, 16, 8, softcap=1e9)
    assert_attention_close(capped, want, "f16 KV prefill, cap -> inf")
    tight, want_tight = run_f16_case(5000, 256, 400, 30, 16, 8, softcap=2.0, scale=1.0)
    assert_attention_close(tight, want_tight, "f16 KV prefill, cap 2 on large logits")


def test_prefill_f16_kv_wide_groups_take_the_decode_route():
    """More query heads per KV head than a workgroup of the f16 chunk kernel has columns (128 at head_dim 256): the rows run
    through the decode kernels instead, same results."""
    out, want = run_f16_case(4000, 256, 300, 5, 160, 1)
    print("prefill f16 wide group", assert_attention_close(out, want, "f16 KV prefill, 160 heads per KV head"))


@pytest.mark.parametrize("d,q_bf16", [(256, False), (256, True), (64, False), (64, True)])
def test_prefill_q8_tiles_and_the_decode_route_agree(d, q_bf16):
    """head_dim 64 and 256 over Q8g64 run the matrix-core tile kernel, which carries queries as f16 (exact for bf16
    activations); f32 queries take the decode kernels' route instead, whose query is wider.  Outlier channels
    and large logits are what separate the two."""
    out, want = run_case(800 + d, 1200, 96, 16, 4, d=d, q_bf16=q_bf16, outliers=True, scale=0.25 if d == 64 else 0.125)
    print("prefill q8 tiles", d, q_bf16, assert_attention_close(out.cpu().numpy(), want, f"Q8 prefill d={d} bf16={q_bf16}"))


@pytest.mark.parametrize("d,q_bf16", [(128, True), (64, True), (256, True), (128, False)])
def test_prefill_f32_scale_cache(d, q_bf16):
    """A chunk over a cache with f32 scales (CUDA convention): appended by the library, attended by the tile kernel (bf16
    queries) or through the decode kernels (f32 queries)."""
    out, want = run_case(321 + d, 400, 60, 16, 4, rule=O.RULE_CUDA_GQA, d=d, q_bf16=q_bf16, outliers=True)
    print("prefill f32 scales", d, q_bf16, assert_attention_close(out.cpu().numpy(), want, f"f32-scale prefill d={d}"))


@pytest.mark.parametrize("prefix,chunk,hq,hkv,window,q_bf16,rule", [(700, 40, 16, 4, 0, True, O.RULE_METAL_GQA), (0, 130, 8, 2, 0, False, O.RULE_ROCM_MLA),
                                                                   (2500, 1, 12, 3, 0, True, O.RULE_METAL_GQA), (900, 64, 8, 1, 300, True, O.RULE_CUDA_GQA)])
def test_head_dim_192_chunks_run_as_decode_items(prefix, chunk, hq, hkv, window, q_bf16, rule):
    """A chunk at head_dim 192 (three Q8g64 groups a head) has no matrix-core chunk kernel: its rows run as items of the
    split-KV decode kernels, whatever their number; f32 and bf16 output, visible ends, and no workspace -> refused."""
    from zllm_amd import capi

    out, want = run_case(192 + chunk, prefix, chunk, hq, hkv, window=window, d=192, q_bf16=q_bf16, rule=rule, outliers=True)
    print("d=192 chunk", prefix, chunk, assert_attention_close(out.cpu().numpy(), want, f"d=192 prefix={prefix} chunk={chunk} window={window}"))
    if window == 0 and chunk > 1:
        total = prefix + chunk
        ends = np.minimum((np.arange(chunk) // 16 + 1) * 16 + prefix, total).astype(np.uint32)
        out, want = run_case(192 + chunk, prefix, chunk, hq, hkv, d=192, q_bf16=q_bf16, rule=rule, visible_ends=ends, out_dtype=torch.bfloat16)
        got = out.float().cpu().numpy()
        assert np.abs(got - want).max() <= 2e-3 + np.abs(want).max() * 2.0 ** -8
    with pytest.raises(capi.ZllmAttnError, match="needs a 16-byte aligned workspace"):
        run_case(192 + chunk, prefix, chunk, hq, hkv, window=window, d=192, q_bf16=q_bf16, rule=rule, workspace=False)

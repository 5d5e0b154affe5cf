"""Seeded random parity sweeps: every case draws its shape, page size, window, soft cap, scale rule, query type and
magnitudes from one generator seeded by (sweep, case number), runs the HIP path through the C-ABI and compares with the
CPU oracle at the tolerance of the fixed cases.  The fixed cases in the other GPU test modules cover the shapes the
reference tests name; these cover combinations nobody thought to write down (odd group sizes, a window of one token over
a 48-token page, a 2^-8 value gain with a per-head gate, ...)."""
import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, make_gqa_q8_case, oracle_gqa_decode
from tests.test_gpu_gqa_decode import make_f16_case, run_decode, run_f16
from tests.test_gpu_gqa_prefill import run_case, run_f16_case
from tests.test_gpu_mla_decode import (draw_selection, make_mla_case, make_mla_chunk_case, oracle_mla, oracle_mla_chunk, run_mla,
                                       run_mla_chunk)

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

LENGTHS = [0, 1, 15, 16, 17, 31, 32, 33, 64, 100, 255, 256, 257, 700, 1024, 2049, 4100]
MLA_LENGTHS = [1, 2, 31, 32, 33, 63, 64, 65, 95, 96, 97, 255, 256, 257, 511, 513, 700, 1023, 1025, 2047, 2049, 3000]
PAGE_SIZES = [1, 4, 16, 16, 64, 48]


def pick(rng, values):
    return values[int(rng.integers(0, len(values)))]


def block_ends(rng, prefix, chunk, max_block, keep):
    """Visible ends in blocks of a random size; about one row in `keep` sees nothing (end 0)."""
    block = int(rng.integers(1, max_block))
    return np.array([min(prefix + chunk, prefix + ((r // block) + 1) * block) if rng.integers(0, keep) else 0 for r in range(chunk)],
                    dtype=np.uint32)


def close_at_scale(got, want, what, extra=0.0):
    """The tolerance applies to outputs of order one: outputs grow with the value gain, so divide by the largest."""
    want = np.asarray(want, dtype=np.float64)
    top = max(1.0, float(np.abs(want).max()))
    return assert_attention_close(np.asarray(got, dtype=np.float64) / top, want / top, what, atol=2e-3 + extra)


@pytest.mark.parametrize("it", [*range(40), 265, 273, 497])  # the last three: 128 query heads at head_dim 256 over outlier channels
def test_random_q8_decode(it):
    rng = np.random.default_rng([101, it])
    hkv = pick(rng, [1, 2, 4, 8])
    group = pick(rng, [1, 2, 3, 4, 8, 16])
    d = pick(rng, [64, 128, 128, 256])
    lens = [pick(rng, LENGTHS) for _ in range(int(rng.integers(1, 6)))]
    if max(lens) == 0:
        lens[0] = 5
    window = pick(rng, [0, 0, 1, 33, 128, 1024])
    softcap = pick(rng, [0.0, 0.0, 30.0])
    what = f"decode {it}: {hkv * group}/{hkv} d={d} lens={lens} window={window} softcap={softcap}"
    print(what, flush=True)
    case = make_gqa_q8_case(2000 + it, lens, hkv * group, hkv, d, outliers=bool(it % 2), q_bf16=bool(it % 3 == 0))
    got = run_decode(case, 0.09, window=window, softcap=softcap)
    assert_attention_close(got, oracle_gqa_decode(case, 0.09, window=window, softcap=softcap), what)


@pytest.mark.parametrize("it", [*range(32), 52, 190, 266, 814])  # the last four: score scale 0.2 over outlier channels
def test_random_q8_decode_pages_rules_and_hints(it):
    """The decode sweep over what the one above keeps fixed: the three scale rules, pages of 1 to 64 tokens in random,
    identity or reversed pool order, pools that were never cleared, longer sequences, a gate, the score scale, and the
    token-count hint (records over the live splits) on every other case."""
    rng = np.random.default_rng([606, it])
    hkv = pick(rng, [1, 2, 3, 4, 8])
    group = pick(rng, [1, 2, 4, 5, 8, 16])
    d = pick(rng, [64, 128, 128, 128, 256])
    rule = pick(rng, [O.RULE_METAL_GQA, O.RULE_ROCM_MLA, O.RULE_CUDA_GQA])
    page = pick(rng, PAGE_SIZES + [32, 128])
    lens = [pick(rng, LENGTHS + [6000, 9000, 20000]) for _ in range(int(rng.integers(1, 9)))]
    if max(lens) == 0:
        lens[0] = 5
    window = pick(rng, [0, 0, 0, 1, 33, 500, 4096])
    softcap = pick(rng, [0.0, 0.0, 50.0])
    scale = pick(rng, [0.09, 1.0 / np.sqrt(d), 0.2])
    layout = pick(rng, ["random", "random", "identity", "reversed"])
    gated = bool(rng.integers(0, 4) == 0)
    hint = it % 2 == 0
    what = (f"decode {it}: {hkv * group}/{hkv} d={d} rule={rule} page={page} layout={layout} lens={lens} window={window} "
            f"softcap={softcap} scale={scale:.3f} gated={gated} hint={hint}")
    print(what, flush=True)
    case = make_gqa_q8_case(6000 + it, lens, hkv * group, hkv, d, block_tokens=page, rule=rule, outliers=bool(it % 3), layout=layout,
                            q_bf16=bool(it % 4 == 1), poison=bool(it % 5 == 0))
    gate = (rng.standard_normal((len(lens), hkv * group * d)) * 3).astype(np.float32) if gated else None
    visible = [min(l, window) if window else l for l in lens]
    from tests.cases import upload
    got = run_decode(case, scale, window=window, softcap=softcap, gate=None if gate is None else upload(gate),
                     total_kv_tokens=sum(visible) if hint else 0)
    want = oracle_gqa_decode(case, scale, window=window, softcap=softcap)
    if gated:
        rc, want = O.sigmoid_gate(want, gate)
        assert rc == 0
    assert_attention_close(got, want, what)


@pytest.mark.parametrize("it", range(24))
def test_random_f16_decode(it):
    """Decode over f16 rows (the cache of the f16 model family, src/kv_cache/mod.rs:179-331) at head_dim 128 and 256: pages
    of 1 to 64 tokens, windows, soft caps, score scales up to 0.2 over outlier channels, never-cleared pools."""
    rng = np.random.default_rng([707, it])
    hkv = pick(rng, [1, 2, 4, 8])
    group = pick(rng, [1, 2, 4, 8, 16])
    d = pick(rng, [128, 256])
    page = pick(rng, PAGE_SIZES)
    lens = [max(1, pick(rng, LENGTHS + [6000])) for _ in range(int(rng.integers(1, 7)))]
    window = pick(rng, [0, 0, 1, 33, 1024])
    softcap = pick(rng, [0.0, 0.0, 50.0])
    scale = pick(rng, [1.0 / np.sqrt(d), 0.09, 0.2])
    what = f"f16 decode {it}: {hkv * group}/{hkv} d={d} page={page} lens={lens} window={window} softcap={softcap} scale={scale:.3f}"
    print(what, flush=True)
    case = make_f16_case(7000 + it, lens, hkv * group, hkv, d, block_tokens=page, poison=bool(it % 3 == 0), outliers=bool(it % 2))
    got = run_f16(case, scale, window=window, softcap=softcap)
    assert_attention_close(got, oracle_gqa_decode(case, scale, window=window, softcap=softcap, fmt=O.FMT_F16), what)


@pytest.mark.parametrize("it", [*range(48), 1298])  # 1298: f32 queries, score scale 0.3, outlier channels
def test_random_q8_prefill_chunk(it):
    """All three head sizes, the three scale-storage rules, visible ends, gates, K and V gains over 2^-8..2^8."""
    rng = np.random.default_rng([202, it])
    d = pick(rng, [64, 128, 128, 256])
    hkv = pick(rng, [1, 2, 4, 8])
    hq = hkv * pick(rng, [1, 2, 3, 4, 8, 16])
    prefix = int(rng.integers(0, 2500))
    chunk = int(rng.integers(1, 260))
    window = pick(rng, [0, 0, 0, 1, 33, 200, 1000])
    softcap = pick(rng, [0.0, 0.0, 30.0, 50.0])
    bt = pick(rng, PAGE_SIZES)
    rule = pick(rng, [O.RULE_METAL_GQA, O.RULE_ROCM_MLA, O.RULE_CUDA_GQA])
    q_bf16 = True if d == 256 else bool(rng.integers(0, 2))
    scale = pick(rng, [1 / np.sqrt(d), 0.3])
    v_gain = float(2.0 ** rng.integers(-8, 9))
    k_gain = float(2.0 ** rng.integers(-3, 4))
    ends = block_ends(rng, prefix, chunk, 60, 3) if rng.integers(0, 3) == 0 else None
    gate_cols = pick(rng, [0, 0, 1, hq * d])
    # f32 queries run row by row through the decode kernels, which need their split records, except at head_dim 128 with
    # 16-bit scales; every other case may run without a workspace (the unsplit chunk kernel)
    workspace = bool(rng.integers(0, 4)) or not (q_bf16 or (d == 128 and rule != O.RULE_CUDA_GQA))
    what = (f"prefill {it}: d={d} {hq}/{hkv} prefix={prefix} chunk={chunk} window={window} softcap={softcap} page={bt} rule={rule} "
            f"q_bf16={q_bf16} scale={scale:.3f} v_gain={v_gain} k_gain={k_gain} ends={ends is not None} gate_cols={gate_cols} "
            f"workspace={workspace}")
    print(what, flush=True)
    out, want = run_case(7000 + it, prefix, chunk, hq, hkv, window=window, softcap=softcap, block_tokens=bt, rule=rule, q_bf16=q_bf16,
                         scale=scale / k_gain, outliers=bool(rng.integers(0, 2)), v_gain=v_gain, k_gain=k_gain, d=d, visible_ends=ends,
                         gate_cols=gate_cols, workspace=workspace)
    got = out.cpu().numpy().astype(np.float64)
    want = want.astype(np.float64)
    top = max(1.0, float(np.abs(want).max())) if v_gain >= 1 else max(1e-30, float(np.abs(want).max()))
    assert_attention_close(got / top, want / top, what)


@pytest.mark.parametrize("it", range(30))
def test_random_f16_prefill_chunk(it):
    rng = np.random.default_rng([303, it])
    d = pick(rng, [128, 256])
    hkv = pick(rng, [1, 2, 4, 8])
    hq = hkv * pick(rng, [1, 2, 3, 4, 8, 16])
    prefix = int(rng.integers(0, 2200))
    chunk = int(rng.integers(1, 300))
    window = pick(rng, [0, 0, 1, 40, 700, 1024])
    softcap = pick(rng, [0.0, 0.0, 50.0, 20.0])
    bt = pick(rng, PAGE_SIZES)
    q_kind = pick(rng, ["f32", "bf16", "f16"])
    gain = float(2.0 ** rng.integers(-3, 4))
    scale = pick(rng, [1.0 / np.sqrt(d), 0.2])
    ends = block_ends(rng, prefix, chunk, 70, 4) if rng.integers(0, 3) == 0 else None
    gate_cols = pick(rng, [0, 0, 1, hq * d])
    out_dtype = pick(rng, [torch.float32, torch.bfloat16, torch.float16])
    workspace = bool(rng.integers(0, 4)) or q_kind == "f32"  # f32 queries over an f16 cache need the decode kernels' records
    what = (f"f16 prefill {it}: d={d} {hq}/{hkv} prefix={prefix} chunk={chunk} window={window} softcap={softcap} page={bt} q={q_kind} "
            f"gain={gain} ends={ends is not None} gate_cols={gate_cols} out={out_dtype} workspace={workspace}")
    print(what, flush=True)
    got, want = run_f16_case(4000 + it, d, prefix, chunk, hq, hkv, window=window, softcap=softcap, block_tokens=bt, q_kind=q_kind, gain=gain,
                             visible_ends=ends, gate_cols=gate_cols, out_dtype=out_dtype, scale=scale, workspace=workspace)
    # a 16-bit output rounds once more: half an ulp of the largest output
    extra = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[out_dtype]
    close_at_scale(got, want.reshape(got.shape), what, extra)


@pytest.mark.parametrize("it", range(45))
def test_random_mla_decode(it):
    rng = np.random.default_rng([404, it])
    heads = pick(rng, [1, 3, 16, 20, 40, 64, 65, 128])
    bt = pick(rng, [1, 16, 32, 48, 64, 128])
    batch = pick(rng, [1, 2, 3, 4, 4, 17, 33])  # 16 rows and more take the matrix-core absorb and projection
    lens = [pick(rng, MLA_LENGTHS) for _ in range(batch)]
    if heads >= 64 or batch > 4:
        lens = [min(l, 700) for l in lens]
    if heads >= 64 and batch > 4:
        lens = [min(l, 257) for l in lens]
    selection = None
    if it % 3 == 0:
        selection = draw_selection(rng, lens, pick(rng, [1, 7, 32, 100, 300]), bool(it % 2))
    hint = sum(lens) if (selection is None and rng.integers(0, 2)) else 0
    what = f"mla {it}: heads={heads} page={bt} lens={lens} top_k={None if selection is None else selection.shape[1]} hint={hint}"
    print(what, flush=True)
    case = make_mla_case(1000 + it, lens, heads, block_tokens=bt, poison=bool(it % 2))
    want, _ = oracle_mla(case, selection=selection)
    got = run_mla(case, selection=selection, total_ctx_tokens=hint).cpu().numpy()
    assert_attention_close(got.reshape(want.shape), want, what)
    if heads > 32 and bt % 32 == 0 and selection is None:  # a shape the second split-KV kernel takes
        wide = run_mla(case, total_ctx_tokens=hint, wide_tiles=True).cpu().numpy()
        assert_attention_close(wide.reshape(want.shape), want, what + " (wide tiles)")


@pytest.mark.parametrize("it", range(14))
def test_random_mla_chunk(it):
    rng = np.random.default_rng([505, it])
    heads = pick(rng, [8, 16, 20, 64, 128])
    rows = pick(rng, [2, 3, 8, 17, 40])
    lens = [int(rng.integers(rows, 1500)) for _ in range(int(rng.integers(1, 4)))]
    bt = pick(rng, [16, 64, 48, 1])
    q_kind = pick(rng, ["bf16", "bf16", "f32"])
    what = f"mla chunk {it}: heads={heads} lens={lens} rows={rows} page={bt} q={q_kind}"
    print(what, flush=True)
    case = make_mla_chunk_case(4000 + it, lens, rows, heads, block_tokens=bt)
    want, _ = oracle_mla_chunk(case)
    got = run_mla_chunk(case, q_kind=q_kind).cpu().numpy()
    assert_attention_close(got.reshape(want.shape), want, what)
    if heads > 32 and bt % 32 == 0:
        wide = run_mla_chunk(case, q_kind=q_kind, wide_tiles=True).cpu().numpy()
        assert_attention_close(wide.reshape(want.shape), want, what + " (wide tiles)")


@pytest.mark.parametrize("it", [*range(16), 779])  # 779: 24 heads on 3, soft cap, a first chunk of 64 rows
def test_random_q8_head_dim_192(it):
    """Decode steps and prefill chunks at head_dim 192 (three Q8g64 groups a head): every scale rule, pages of 1 to 64 tokens,
    windows, soft caps, the token-count hint on every other case."""
    rng = np.random.default_rng([505, it])
    hkv = pick(rng, [1, 2, 3, 4, 8])
    group = pick(rng, [1, 2, 3, 4, 8, 16])
    rule = pick(rng, [O.RULE_METAL_GQA, O.RULE_ROCM_MLA, O.RULE_CUDA_GQA])
    page = pick(rng, PAGE_SIZES)
    window = pick(rng, [0, 0, 1, 33, 1024])
    softcap = pick(rng, [0.0, 0.0, 30.0])
    if it % 2 == 0:
        lens = [pick(rng, LENGTHS) for _ in range(int(rng.integers(1, 6)))]
        if max(lens) == 0:
            lens[0] = 5
        what = f"decode d=192 {it}: {hkv * group}/{hkv} rule={rule} page={page} lens={lens} window={window} softcap={softcap}"
        print(what, flush=True)
        case = make_gqa_q8_case(5000 + it, lens, hkv * group, hkv, 192, block_tokens=page, rule=rule, outliers=bool(it % 4), poison=True)
        visible = [min(l, window) if window else l for l in lens]
        got = run_decode(case, 0.07, window=window, softcap=softcap, total_kv_tokens=sum(visible) if it % 4 == 0 else 0)
        assert_attention_close(got, oracle_gqa_decode(case, 0.07, window=window, softcap=softcap), what)
    else:
        prefix, chunk = pick(rng, [0, 1, 100, 777, 2100]), pick(rng, [1, 2, 17, 64, 100])
        what = f"prefill d=192 {it}: {hkv * group}/{hkv} rule={rule} page={page} prefix={prefix} chunk={chunk} window={window} softcap={softcap}"
        print(what, flush=True)
        out, want = run_case(5000 + it, prefix, chunk, hkv * group, hkv, window=window, softcap=softcap, block_tokens=page, rule=rule,
                             q_bf16=bool(it % 3), d=192, outliers=True)
        assert_attention_close(out.cpu().numpy(), want, what)


@pytest.mark.parametrize("it", range(24))
def test_random_mla_other_widths_and_weight_forms(it):
    """MLA decode steps and chunks at latent widths of one to sixteen Q8g64 groups, rope widths of 2 to 256, and kv_b as bf16,
    f32, W8A16 or W4A16 (at 512 + 64 too, where only absorb and projection change kernels)."""
    from tests.test_gpu_mla_decode import set_weight_form

    rng = np.random.default_rng([606, it])
    usual = it % 4 == 3
    latent = 512 if usual else pick(rng, [64, 128, 192, 256, 320, 448, 576, 1024])
    rope = 64 if usual else pick(rng, [2, 16, 32, 64, 96, 128, 256])
    nope, value = pick(rng, [16, 32, 64, 128, 192]), pick(rng, [16, 64, 128, 160])
    heads = pick(rng, [1, 2, 3, 8, 20, 33])
    page = pick(rng, [1, 16, 32, 48, 64])
    form = pick(rng, ["bf16", "f32", "w8", "w8", "w4"]) if not usual else pick(rng, ["f32", "w8", "w4"])
    rows = pick(rng, [1, 1, 1, 3, 9])
    lens = [max(rows, pick(rng, MLA_LENGTHS[:18])) for _ in range(int(rng.integers(1, 4)))]
    what = f"mla other {it}: latent={latent} rope={rope} nope={nope} value={value} heads={heads} page={page} kv_b={form} rows={rows} lens={lens}"
    print(what, flush=True)
    kw = dict(nope=nope, rope=rope, value=value, latent=latent, block_tokens=page)
    case = make_mla_case(6000 + it, lens, heads, poison=bool(it % 2), **kw) if rows == 1 else make_mla_chunk_case(6000 + it, lens, rows, heads, **kw)
    if form != "bf16":
        group = pick(rng, [g for g in (32, 64, 128, latent) if latent % g == 0])
        set_weight_form(case, {"f32": 32, "w8": 8, "w4": 4}[form], group=group, scale_dtype=pick(rng, [O.SCALE_BF16, O.SCALE_F16, O.SCALE_F32]))
    if rows == 1:
        want, _ = oracle_mla(case)
        got = run_mla(case, total_ctx_tokens=int(sum(lens)) if it % 3 == 0 else 0).cpu().numpy()
        assert_attention_close(got.reshape(want.shape), want, what)
    else:
        want, _ = oracle_mla_chunk(case)
        assert_attention_close(run_mla_chunk(case).cpu().numpy(), want, what)


@pytest.mark.parametrize("it", range(40))
def test_random_q8g64_append(it):
    """The quantizing append, bit for bit: the three scale rules, f32 / bf16 / f16 sources, 64 to 4,096 columns, pages of 1
    to 128 tokens, any start row, rings, and the values a quantizer can get wrong -- codes exactly between two integers,
    all-zero and one-element groups, subnormal and huge magnitudes, negative zero."""
    from zllm_amd import ops
    from tests.cases import draw_tables, upload

    rng = np.random.default_rng([808, it])
    rule = pick(rng, [O.RULE_ROCM_MLA, O.RULE_METAL_GQA, O.RULE_CUDA_GQA])
    cols = pick(rng, [64, 128, 192, 512, 576, 1024, 2048, 4096])
    page = pick(rng, PAGE_SIZES + [128])
    rows = int(rng.integers(1, 300))
    start = int(rng.integers(0, 200))
    src = pick(rng, ["f32", "f32", "bf16", "f16"])
    ring = pick(rng, [0, 0, 0, 64, 100])
    what = f"append {it}: rule={rule} cols={cols} page={page} rows={rows} start={start} src={src} ring={ring}"
    print(what, flush=True)
    x = rng.standard_normal((rows, cols)).astype(np.float32) * np.float32(2.0 ** rng.integers(-20, 20))
    groups = x.reshape(rows, cols // 64, 64)
    for _ in range(min(rows, 12)):  # special groups
        r, g, kind = int(rng.integers(0, rows)), int(rng.integers(0, cols // 64)), int(rng.integers(0, 6))
        if kind == 0:
            groups[r, g] = 0.0
        elif kind == 1:
            groups[r, g] = -0.0
            groups[r, g, 3] = 1e-41  # a subnormal alone
        elif kind == 2:  # codes exactly halfway: the largest element is 127 units, the others k + 0.5 units
            unit = np.float32(2.0 ** rng.integers(-10, 10))
            groups[r, g] = (rng.integers(-126, 126, size=64) + 0.5).astype(np.float32) * unit
            groups[r, g, 0] = 127.0 * unit
        elif kind == 3:
            groups[r, g] = np.clip(groups[r, g].astype(np.float64) * 1e30, -3e38, 3e38).astype(np.float32)
        elif kind == 4:
            groups[r, g] = 0.0
            groups[r, g, 63] = -3.0
        else:
            groups[r, g] = np.float32(65504.0) if src == "f16" else np.float32(3e38)
    if src == "bf16":
        bits = O.f32_to_bf16(x)
        x = O.bf16_to_f32(bits)
        dev = upload(bits).view(torch.bfloat16)
    elif src == "f16":
        x = np.clip(x, -65504.0, 65504.0)
        half = x.astype(np.float16)
        x = half.astype(np.float32)
        dev = upload(half)
    else:
        dev = upload(x)
    stored = min(start + rows, ring) if ring else start + rows
    tables, pool_blocks = draw_tables(rng, [max(stored, 1)], page)
    pool_rows = pool_blocks * page
    sdt = {O.RULE_ROCM_MLA: O.SCALE_BF16, O.RULE_METAL_GQA: O.SCALE_F16, O.RULE_CUDA_GQA: O.SCALE_F32}[rule]
    ref_codes = np.full((pool_rows, cols), 77, dtype=np.int8)
    ref_scales = np.full((pool_rows, cols // 64), 3, dtype=np.float32 if sdt == O.SCALE_F32 else np.uint16)
    codes, scales = upload(ref_codes), upload(ref_scales)
    if ring and rows > ring:  # a ring takes at most its capacity in one call
        x, dev, rows = x[:ring], dev[:ring], ring
    O.q8g64_append_paged(rule, x, ref_codes, ref_scales, tables[0], start, page, ring_capacity=ring)
    ops.q8g64_append(dev, codes, scales, upload(tables[0]), start, page, rule, ring_capacity=ring)
    torch.cuda.synchronize()
    assert np.array_equal(scales.cpu().numpy().view(ref_scales.dtype).view(np.uint8), ref_scales.view(np.uint8)), what + ": scale bits differ"
    assert np.array_equal(codes.cpu().numpy(), ref_codes), what + ": codes differ"


@pytest.mark.parametrize("it", range(24))
def test_random_gqa_prologue(it):
    """Per-head RMSNorm + RoPE of Q and K and the quantizing append of K and V in one launch, against the CPU chain
    rmsnorm_heads -> rope_apply -> q8g64_append_paged: head sizes 64 to 256, rotary widths, both layouts, the Gemma weight
    offset, pages of 1 to 128 tokens, any start row; Q, codes and scale bits compared bit for bit."""
    from zllm_amd import ops
    from tests.cases import draw_tables, upload
    from tests.test_gpu_gqa_prologue import cpu_chain, rope_table

    rng = np.random.default_rng([909, it])
    d = pick(rng, [64, 128, 128, 256])
    hkv = pick(rng, [1, 2, 4, 8])
    hq = hkv * pick(rng, [1, 2, 4, 8])
    rotary = pick(rng, [0, d // 2, d, d])
    split_half = bool(rng.integers(0, 2))
    offset = pick(rng, [0.0, 1.0])
    rows = int(rng.integers(1, 90))
    position = int(rng.integers(0, 300))
    page = pick(rng, PAGE_SIZES + [128])
    eps = pick(rng, [1e-6, 1e-5])
    what = f"prologue {it}: d={d} {hq}/{hkv} rotary={rotary} split_half={split_half} offset={offset} rows={rows} position={position} page={page}"
    print(what, flush=True)
    q = rng.standard_normal((rows, hq * d)).astype(np.float32) * np.float32(2.0 ** rng.integers(-6, 7))
    k = rng.standard_normal((rows, hkv * d)).astype(np.float32) * np.float32(2.0 ** rng.integers(-6, 7))
    v = rng.standard_normal((rows, hkv * d)).astype(np.float32) * np.float32(2.0 ** rng.integers(-6, 7))
    k[:, :64] *= 40.0
    if rows > 2:
        k[1] = 0.0  # an all-zero row: the norm divides by sqrt(eps)
        v[2, 64:128] = 0.0 if hkv * d > 64 else v[2, 64:128]
    qw = (rng.standard_normal(d) * 0.2).astype(np.float32)
    kw = (rng.standard_normal(d) * 0.2).astype(np.float32)
    cos, sin = rope_table(position + rows + 3, max(rotary // 2, 1))
    tables, pool_blocks = draw_tables(rng, [position + rows], page)
    pool_rows = pool_blocks * page
    want_q = cpu_chain(q, hq, d, qw, eps, offset, rotary, position, cos, sin, split_half)
    want_k = cpu_chain(k, hkv, d, kw, eps, offset, rotary, position, cos, sin, split_half)
    ref = {n: np.zeros((pool_rows, hkv * d), dtype=np.int8) for n in ("k", "v")}
    ref_s = {n: np.zeros((pool_rows, hkv * d // 64), dtype=np.uint16) for n in ("k", "v")}
    O.q8g64_append_paged(O.RULE_METAL_GQA, want_k, ref["k"], ref_s["k"], tables[0], position, page)
    O.q8g64_append_paged(O.RULE_METAL_GQA, v, ref["v"], ref_s["v"], tables[0], position, page)
    dev = {n: torch.zeros((pool_rows, hkv * d), dtype=torch.int8, device="cuda") for n in ("k", "v")}
    dev_s = {n: torch.zeros((pool_rows, hkv * d // 64), dtype=torch.int16, device="cuda") for n in ("k", "v")}
    got_q = ops.gqa_prologue(upload(q), upload(k), upload(v), upload(qw), upload(kw), upload(cos) if rotary else None,
                             upload(sin) if rotary else None, dev["k"], dev_s["k"], dev["v"], dev_s["v"], upload(tables[0]),
                             position, hq, hkv, d, rotary, page, eps=eps, weight_offset=offset, split_half=split_half)
    torch.cuda.synchronize()
    assert np.array_equal(got_q.cpu().numpy().view(np.uint32), want_q.view(np.uint32)), what + ": Q bits differ"
    for n in ("k", "v"):
        assert np.array_equal(dev_s[n].cpu().numpy().view(np.uint16), ref_s[n]), what + f": {n} scale bits differ"
        assert np.array_equal(dev[n].cpu().numpy(), ref[n]), what + f": {n} codes differ"


@pytest.mark.parametrize("it", range(24))
def test_random_mla_append(it):
    """The fused MLA append (latent rows quantized with the bf16-scale rule, rope rows rotated and stored as bf16) at latent
    widths of 64 to 1,024 and rope widths of 2 to 256, both rotary layouts, any page size and start row, rope positions
    apart from cache positions: every byte against q8g64_append_paged + rope_apply + half_append_paged."""
    from zllm_amd import ops
    from tests.cases import draw_tables, upload

    rng = np.random.default_rng([1010, it])
    latent_cols = pick(rng, [64, 128, 256, 512, 512, 512, 576, 1024])
    rope_cols = pick(rng, [2, 32, 64, 64, 64, 128, 256])
    rotary_dim = pick(rng, [0, rope_cols, rope_cols, max(2, rope_cols // 2)])
    layout = int(rng.integers(0, 2))
    rows = int(rng.integers(1, 120))
    position = int(rng.integers(0, 300))
    rope_position = position + int(rng.integers(0, 5))
    page = pick(rng, PAGE_SIZES + [128])
    what = f"mla append {it}: latent={latent_cols} rope={rope_cols} rotary={rotary_dim} layout={layout} rows={rows} position={position} page={page}"
    print(what, flush=True)
    tables, pool_blocks = draw_tables(rng, [position + rows], page)
    latent = rng.standard_normal((rows, latent_cols)).astype(np.float32) * np.float32(2.0 ** rng.integers(-8, 9))
    k_rope = rng.standard_normal((rows, rope_cols)).astype(np.float32) * np.float32(2.0 ** rng.integers(-4, 5))
    half = max(rotary_dim // 2, 1)
    angles = rng.uniform(0, 6.28, size=(rope_position + rows + 3, half)).astype(np.float32)
    cos, sin = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
    pool = pool_blocks * page
    ref_codes = np.zeros((pool, latent_cols), dtype=np.int8)
    ref_scales = np.zeros((pool, latent_cols // 64), dtype=np.uint16)
    ref_rope = np.zeros((pool, rope_cols), dtype=np.uint16)
    O.q8g64_append_paged(O.RULE_ROCM_MLA, latent, ref_codes, ref_scales, tables[0], position, page)
    rotated = k_rope
    if rotary_dim:
        rc, rotated = O.rope_apply(k_rope, 1, rotary_dim, rope_position, cos, sin, layout=0 if layout == 1 else 1, placement=1)
        assert rc == 0
    O.half_append_paged(0, rotated, ref_rope, tables[0], position, page)
    codes = torch.zeros((pool, latent_cols), dtype=torch.int8, device="cuda")
    scales = torch.zeros((pool, latent_cols // 64), dtype=torch.int16, device="cuda")
    rope_cache = torch.zeros((pool, rope_cols), dtype=torch.int16, device="cuda")
    ops.mla_append(upload(latent), upload(k_rope), codes, scales, rope_cache, upload(tables[0]), position, page,
                   cos=upload(cos) if rotary_dim else None, sin=upload(sin) if rotary_dim else None,
                   rotary_dim=rotary_dim, rotary_layout=layout, rope_position=rope_position)
    torch.cuda.synchronize()
    assert np.array_equal(codes.cpu().numpy(), ref_codes), what + ": codes differ"
    assert np.array_equal(scales.cpu().numpy().view(np.uint16), ref_scales), what + ": scale bits differ"
    assert np.array_equal(rope_cache.cpu().numpy().view(np.uint16), ref_rope), what + ": rope bits differ"


@pytest.mark.parametrize("it", range(24))
def test_random_block_attention(it):
    """Explicit per-row key ranges (BlockAttentionSpec::visible and its varlen form, src/attention/block.rs:10-119) drawn at
    random: free [start, end) per row, packed isolated segments, one-key rows, more rows than keys; Q8g64 and f16 rows, every
    head size a chunk kernel takes, with and without the workspace."""
    from tests.test_gpu_block_attention import run_block, varlen_ranges

    rng = np.random.default_rng([1111, it])
    kv = pick(rng, ["q8", "q8", "f16"])
    d = pick(rng, [128, 256] if kv == "f16" else [64, 128, 128, 256])
    hkv = pick(rng, [1, 2, 4, 8])
    hq = hkv * pick(rng, [1, 2, 4, 8])
    q_kind = "bf16" if d != 128 or kv == "f16" else pick(rng, ["bf16", "f32"])
    page = pick(rng, [16, 16, 64, 48, 1])
    workspace = bool(rng.integers(0, 3))
    if rng.integers(0, 2):  # isolated segments packed into one call
        segments = int(rng.integers(1, 7))
        q_off = np.concatenate([[0], np.cumsum(rng.integers(1, 120, size=segments))])
        kv_off = np.concatenate([[0], np.cumsum(rng.integers(1, 900, size=segments))])
        visible = varlen_ranges([int(x) for x in q_off], [int(x) for x in kv_off])
        q_rows, kv_rows = int(q_off[-1]), int(kv_off[-1])
    else:
        q_rows, kv_rows = int(rng.integers(1, 200)), int(rng.integers(2, 4000))
        starts = rng.integers(0, kv_rows - 1, size=q_rows)
        ends = np.minimum(starts + rng.integers(1, max(2, kv_rows), size=q_rows), kv_rows)
        visible = np.stack([starts, ends], axis=1)
    what = f"block {it}: {kv} d={d} {hq}/{hkv} q={q_kind} page={page} rows={q_rows} keys={kv_rows} workspace={workspace}"
    print(what, flush=True)
    out, want = run_block(11000 + it, q_rows, kv_rows, hq, hkv, d, visible, kv=kv, q_kind=q_kind, block_tokens=page, workspace=workspace)
    assert_attention_close(out, want, what)


def test_the_cases_that_found_the_query_step_stay_far_inside_the_bound(monkeypatch):
    """Nine draws of the sweeps once exceeded 2e-3 through the query alone (a fixed-point step of 2^-15 of the row's largest
    element in the decode kernels, f16's eleven bits for an f32 query in the chunk kernel).  With three query digits and
    hi + lo fragments they measure 1.5e-5 to 1.4e-4 on outputs of magnitude 12 to 22: held to 4e-4 here, a fifth of the
    bound, so that a query carried with fewer bits again shows."""
    import sys

    this = sys.modules[__name__]
    usual = assert_attention_close
    monkeypatch.setattr(this, "assert_attention_close", lambda got, want, what="", atol=4e-4, rtol=1e-2: usual(got, want, what, atol=4e-4, rtol=rtol))
    for it in (52, 190, 266, 814):
        test_random_q8_decode_pages_rules_and_hints(it)
    for it in (265, 273, 497):
        test_random_q8_decode(it)
    test_random_q8_head_dim_192(779)
    test_random_q8_prefill_chunk(1298)

"""Parity of the split-KV GQA decode kernels with the CPU oracle, through the C ABI.

Tolerance (stated by the north star): max-abs <= 2e-3 and relative <= 1e-2, fp32 accumulation.
"""
import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, draw_tables, make_gqa_q8_case, oracle_gqa_decode, to_torch_bf16, upload

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def run_decode(case, score_scale, window=0, softcap=0.0, max_kv_len=None, ring_capacity=0, gate=None, total_kv_tokens=0):
    from zllm_amd import capi, ops

    pl = case["planes"]
    lens = case["lens"]
    q = to_torch_bf16(case["q_bits"], "cuda") if case["q_bits"] is not None else upload(case["q"])
    first = None
    if window:
        first = upload(np.array([O.key_range(window, int(l) - 1, int(l))[0] if l else 0 for l in lens], dtype=np.uint32))
    out = ops.gqa_decode(q, upload(pl["k_codes"]), upload(pl["k_scales"]), upload(pl["v_codes"]), upload(pl["v_scales"]),
                         upload(case["tables"]), upload(lens), case["hq"], case["hkv"], case["d"], case["block_tokens"],
                         score_scale, max_kv_len or max(int(lens.max()), 1), first_visible=first, softcap=softcap,
                         ring_capacity=ring_capacity, kv_format=capi.KV_Q8G64, scale_dtype=case["scale_dtype"], gate=gate,
                         total_kv_tokens=total_kv_tokens)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("hq,hkv,d,lens,window,gated", [(64, 8, 128, [9000], 0, False), (16, 2, 128, [20000], 0, True),
                                                        (32, 4, 128, [9000, 100], 5000, False), (16, 8, 256, [5000], 0, True),
                                                        (32, 8, 64, [17000], 0, False)])
def test_one_or_two_long_sequences_take_the_wide_merge(hq, hkv, d, lens, window, gated):
    """A sequence alone on the GPU is cut into a split per compute unit and KV-head block, 128 to 512 records per head:
    the merge then runs as head_dim / 32 workgroups per (head, sequence), one round trip for 256 records (20,000 tokens of
    two KV heads: 313 records, two trips).  With a short sequence beside the long one, a window, and the fused gate."""
    case = make_gqa_q8_case(70 + hq, lens, hq, hkv, d, outliers=True)
    gate = dev_gate = None
    if gated:
        gate = (np.random.default_rng(71).standard_normal((len(lens), hq * d)) * 3).astype(np.float32)
        dev_gate = upload(gate)
    got = run_decode(case, 0.09, window=window, gate=dev_gate)
    want = oracle_gqa_decode(case, 0.09, window=window)
    if gated:
        rc, want = O.sigmoid_gate(want, gate)
        assert rc == 0
    print("wide merge", hq, hkv, d, lens, assert_attention_close(got, want, f"{hq}/{hkv} d={d} lens={lens}"))


@pytest.mark.parametrize("per_row,gate_bf16", [(False, False), (True, False), (False, True)])
def test_decode_output_gate(per_row, gate_bf16):
    """out * sigmoid(gate) fused into the split merge (src/attention/hybrid.rs:79, src/backend/cpu/context.rs:419-432)."""
    case = make_gqa_q8_case(91, [700, 33, 2049], 16, 4, 128)
    rng = np.random.default_rng(92)
    gate = (rng.standard_normal((3, 1 if per_row else 16 * 128)) * 3).astype(np.float32)
    if gate_bf16:
        gate = O.bf16_to_f32(O.f32_to_bf16(gate))
    dev_gate = to_torch_bf16(O.f32_to_bf16(gate), "cuda") if gate_bf16 else upload(gate)
    got = run_decode(case, 0.088, gate=dev_gate)
    rc, want = O.sigmoid_gate(oracle_gqa_decode(case, 0.088), gate)
    assert rc == 0
    assert_attention_close(got, want, "gated decode")


def test_config1_cpu_oracle_case():
    """Benchmark config 1: B=1, 16q/4kv, d=128, L=4096, f32 q, f16 scales, 16-token pages, random table."""
    case = make_gqa_q8_case(1, [4096], 16, 4, 128)
    scale = 1.0 / np.sqrt(128.0)
    got = run_decode(case, scale)
    want = oracle_gqa_decode(case, scale)
    print("config1", assert_attention_close(got, want, "config 1"))


def test_config2_shape_ragged_batch_bf16_queries_outliers():
    """Benchmark config 2 at oracle-sized lengths: B=8, 64q/8kv, ragged, bf16 q, 1 % outlier channels x8."""
    rng = np.random.default_rng(2)
    lens = rng.integers(100, 3000, size=8)
    case = make_gqa_q8_case(2, lens, 64, 8, 128, outliers=True, q_bf16=True)
    scale = 1.0 / np.sqrt(128.0)
    got = run_decode(case, scale)
    want = oracle_gqa_decode(case, scale)
    print("config2-small", assert_attention_close(got, want, "config 2 (small)"))


@pytest.mark.parametrize("block_tokens,layout", [(1, "random"), (4, "random"), (64, "reversed"), (128, "identity"), (1024, "random"), (48, "random")])
def test_page_sizes_and_tables(block_tokens, layout):
    """block_size is a run-time argument in the reference (tests use 1, 4, 64, 128, 1024); 48 is not a power of two."""
    case = make_gqa_q8_case(block_tokens, [777, 1500], 8, 2, 128, block_tokens=block_tokens, layout=layout)
    got = run_decode(case, 0.09)
    want = oracle_gqa_decode(case, 0.09)
    assert_attention_close(got, want, f"block_tokens={block_tokens}")


@pytest.mark.parametrize("lens", [[1], [15, 16, 17], [31, 32, 33, 0], [255, 256, 257, 1023], [0]])
def test_edge_lengths(lens):
    case = make_gqa_q8_case(sum(lens) + 3, lens, 16, 4, 128)
    got = run_decode(case, 0.1, max_kv_len=max(max(lens), 1))
    want = oracle_gqa_decode(case, 0.1)
    assert_attention_close(got, want, f"lens={lens}")
    for b, l in enumerate(lens):
        if l == 0:
            assert (got[b] == 0).all()  # nothing visible -> zeros, never NaN


@pytest.mark.parametrize("hq,hkv,d", [(8, 8, 128), (32, 1, 128), (40, 2, 128), (12, 3, 128), (8, 2, 64), (8, 2, 256), (64, 16, 128),
                                      (8, 2, 192), (12, 3, 192), (40, 1, 192), (16, 8, 192)])
def test_head_geometries(hq, hkv, d):
    case = make_gqa_q8_case(hq * 7 + d, [600, 90], hq, hkv, d)
    got = run_decode(case, 1.0 / np.sqrt(d))
    want = oracle_gqa_decode(case, 1.0 / np.sqrt(d))
    assert_attention_close(got, want, f"{hq}/{hkv} d={d}")


@pytest.mark.parametrize("rule", [O.RULE_ROCM_MLA, O.RULE_METAL_GQA])
def test_scale_storage_conventions(rule):
    case = make_gqa_q8_case(33 + rule, [900], 16, 4, 128, rule=rule)
    got = run_decode(case, 0.088)
    want = oracle_gqa_decode(case, 0.088)
    assert_attention_close(got, want, f"rule={rule}")


@pytest.mark.parametrize("window", [1, 100, 1024])
def test_sliding_window(window):
    case = make_gqa_q8_case(70 + window, [2100, 50, 1024], 16, 4, 128)
    got = run_decode(case, 0.088, window=window)
    want = oracle_gqa_decode(case, 0.088, window=window)
    assert_attention_close(got, want, f"window={window}")


def test_softcap():
    case = make_gqa_q8_case(81, [1200, 333], 16, 8, 128, q_std=4.0)
    got = run_decode(case, 0.5, softcap=50.0)
    want = oracle_gqa_decode(case, 0.5, softcap=50.0)
    assert_attention_close(got, want, "softcap 50")
    plain = run_decode(case, 0.5)
    assert np.abs(plain - got).max() > 1e-4  # the cap changes these logits
    huge = run_decode(case, 0.5, softcap=1e9)
    assert_attention_close(huge, oracle_gqa_decode(case, 0.5), "softcap -> inf recovers the uncapped result")


def test_zero_query_gives_mean_of_values_and_split_invariance():
    case = make_gqa_q8_case(90, [5000], 8, 2, 128)
    case["q"][:] = 0.0
    got = run_decode(case, 0.1)
    v = O.gather_dequant_rows(O.FMT_Q8, case["planes"]["v_codes"], case["planes"]["v_scales"], case["scale_dtype"],
                              case["tables"][0], 16, 0, 5000, 256)
    mean = v.reshape(5000, 2, 128).mean(0)
    assert np.abs(got.reshape(8, 128) - np.repeat(mean, 4, axis=0)).max() < 1e-4
    # any number of KV splits gives the same answer: max_kv_len only changes the split plan
    case2 = make_gqa_q8_case(91, [5000], 8, 2, 128)
    case2["tables"] = np.pad(case2["tables"], ((0, 0), (0, 25000 - case2["tables"].shape[1])))
    a = run_decode(case2, 0.1, max_kv_len=5000)
    b = run_decode(case2, 0.1, max_kv_len=400000)
    assert np.abs(a - b).max() < 2e-5


def test_dominant_key_returns_its_value_row():
    case = make_gqa_q8_case(92, [3000], 8, 2, 128)
    k = O.gather_dequant_rows(O.FMT_Q8, case["planes"]["k_codes"], case["planes"]["k_scales"], case["scale_dtype"],
                              case["tables"][0], 16, 1234, 1, 256).reshape(2, 128)
    case["q"][0] = np.repeat(k, 4, axis=0).reshape(-1) * 3.0  # |k|^2 * 3 ~ 380 >> any other logit
    got = run_decode(case, 1.0)
    want = oracle_gqa_decode(case, 1.0)
    assert_attention_close(got, want, "dominant key")
    v = O.gather_dequant_rows(O.FMT_Q8, case["planes"]["v_codes"], case["planes"]["v_scales"], case["scale_dtype"],
                              case["tables"][0], 16, 1234, 1, 256).reshape(2, 128)
    assert np.abs(got.reshape(8, 128) - np.repeat(v, 4, axis=0)).max() < 1e-4


def test_large_pool_exercises_64_bit_offsets():
    """Physical block ids beyond 2^32 bytes of plane offset (the reference casts to u64 for the same reason)."""
    from zllm_amd import capi, ops

    hq, hkv, d, bt = 16, 8, 128, 16
    cols = hkv * d
    pool_rows = (5 << 30) // cols  # 5 GiB codes plane per tensor
    pool_blocks = pool_rows // bt
    rng = np.random.default_rng(5)
    lens = [700]
    nblk = (lens[0] + bt - 1) // bt
    table = np.sort(rng.choice(np.arange(pool_blocks - 4096, pool_blocks), size=nblk, replace=False)).astype(np.uint32)[::-1].copy()
    k = rng.standard_normal((lens[0], cols)).astype(np.float32)
    v = rng.standard_normal((lens[0], cols)).astype(np.float32)
    q = rng.standard_normal((1, hq * d)).astype(np.float32)
    kc = torch.zeros((pool_rows, cols), dtype=torch.int8, device="cuda")
    vc = torch.zeros((pool_rows, cols), dtype=torch.int8, device="cuda")
    ks = torch.zeros((pool_rows, cols // 64), dtype=torch.int16, device="cuda")
    vs = torch.zeros((pool_rows, cols // 64), dtype=torch.int16, device="cuda")
    tbl = upload(table)
    ops.q8g64_append(upload(k), kc, ks, tbl, 0, bt, capi.QUANT_METAL_GQA)
    ops.q8g64_append(upload(v), vc, vs, tbl, 0, bt, capi.QUANT_METAL_GQA)
    out = ops.gqa_decode(upload(q), kc, ks, vc, vs, tbl.view(1, -1), upload(np.array(lens, dtype=np.uint32)), hq, hkv, d, bt,
                         0.088, lens[0]).cpu().numpy()
    # oracle on a compact identity pool built from the same rows
    codes = np.zeros((nblk * bt, cols), dtype=np.int8)
    kscale = np.zeros((nblk * bt, cols // 64), dtype=np.uint16)
    vcodes, vscale = codes.copy(), kscale.copy()
    O.q8g64_append_paged(O.RULE_METAL_GQA, k, codes, kscale, None, 0, bt)
    O.q8g64_append_paged(O.RULE_METAL_GQA, v, vcodes, vscale, None, 0, bt)
    # the appended device bytes are the oracle's bytes (gathered back through the far table)
    got_rows = ops.gather_rows(kc, tbl, 0, lens[0], cols, bt).cpu().numpy()
    assert np.array_equal(got_rows.view(np.int8), codes[: lens[0]])
    kd = O.gather_dequant_rows(O.FMT_Q8, codes, kscale, O.SCALE_F16, None, bt, 0, lens[0], cols)
    vd = O.gather_dequant_rows(O.FMT_Q8, vcodes, vscale, O.SCALE_F16, None, bt, 0, lens[0], cols)
    rc, want = O.gqa_prefill_at_visible(q, kd, vd, 0, lens[0], lens[0] - 1, hq, hkv, d, score_scale=0.088)
    assert rc == 0
    assert_attention_close(out, want, "far pool")


def test_pages_spread_over_64_gib_give_the_compact_pool_bits():
    """Config 2's geometry with every sequence's pages drawn from all over a 64 GiB code plane (the span the benchmark's
    pool has per plane and more than a serving pool hands one sequence), beside the same rows in a compact pool: where a
    page lies changes no bit of the output, and both meet the oracle."""
    from zllm_amd import capi, ops

    hq, hkv, d, bt = 64, 8, 128, 16
    cols = hkv * d
    lens = [8192, 3000, 8192, 1025]
    rng = np.random.default_rng(64)
    blocks = [(l + bt - 1) // bt for l in lens]
    stride = max(blocks)
    far_blocks = (64 << 30) // (cols * bt)
    far_ids = rng.choice(far_blocks, size=sum(blocks), replace=False).astype(np.uint32)
    far_ids[0], far_ids[-1] = far_blocks - 1, 0  # both ends of the plane are in use
    near_ids = rng.permutation(sum(blocks)).astype(np.uint32)
    q_bits = O.f32_to_bf16(rng.standard_normal((len(lens), hq * d)).astype(np.float32))
    rows = [(rng.standard_normal((l, cols)).astype(np.float32), rng.standard_normal((l, cols)).astype(np.float32)) for l in lens]
    torch.cuda.empty_cache()
    outs = {}
    for name, ids, pool_blocks in (("near", near_ids, sum(blocks)), ("far", far_ids, far_blocks)):
        tables = np.zeros((len(lens), stride), dtype=np.uint32)
        at = 0
        for b, n in enumerate(blocks):
            tables[b, :n] = ids[at:at + n]
            at += n
        kc = torch.empty((pool_blocks * bt, cols), dtype=torch.int8, device="cuda")
        vc = torch.empty((pool_blocks * bt, cols), dtype=torch.int8, device="cuda")
        ks = torch.empty((pool_blocks * bt, cols // 64), dtype=torch.int16, device="cuda")
        vs = torch.empty((pool_blocks * bt, cols // 64), dtype=torch.int16, device="cuda")
        tbl = upload(tables)
        for b, (k, v) in enumerate(rows):
            ops.q8g64_append(upload(k), kc, ks, tbl[b], 0, bt, capi.QUANT_METAL_GQA)
            ops.q8g64_append(upload(v), vc, vs, tbl[b], 0, bt, capi.QUANT_METAL_GQA)
        out = ops.gqa_decode(to_torch_bf16(q_bits, "cuda"), kc, ks, vc, vs, tbl, upload(np.array(lens, dtype=np.uint32)), hq, hkv, d, bt,
                             0.088, max(lens))
        torch.cuda.synchronize()
        outs[name] = out.cpu().numpy()
        if name == "far":
            assert int(tables.max()) * bt * cols >= (64 << 30) - bt * cols
        del kc, vc, ks, vs
        torch.cuda.empty_cache()
    assert np.array_equal(outs["near"], outs["far"])
    q = O.bf16_to_f32(q_bits)
    for b, (k, v) in enumerate(rows):
        l = lens[b]
        codes = np.zeros((blocks[b] * bt, cols), dtype=np.int8)
        kscale = np.zeros((blocks[b] * bt, cols // 64), dtype=np.uint16)
        vcodes, vscale = codes.copy(), kscale.copy()
        O.q8g64_append_paged(O.RULE_METAL_GQA, k, codes, kscale, None, 0, bt)
        O.q8g64_append_paged(O.RULE_METAL_GQA, v, vcodes, vscale, None, 0, bt)
        kd = O.gather_dequant_rows(O.FMT_Q8, codes, kscale, O.SCALE_F16, None, bt, 0, l, cols)
        vd = O.gather_dequant_rows(O.FMT_Q8, vcodes, vscale, O.SCALE_F16, None, bt, 0, l, cols)
        rc, want = O.gqa_prefill_at_visible(q[b:b + 1], kd, vd, 0, l, l - 1, hq, hkv, d, score_scale=0.088)
        assert rc == 0
        assert_attention_close(outs["far"][b:b + 1], want, f"pages over 64 GiB, sequence {b}")


# ---------------------------------------------------------------------------- f16 KV (config 3)
def make_f16_case(seed, lens, hq, hkv, d, block_tokens=16, ring_capacity=0, k_gain=1.0, v_gain=1.0, q_std=1.0, poison=False, outliers=False):
    rng = np.random.default_rng(seed)
    cols = hkv * d
    channel_gain = np.ones(cols, dtype=np.float32)
    if outliers:  # 1 % of the channels carry values eight times larger
        channel_gain[rng.choice(cols, size=max(1, cols // 100), replace=False)] = 8.0
    cap_lens = [min(l, ring_capacity) if ring_capacity else l for l in lens]
    tables, pool_blocks = draw_tables(rng, cap_lens, block_tokens)
    rows = pool_blocks * block_tokens
    planes = {"k": np.zeros((rows, cols), dtype=np.uint16), "v": np.zeros((rows, cols), dtype=np.uint16)}
    if poison:  # rows no sequence wrote: f16 NaN
        planes["k"][:] = 0x7E00
        planes["v"][:] = 0x7E00
    for b, l in enumerate(lens):
        kg = np.reshape(np.asarray(k_gain, dtype=np.float32), (-1, 1))
        vg = np.reshape(np.asarray(v_gain, dtype=np.float32), (-1, 1))
        k = rng.standard_normal((l, cols)).astype(np.float32) * channel_gain * (kg if kg.shape[0] == 1 else kg[:l])
        v = rng.standard_normal((l, cols)).astype(np.float32) * channel_gain * (vg if vg.shape[0] == 1 else vg[:l])
        O.half_append_paged(1, k, planes["k"], tables[b], 0, block_tokens, ring_capacity=ring_capacity)
        O.half_append_paged(1, v, planes["v"], tables[b], 0, block_tokens, ring_capacity=ring_capacity)
    q = (rng.standard_normal((len(lens), hq * d)) * q_std).astype(np.float32)
    return dict(q=q, q_bits=None, lens=np.array(lens, dtype=np.uint32), tables=tables, planes=planes, hq=hq, hkv=hkv, d=d,
                block_tokens=block_tokens, scale_dtype=0)


def run_f16(case, score_scale, window=0, softcap=0.0, ring_capacity=0):
    from zllm_amd import capi, ops

    lens = case["lens"]
    first = None
    if window:
        first = upload(np.array([O.key_range(window, int(l) - 1, int(l))[0] for l in lens], dtype=np.uint32))
    out = ops.gqa_decode(upload(case["q"]), upload(case["planes"]["k"]), None, upload(case["planes"]["v"]), None,
                         upload(case["tables"]), upload(lens), case["hq"], case["hkv"], case["d"], case["block_tokens"],
                         score_scale, int(lens.max()), first_visible=first, softcap=softcap, ring_capacity=ring_capacity,
                         kv_format=capi.KV_F16)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("window,ring", [(0, 0), (1024, 0), (1024, 1024)])
def test_config3_f16_kv_sliding_window_softcap(window, ring):
    """Benchmark config 3: B=4, 16q/8kv, d=256, ctx 8192, window 1024 on sliding layers (optionally stored as a
    1024-row ring), soft-cap 50."""
    case = make_f16_case(3, [8192, 8192, 5000, 8192], 16, 8, 256, ring_capacity=ring)
    scale = 1.0 / 16.0
    got = run_f16(case, scale, window=window, softcap=50.0, ring_capacity=ring)
    want = oracle_gqa_decode(case, scale, window=window, softcap=50.0, fmt=O.FMT_F16, ring_capacity=ring)
    print("config3", window, ring, assert_attention_close(got, want, f"config 3 window={window} ring={ring}"))


def test_f16_kv_head_dim_128():
    case = make_f16_case(4, [333, 1000], 8, 2, 128, block_tokens=64)
    got = run_f16(case, 0.088)
    want = oracle_gqa_decode(case, 0.088, fmt=O.FMT_F16)
    assert_attention_close(got, want, "f16 d=128")


def test_batch_larger_than_a_wave_with_empty_sequences():
    """Work items are numbered over the batch by a 64-lane prefix sum: 70 sequences need two passes of it, and
    empty sequences in the middle must take no work item and still produce zero rows."""
    rng = np.random.default_rng(70)
    lens = rng.integers(1, 600, size=70)
    lens[[3, 17, 64, 69]] = 0
    case = make_gqa_q8_case(70, lens, 8, 2, 128)
    got = run_decode(case, 0.1)
    want = oracle_gqa_decode(case, 0.1)
    assert_attention_close(got, want, "batch 70")
    assert not got[[3, 17, 64, 69]].any()


@pytest.mark.parametrize("fmt,hq,hkv,d,window", [("q8", 8, 1, 128, 0), ("q8", 16, 2, 128, 100), ("q8", 6, 3, 128, 0), ("q8", 4, 1, 64, 0),
                                                  ("q8", 8, 2, 64, 33), ("q8", 4, 1, 256, 0), ("q8", 16, 2, 256, 700), ("q8", 6, 3, 256, 0),
                                                  ("f16", 8, 1, 128, 0), ("f16", 4, 2, 128, 64), ("f16", 4, 1, 256, 0), ("f16", 32, 2, 256, 500),
                                                  ("f16", 6, 3, 256, 0)])
def test_few_kv_heads_share_a_workgroup(fmt, hq, hkv, d, window):
    """With one to three KV heads a workgroup runs several (sequence, split) items side by side.  The item count here
    is not a multiple of the items in a workgroup (the last workgroup has idle waves), one sequence is empty and the
    lengths cut into different numbers of splits."""
    lens = [1000, 0, 37, 2049, 515, 3000, 64]
    if fmt == "q8":
        case = make_gqa_q8_case(900 + hq + d, lens, hq, hkv, d, outliers=True)
        got = run_decode(case, 0.09, window=window)
        want = oracle_gqa_decode(case, 0.09, window=window)
        hinted = run_decode(case, 0.09, window=window, total_kv_tokens=sum(lens))  # the ragged plan counts the shared workgroups too
        assert_attention_close(hinted, want, f"{fmt} {hq}/{hkv} d={d} window={window} with the token-count hint")
    else:
        case = make_f16_case(900 + hq + d, lens, hq, hkv, d)
        got = run_f16(case, 0.09, window=window)
        want = oracle_gqa_decode(case, 0.09, window=window, fmt=O.FMT_F16)
    assert_attention_close(got, want, f"{fmt} {hq}/{hkv} d={d} window={window}")
    assert not got[1].any()


@pytest.mark.parametrize("d", [64, 128, 256])
def test_every_kv_head_count_fits_its_workgroup(d):
    """One to eight KV heads at every head_dim: waves x items of a workgroup must stay inside the kernels' launch bounds
    (three KV heads of head_dim 256 once asked for 384 threads of a 256-thread kernel), Q8g64 and f16 rows alike."""
    for hkv in range(1, 9):
        lens = [130, 0, 700]
        case = make_gqa_q8_case(1200 + 10 * d + hkv, lens, 2 * hkv, hkv, d)
        assert_attention_close(run_decode(case, 0.09), oracle_gqa_decode(case, 0.09), f"q8 {2 * hkv}/{hkv} d={d}")
        if d != 64:
            case = make_f16_case(1300 + 10 * d + hkv, lens, 2 * hkv, hkv, d)
            assert_attention_close(run_f16(case, 0.09), oracle_gqa_decode(case, 0.09, fmt=O.FMT_F16), f"f16 {2 * hkv}/{hkv} d={d}")


@pytest.mark.parametrize("q_kind", ["f32", "bf16", "f16"])
def test_query_dtypes_through_fixed_point_digits(q_kind):
    """The kernel quantizes each query row to 24-bit fixed point (three signed-byte digits) for the int8 matrix cores; every input
    dtype must stay within the attention tolerance, including rows whose elements span a wide range."""
    from zllm_amd import capi, ops

    case = make_gqa_q8_case(11, [900, 333], 16, 4, 128)
    q = case["q"].copy().reshape(2, 16, 128)
    q[0, 0, :] *= 1e-3           # a tiny head
    q[0, 1, 5] = 40.0            # one dominant element: the other 127 fall to few fixed-point levels
    q[1, 2, :] = 0.0             # an all-zero head: uniform attention
    q = q.reshape(2, -1)
    if q_kind == "bf16":
        qt = torch.from_numpy(q).to(torch.bfloat16)
    elif q_kind == "f16":
        qt = torch.from_numpy(q).to(torch.float16)
    else:
        qt = torch.from_numpy(q)
    case["q"] = qt.float().numpy()
    case["q_bits"] = None
    pl, lens = case["planes"], case["lens"]
    out = ops.gqa_decode(qt.cuda(), upload(pl["k_codes"]), upload(pl["k_scales"]), upload(pl["v_codes"]), upload(pl["v_scales"]),
                         upload(case["tables"]), upload(lens), 16, 4, 128, case["block_tokens"], 0.09, int(lens.max()),
                         kv_format=capi.KV_Q8G64, scale_dtype=case["scale_dtype"])
    torch.cuda.synchronize()
    want = oracle_gqa_decode(case, 0.09)
    assert_attention_close(out.cpu().numpy(), want, f"q dtype {q_kind}")


def _close_at_scale(got, want, what):
    """The 2e-3 / 1e-2 bounds, with the absolute one taken relative to the largest expected magnitude."""
    assert np.isfinite(got).all(), what
    top = float(np.abs(want).max())
    assert top > 0
    return assert_attention_close(got / top, want / top, what)


@pytest.mark.parametrize("rule,exponent", [(O.RULE_ROCM_MLA, 40), (O.RULE_ROCM_MLA, -40), (O.RULE_METAL_GQA, 11), (O.RULE_METAL_GQA, -12)])
def test_q8_value_and_key_magnitudes(rule, exponent):
    """Scales far from 1 in both 16-bit storage conventions: uniformly, with the large rows first, last, or alone in the
    middle; keys and queries scaled against a compensating score scale."""
    lens = [1500, 300, 64]
    flat = float(2.0 ** exponent)
    case = make_gqa_q8_case(500, lens, 16, 4, 128, rule=rule, v_gain=flat)
    print("uniform v", _close_at_scale(run_decode(case, 0.088), oracle_gqa_decode(case, 0.088), f"v * 2^{exponent}"))
    big = float(2.0 ** abs(exponent))
    for name, rows in (("large first", slice(0, 40)), ("large last", slice(1400, 1500)), ("spike", slice(700, 701))):
        gain = np.ones(max(lens), dtype=np.float32)
        gain[rows] = big
        case = make_gqa_q8_case(501, lens, 16, 4, 128, rule=rule, v_gain=gain)
        print(name, _close_at_scale(run_decode(case, 0.088), oracle_gqa_decode(case, 0.088), f"{name}, 2^{abs(exponent)}"))
    scale = 0.088 / flat
    case = make_gqa_q8_case(502, lens, 16, 4, 128, rule=rule, k_gain=flat)
    print("k", assert_attention_close(run_decode(case, scale), oracle_gqa_decode(case, scale), f"k * 2^{exponent}"))
    case = make_gqa_q8_case(503, lens, 16, 4, 128, rule=rule, q_std=flat)
    print("q", assert_attention_close(run_decode(case, scale), oracle_gqa_decode(case, scale), f"q * 2^{exponent}"))


@pytest.mark.parametrize("exponent", [10, -10])
def test_f16_kv_magnitudes(exponent):
    """f16 K/V near the ends of what f16 rows can hold, and queries far from unit size."""
    lens = [2000, 77]
    flat = float(2.0 ** exponent)
    case = make_f16_case(510, lens, 16, 8, 256, v_gain=flat)
    print("uniform v", _close_at_scale(run_f16(case, 0.0625), oracle_gqa_decode(case, 0.0625, fmt=O.FMT_F16), f"v * 2^{exponent}"))
    gain = np.full(max(lens), 2.0 ** -abs(exponent), dtype=np.float32)
    gain[1234] = 2.0 ** abs(exponent)
    case = make_f16_case(511, lens, 16, 8, 256, v_gain=gain)
    print("spike", _close_at_scale(run_f16(case, 0.0625), oracle_gqa_decode(case, 0.0625, fmt=O.FMT_F16), "one large row"))
    case = make_f16_case(512, lens, 16, 8, 256, k_gain=flat)
    print("k", assert_attention_close(run_f16(case, 0.0625 / flat), oracle_gqa_decode(case, 0.0625 / flat, fmt=O.FMT_F16), f"k * 2^{exponent}"))
    case = make_f16_case(513, lens, 16, 8, 256, q_std=flat * flat)
    print("q", assert_attention_close(run_f16(case, 0.0625 / (flat * flat)), oracle_gqa_decode(case, 0.0625 / (flat * flat), fmt=O.FMT_F16), "q"))


# ---------------------------------------------------------------------------- pools that were never cleared
@pytest.mark.parametrize("hq,hkv,d,block_tokens,rule", [(8, 2, 64, 16, O.RULE_METAL_GQA), (16, 4, 128, 16, O.RULE_METAL_GQA),
                                                       (64, 8, 128, 16, O.RULE_METAL_GQA), (8, 2, 256, 32, O.RULE_ROCM_MLA),
                                                       (16, 4, 128, 64, O.RULE_ROCM_MLA)])
@pytest.mark.parametrize("window", [0, 1000])
def test_q8_rows_outside_the_visible_range_contribute_nothing(hq, hkv, d, block_tokens, rule, window):
    """The caller owns the pool and need not clear it: the rest of a sequence's last page holds NaN scale bits and the
    code -128 here.  The fast paths load whole 16-token tiles, so those rows (and, with a window, the rows in front of
    a first visible token that is not tile-aligned: 2100 - 1000 = 1100 = 68 * 16 + 12) are really read; masked rows
    must multiply as exact zeros."""
    lens = [2100, 1, 17, 33, 1023, 4099]
    case = make_gqa_q8_case(600 + d + block_tokens, lens, hq, hkv, d, block_tokens=block_tokens, rule=rule, poison=True, q_bf16=True)
    got = run_decode(case, 1.0 / np.sqrt(d), window=window)
    assert np.isfinite(got).all()
    assert_attention_close(got, oracle_gqa_decode(case, 1.0 / np.sqrt(d), window=window), f"poisoned pool d={d} window={window}")


@pytest.mark.parametrize("d,block_tokens", [(128, 16), (256, 64)])
@pytest.mark.parametrize("window", [0, 1000])
def test_f16_rows_outside_the_visible_range_contribute_nothing(d, block_tokens, window):
    lens = [2100, 1, 17, 33, 1023]
    case = make_f16_case(700 + d, lens, 16, 8, d, block_tokens=block_tokens, poison=True)
    got = run_f16(case, 1.0 / np.sqrt(d), window=window)
    assert np.isfinite(got).all()
    assert_attention_close(got, oracle_gqa_decode(case, 1.0 / np.sqrt(d), window=window, fmt=O.FMT_F16), f"poisoned f16 pool d={d}")


# ---------------------------------------------------------------------------- Q8g64 sliding window stored as a ring
@pytest.mark.parametrize("d,ring,window,block_tokens", [(128, 1024, 1024, 16), (128, 1000, 1000, 16), (256, 512, 400, 32),
                                                        (128, 200, 150, 8), (256, 1000, 1000, 16)])
def test_q8_sliding_window_ring(d, ring, window, block_tokens):
    """token -> token % capacity before the page lookup (src/kernel/cuda/attention.rs:82-88,108-116): a ring that is a
    multiple of 16 rows keeps the tile path (per-tile table lookups), any other capacity takes the per-token path; the
    sequences are longer than the ring, so the visible window wraps."""
    lens = [3 * ring + 77, ring - 5, ring, 2 * ring + 1]
    case = make_gqa_q8_case(800 + ring, lens, 16, 4, d, block_tokens=block_tokens, ring_capacity=ring, poison=True)
    scale = 1.0 / np.sqrt(d)
    got = run_decode(case, scale, window=window, ring_capacity=ring)
    want = oracle_gqa_decode(case, scale, window=window, ring_capacity=ring)
    assert_attention_close(got, want, f"Q8 ring {ring} window {window} d={d}")


# ---------------------------------------------------------------------------- every way a split can end
def test_splits_of_one_to_six_steps():
    """The head_dim-128 streaming kernel runs its steps in pairs and ends a split with one, two or three steps that
    request nothing further, each with its own wait counts.  64 sequences with one split plan of 160-token parts
    (max_kv_len 640) give splits of 1 to 5 steps, alone and behind full parts, with and without a ragged last tile;
    poisoned pool tails make a step that waited for too little show as NaN or as a wrong row."""
    lens = [1, 16, 17, 32, 33, 64, 65, 96, 97, 128, 129, 159, 160, 161, 192, 200, 224, 256, 288, 320, 321, 352, 384, 400, 416, 448,
            479, 480, 481, 512, 544, 576, 600, 608, 639, 640] + [int(x) for x in np.random.default_rng(5).integers(1, 641, size=28)]
    case = make_gqa_q8_case(905, lens, 16, 8, 128, block_tokens=16, poison=True, q_bf16=True)
    scale = 1.0 / np.sqrt(128.0)
    got = run_decode(case, scale, max_kv_len=640)
    assert np.isfinite(got).all()
    assert_attention_close(got, oracle_gqa_decode(case, scale), "splits of 1..5 steps")
    # one long sequence: six-step splits and more, all full
    case = make_gqa_q8_case(906, [192 * 256], 16, 8, 128, block_tokens=16, q_bf16=True)
    got = run_decode(case, scale)
    assert_attention_close(got, oracle_gqa_decode(case, scale), "six-step splits")


# ---------------------------------------------------------------------------- the benchmarked shape at its full size
def _oracle_rows(case, rows, scale):
    sub = dict(case)
    sub["lens"] = case["lens"][rows]
    sub["tables"] = case["tables"][rows]
    sub["q"] = case["q"][rows]
    return oracle_gqa_decode(sub, scale)


@pytest.mark.parametrize("ragged", [False, True])
def test_config2_full_size(ragged):
    """Benchmark config 2 at its own size -- B = 8, 64q/8kv, d = 128, 16-token pages, bf16 queries, outlier channels --
    every sequence at 32,768 tokens (the kernel instantiation and split plan the bench times) and the ragged draw in
    [1024, 32768].  The oracle runs on two sequences of the call's output; the zero-query mean is checked on one."""
    rng = np.random.default_rng(2)
    lens = [int(x) for x in rng.integers(1024, 32769, size=8)] if ragged else [32768] * 8
    case = make_gqa_q8_case(2, lens, 64, 8, 128, outliers=True, q_bf16=True)
    scale = 1.0 / np.sqrt(128.0)
    got = run_decode(case, scale, total_kv_tokens=sum(lens))  # the bench passes the same hint
    picks = [0, int(np.argmax(lens)) if ragged else 5]
    want = _oracle_rows(case, picks, scale)
    print("config2 full", ragged, assert_attention_close(got[picks], want, f"config 2 full size ragged={ragged}"))
    case["q"][:] = 0.0
    case["q_bits"][:] = 0
    zero = run_decode(case, scale, total_kv_tokens=sum(lens))
    b = picks[1]
    v = O.gather_dequant_rows(O.FMT_Q8, case["planes"]["v_codes"], case["planes"]["v_scales"], case["scale_dtype"], case["tables"][b],
                              16, 0, lens[b], 1024).astype(np.float64)
    mean = v.reshape(lens[b], 8, 128).mean(0)
    assert np.abs(zero[b].reshape(64, 128) - np.repeat(mean, 8, axis=0)).max() < 1e-4


@pytest.mark.parametrize("d,hq,hkv,lens,block_tokens,window", [(128, 16, 4, [700, 33, 2049], 16, 0), (64, 8, 2, [300, 1], 16, 0),
                                                              (256, 8, 2, [1500, 97], 64, 128), (128, 8, 8, [555], 4, 0)])
def test_f32_scale_cache(d, hq, hkv, lens, block_tokens, window):
    """Q8g64 with f32 scales, the CUDA backend's convention (src/kernel/cuda/attention.rs:331-341, dequantised at :391):
    the appends write such caches (tests/test_gpu_append.py), the decode kernels read them."""
    case = make_gqa_q8_case(d + len(lens), lens, hq, hkv, d, block_tokens=block_tokens, rule=O.RULE_CUDA_GQA)
    assert case["scale_dtype"] == O.SCALE_F32
    scale = 1.0 / np.sqrt(d)
    got = run_decode(case, scale, window=window)
    want = oracle_gqa_decode(case, scale, window=window)
    print("f32 scales", d, assert_attention_close(got, want, f"f32 scales d={d}"))


@pytest.mark.parametrize("rule,page,window,softcap,gated", [(O.RULE_METAL_GQA, 16, 0, 0.0, False), (O.RULE_ROCM_MLA, 64, 500, 0.0, True),
                                                            (O.RULE_CUDA_GQA, 1, 0, 30.0, False), (O.RULE_METAL_GQA, 48, 37, 50.0, True)])
def test_head_dim_192(rule, page, window, softcap, gated):
    """Three Q8g64 groups a head (the reference takes any head_dim up to 256, src/kernel/rocm/hip/tensor/attention.rs:1022):
    bf16, f16 and f32 scales, pages of 1 to 64 tokens, sliding windows, the soft cap, the fused gate, an empty sequence,
    lengths that cut into different numbers of splits, with and without the token-count hint."""
    lens = [3000, 0, 33, 1, 700, 64, 2049]
    case = make_gqa_q8_case(192 + page, lens, 16, 4, 192, block_tokens=page, rule=rule, outliers=True, poison=True)
    gate = None
    if gated:
        gate = np.random.default_rng(5).standard_normal((len(lens), 16 * 192)).astype(np.float32)
    scale = 1.0 / np.sqrt(192.0)
    want = oracle_gqa_decode(case, scale, window=window, softcap=softcap)
    if gate is not None:
        rc, want = O.sigmoid_gate(want.reshape(len(lens), -1), gate)
        assert rc == 0
    got = run_decode(case, scale, window=window, softcap=softcap, gate=None if gate is None else upload(gate))
    assert_attention_close(got, want.reshape(got.shape), f"d=192 rule={rule} page={page} window={window} cap={softcap}")
    visible = [min(l, window) if window else l for l in lens]
    hinted = run_decode(case, scale, window=window, softcap=softcap, gate=None if gate is None else upload(gate), total_kv_tokens=sum(visible))
    assert_attention_close(hinted, want.reshape(got.shape), "d=192 with the token-count hint")
    assert (got[1] == 0).all()


def test_head_dim_192_over_f16_is_refused():
    from zllm_amd import capi

    case = make_f16_case(7, [100], 8, 2, 128)
    case["d"] = 192
    with pytest.raises(capi.ZllmAttnError, match="f16 KV supports head_dim 128 and 256"):
        run_f16(case, 0.1)

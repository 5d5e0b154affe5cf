"""The pre-attention prologue of a GQA layer (per-head RMSNorm + RoPE of Q and K, quantizing page append of K and V) against
the CPU chain rmsnorm_heads -> rope_apply -> q8g64_append_paged, through the C ABI.  Q in f32, codes and scale bits are
compared bit for bit; the decode kernel is then run on the pages the prologue wrote."""
import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, draw_tables, upload

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def rope_table(rows, half, theta=10000.0):
    angles = np.arange(rows, dtype=np.float64)[:, None] / theta ** (np.arange(half, dtype=np.float64)[None, :] / half)
    return np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)


def cpu_chain(x, heads, d, weight, eps, offset, rotary, position, cos, sin, split_half):
    out = x
    if weight is not None:
        rc, out = O.rmsnorm_heads(out, heads, d, weight, eps, offset)
        assert rc == 0
    if rotary:
        rc, out = O.rope_apply(out, heads, rotary, position, cos, sin, layout=0 if split_half else 1, placement=0)
        assert rc == 0
    return out


@pytest.mark.parametrize("d,rotary,split_half,offset,rows,position", [(128, 128, True, 1.0, 1, 37), (128, 64, True, 1.0, 70, 5),
                                                                       (256, 128, False, 0.0, 9, 0), (64, 0, True, 1.0, 33, 11)])
def test_prologue_matches_cpu_chain_bit_for_bit(d, rotary, split_half, offset, rows, position):
    from zllm_amd import capi, ops

    rng = np.random.default_rng(d + rows)
    hq, hkv, bt, eps = 8, 2, 16, 1e-6
    q = rng.standard_normal((rows, hq * d)).astype(np.float32) * 3
    k = rng.standard_normal((rows, hkv * d)).astype(np.float32) * 0.2
    v = rng.standard_normal((rows, hkv * d)).astype(np.float32)
    k[:, :64] *= 40.0  # one loud group per row
    qw = (rng.standard_normal(d) * 0.2).astype(np.float32)
    kw = (rng.standard_normal(d) * 0.2).astype(np.float32)
    cos, sin = rope_table(position + rows + 3, max(rotary // 2, 1))
    tables, pool_blocks = draw_tables(rng, [position + rows], bt)
    pool_rows = pool_blocks * bt
    want_q = cpu_chain(q, hq, d, qw, eps, offset, rotary, position, cos, sin, split_half)
    want_k = cpu_chain(k, hkv, d, kw, eps, offset, rotary, position, cos, sin, split_half)
    ref = {n: np.zeros((pool_rows, hkv * d), dtype=np.int8) for n in ("k", "v")}
    ref_s = {n: np.zeros((pool_rows, hkv * d // 64), dtype=np.uint16) for n in ("k", "v")}
    O.q8g64_append_paged(O.RULE_METAL_GQA, want_k, ref["k"], ref_s["k"], tables[0], position, bt)
    O.q8g64_append_paged(O.RULE_METAL_GQA, v, ref["v"], ref_s["v"], tables[0], position, bt)
    dev = {n: torch.zeros((pool_rows, hkv * d), dtype=torch.int8, device="cuda") for n in ("k", "v")}
    dev_s = {n: torch.zeros((pool_rows, hkv * d // 64), dtype=torch.int16, device="cuda") for n in ("k", "v")}
    got_q = ops.gqa_prologue(upload(q), upload(k), upload(v), upload(qw), upload(kw), upload(cos) if rotary else None,
                             upload(sin) if rotary else None, dev["k"], dev_s["k"], dev["v"], dev_s["v"], upload(tables[0]),
                             position, hq, hkv, d, rotary, bt, eps=eps, weight_offset=offset, split_half=split_half)
    torch.cuda.synchronize()
    assert np.array_equal(got_q.cpu().numpy().view(np.uint32), want_q.view(np.uint32)), "Q bits differ"
    for n in ("k", "v"):
        assert np.array_equal(dev_s[n].cpu().numpy().view(np.uint16), ref_s[n]), f"{n} scale bits differ"
        assert np.array_equal(dev[n].cpu().numpy(), ref[n]), f"{n} codes differ"


def test_prologue_then_decode_matches_oracle_on_the_same_pages():
    """Token by token: prologue (bf16 projections in, bf16 Q out, position from device memory), then decode over the pages."""
    from zllm_amd import capi, ops

    rng = np.random.default_rng(3)
    hq, hkv, d, bt, steps, eps = 16, 4, 128, 16, 40, 1e-6
    cos, sin = rope_table(steps, d // 2)
    qw = (rng.standard_normal(d) * 0.1).astype(np.float32)
    kw = (rng.standard_normal(d) * 0.1).astype(np.float32)
    tables, pool_blocks = draw_tables(rng, [steps], bt)
    pool_rows = pool_blocks * bt
    dev = {n: torch.zeros((pool_rows, hkv * d), dtype=torch.int8, device="cuda") for n in ("k", "v")}
    dev_s = {n: torch.zeros((pool_rows, hkv * d // 64), dtype=torch.int16, device="cuda") for n in ("k", "v")}
    table = upload(tables[0])
    keys, values = [], []
    pos_dev = torch.zeros(1, dtype=torch.int32, device="cuda")
    for t in range(steps):
        q = O.bf16_to_f32(O.f32_to_bf16(rng.standard_normal((1, hq * d)).astype(np.float32)))
        k = O.bf16_to_f32(O.f32_to_bf16(rng.standard_normal((1, hkv * d)).astype(np.float32)))
        v = O.bf16_to_f32(O.f32_to_bf16(rng.standard_normal((1, hkv * d)).astype(np.float32)))
        pos_dev.fill_(t)
        q_dev = ops.gqa_prologue(upload(q).to(torch.bfloat16), upload(k).to(torch.bfloat16), upload(v).to(torch.bfloat16), upload(qw),
                                 upload(kw), upload(cos), upload(sin), dev["k"], dev_s["k"], dev["v"], dev_s["v"], table, 0, hq, hkv,
                                 d, d, bt, eps=eps, q_out_dtype=torch.bfloat16, positions=pos_dev)
        want_q = cpu_chain(q, hq, d, qw, eps, 1.0, d, t, cos, sin, True)
        keys.append(cpu_chain(k, hkv, d, kw, eps, 1.0, d, t, cos, sin, True))
        values.append(v)
        assert np.array_equal(q_dev.view(torch.int16).cpu().numpy().view(np.uint16), O.f32_to_bf16(want_q))
    out = ops.gqa_decode(q_dev, dev["k"], dev_s["k"], dev["v"], dev_s["v"], table[None, :].contiguous(),
                         upload(np.array([steps], dtype=np.uint32)), hq, hkv, d, bt, 1.0 / np.sqrt(d), steps)
    torch.cuda.synchronize()
    # oracle on the dequantised pages (what the cache really holds)
    ref_codes = {n: np.zeros((pool_rows, hkv * d), dtype=np.int8) for n in ("k", "v")}
    ref_scales = {n: np.zeros((pool_rows, hkv * d // 64), dtype=np.uint16) for n in ("k", "v")}
    O.q8g64_append_paged(O.RULE_METAL_GQA, np.concatenate(keys), ref_codes["k"], ref_scales["k"], tables[0], 0, bt)
    O.q8g64_append_paged(O.RULE_METAL_GQA, np.concatenate(values), ref_codes["v"], ref_scales["v"], tables[0], 0, bt)
    assert np.array_equal(dev["k"].cpu().numpy(), ref_codes["k"]) and np.array_equal(dev["v"].cpu().numpy(), ref_codes["v"])
    kd = O.gather_dequant_rows(O.FMT_Q8, ref_codes["k"], ref_scales["k"], O.SCALE_F16, tables[0], bt, 0, steps, hkv * d)
    vd = O.gather_dequant_rows(O.FMT_Q8, ref_codes["v"], ref_scales["v"], O.SCALE_F16, tables[0], bt, 0, steps, hkv * d)
    q_last = O.bf16_to_f32(O.f32_to_bf16(want_q))
    rc, want = O.gqa_prefill_at_visible(q_last, kd, vd, 0, steps, steps - 1, hq, hkv, d, score_scale=1.0 / np.sqrt(d))
    assert rc == 0
    assert_attention_close(out.cpu().numpy(), want, "prologue + decode")


def test_prologue_rejects_bad_shapes():
    from zllm_amd import capi, ops

    z = torch.zeros((1, 128), device="cuda")
    planes = torch.zeros((16, 128), dtype=torch.int8, device="cuda")
    scales = torch.zeros((16, 2), dtype=torch.int16, device="cuda")
    cos = torch.zeros((1, 32), device="cuda")
    with pytest.raises(capi.ZllmAttnError, match="RoPE table"):
        ops.gqa_prologue(z, z, z, None, None, cos, cos, planes, scales, planes, scales, None, 5, 1, 1, 128, 64, 16)
    with pytest.raises(capi.ZllmAttnError, match="rotary_dim"):
        ops.gqa_prologue(z, z, z, None, None, cos, cos, planes, scales, planes, scales, None, 0, 1, 1, 128, 63, 16)
    with pytest.raises(capi.ZllmAttnError, match="eps"):
        ops.gqa_prologue(z, z, z, z[0], None, cos, cos, planes, scales, planes, scales, None, 0, 1, 1, 128, 64, 16, eps=0.0)

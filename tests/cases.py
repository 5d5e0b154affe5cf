"""Seeded synthetic cases shared by the parity tests (NumPy on the host side; the oracle quantizes)."""
from __future__ import annotations

import numpy as np

import oracle as O

ATOL = 2e-3  # max-abs bound on attention outputs (north-star tolerance)
RTOL = 1e-2  # relative bound, measured on the whole output vector


def assert_attention_close(actual, expected, what="", atol=ATOL, rtol=RTOL):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    assert actual.shape == expected.shape, (actual.shape, expected.shape)
    assert np.isfinite(actual).all(), f"{what}: non-finite output"
    err = np.abs(actual - expected)
    max_abs = err.max() if err.size else 0.0
    denom = np.linalg.norm(expected)
    rel = np.linalg.norm(actual - expected) / denom if denom > 0 else np.linalg.norm(actual - expected)
    assert max_abs <= atol, f"{what}: max-abs {max_abs:.3e} > {atol}"
    assert rel <= rtol, f"{what}: relative {rel:.3e} > {rtol}"
    return max_abs, rel


def draw_tables(rng, lens, block_tokens, pool_blocks=None, layout="random"):
    """Block tables [B, max_blocks] over a shared pool; blocks drawn without replacement."""
    need = [(int(l) + block_tokens - 1) // block_tokens for l in lens]
    total = sum(need)
    pool_blocks = pool_blocks or total + 7
    assert pool_blocks >= total
    if layout == "identity":
        ids = np.arange(total, dtype=np.uint32)
    elif layout == "reversed":
        ids = np.arange(total, dtype=np.uint32)[::-1].copy()
    else:
        ids = rng.permutation(pool_blocks)[:total].astype(np.uint32)
    stride = max(max(need), 1)
    tables = np.zeros((len(lens), stride), dtype=np.uint32)
    at = 0
    for b, n in enumerate(need):
        tables[b, :n] = ids[at:at + n]
        at += n
    return tables, pool_blocks


def make_gqa_q8_case(seed, lens, hq, hkv, d, block_tokens=16, rule=O.RULE_METAL_GQA, outliers=False, layout="random",
                     q_bf16=False, pool_blocks=None, q_std=1.0, k_gain=1.0, v_gain=1.0, poison=False, ring_capacity=0):
    """K/V ~ N(0,1) (optionally 1 % outlier channels x8), quantized Q8g64 by the oracle into a paged pool.
    k_gain / v_gain: one factor, or one per token of the longest sequence (magnitude tests).
    poison: rows no sequence wrote hold NaN scale bits and the code -128 (a pool that was never cleared).
    ring_capacity: sliding-window storage, token t lives in slot t % ring_capacity of the sequence's pages."""
    rng = np.random.default_rng(seed)
    lens = [int(l) for l in lens]
    cols = hkv * d
    stored = [min(l, ring_capacity) if ring_capacity else l for l in lens]
    tables, pool_blocks = draw_tables(rng, stored, block_tokens, pool_blocks, layout)
    rows = pool_blocks * block_tokens
    sdt = {O.RULE_ROCM_MLA: O.SCALE_BF16, O.RULE_METAL_GQA: O.SCALE_F16, O.RULE_CUDA_GQA: O.SCALE_F32}[rule]
    scale_np = np.float32 if sdt == O.SCALE_F32 else np.uint16
    planes = {
        "k_codes": np.zeros((rows, cols), dtype=np.int8),
        "k_scales": np.zeros((rows, cols // 64), dtype=scale_np),
        "v_codes": np.zeros((rows, cols), dtype=np.int8),
        "v_scales": np.zeros((rows, cols // 64), dtype=scale_np),
    }
    if poison:
        for name in ("k_codes", "v_codes"):
            planes[name][:] = -128
        for name in ("k_scales", "v_scales"):
            planes[name][:] = np.nan if sdt == O.SCALE_F32 else (0x7FC0 if sdt == O.SCALE_BF16 else 0x7E00)
    raw_k, raw_v = [], []
    channel_gain = np.ones(cols, dtype=np.float32)
    if outliers:
        picks = rng.choice(cols, size=max(1, cols // 100), replace=False)
        channel_gain[picks] = 8.0
    for b, length in enumerate(lens):
        kg = np.reshape(np.asarray(k_gain, dtype=np.float32), (-1, 1))
        vg = np.reshape(np.asarray(v_gain, dtype=np.float32), (-1, 1))
        k = rng.standard_normal((length, cols)).astype(np.float32) * channel_gain * (kg if kg.shape[0] == 1 else kg[:length])
        v = rng.standard_normal((length, cols)).astype(np.float32) * channel_gain * (vg if vg.shape[0] == 1 else vg[:length])
        raw_k.append(k)
        raw_v.append(v)
        if length:
            O.q8g64_append_paged(rule, k, planes["k_codes"], planes["k_scales"], tables[b], 0, block_tokens, ring_capacity=ring_capacity)
            O.q8g64_append_paged(rule, v, planes["v_codes"], planes["v_scales"], tables[b], 0, block_tokens, ring_capacity=ring_capacity)
    q = (rng.standard_normal((len(lens), hq * d)) * q_std).astype(np.float32)
    q_bits = None
    if q_bf16:
        q_bits = O.f32_to_bf16(q)
        q = O.bf16_to_f32(q_bits)
    return dict(q=q, q_bits=q_bits, lens=np.array(lens, dtype=np.uint32), tables=tables, planes=planes, raw_k=raw_k,
                raw_v=raw_v, hq=hq, hkv=hkv, d=d, block_tokens=block_tokens, scale_dtype=sdt, rule=rule, rows=rows)


def oracle_gqa_decode(case, score_scale, window=0, softcap=0.0, fmt=None, ring_capacity=0):
    """Loop the single-sequence CPU oracle over the batch: gather + dequantize, then O3 for the last row."""
    fmt = O.FMT_Q8 if fmt is None else fmt
    hq, hkv, d = case["hq"], case["hkv"], case["d"]
    cols = hkv * d
    out = np.zeros((len(case["lens"]), hq * d), dtype=np.float32)
    for b, length in enumerate(case["lens"]):
        length = int(length)
        if length == 0:
            continue
        start, end = O.key_range(window, length - 1, length)
        if fmt == O.FMT_Q8:
            k = O.gather_dequant_rows(fmt, case["planes"]["k_codes"], case["planes"]["k_scales"], case["scale_dtype"],
                                      case["tables"][b], case["block_tokens"], start, end - start, cols,
                                      ring_capacity=ring_capacity)
            v = O.gather_dequant_rows(fmt, case["planes"]["v_codes"], case["planes"]["v_scales"], case["scale_dtype"],
                                      case["tables"][b], case["block_tokens"], start, end - start, cols,
                                      ring_capacity=ring_capacity)
        else:
            k = O.gather_dequant_rows(fmt, case["planes"]["k"], None, 0, case["tables"][b], case["block_tokens"], start,
                                      end - start, cols, ring_capacity=ring_capacity)
            v = O.gather_dequant_rows(fmt, case["planes"]["v"], None, 0, case["tables"][b], case["block_tokens"], start,
                                      end - start, cols, ring_capacity=ring_capacity)
        rc, o = O.gqa_prefill_at_visible(case["q"][b:b + 1], k, v, start, end, length - 1, hq, hkv, d, window=window,
                                         score_scale=score_scale, softcap=softcap)
        assert rc == 0
        out[b] = o[0]
    return out


def to_torch_bf16(bits, device):
    import torch

    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(device).view(torch.bfloat16)


def upload(array, device="cuda"):
    import torch

    a = np.ascontiguousarray(array)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(device)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to(device)
    return torch.from_numpy(a).to(device)

"""Writes the golden fixtures of this directory: small seeded inputs of the attention path and the outputs the
CPU oracle computes for them (run from the repo root: `python tests/golden/make_fixtures.py`).

The fixtures are data only.  They freeze the oracle's numbers at the time the oracle was pinned against the
reference's known-answer tests (tests/test_oracle_known_answers.py), so that a later change of the oracle or of a
kernel shows up as a difference against committed bytes:
  q8g64_quantizer.npz   128 rows x 256 columns in three magnitude regimes -> codes and scales of the three rules
  gqa_decode_small.npz  B=3 ragged, 8q/2kv, d=128, 16-token pages -> decode output
  mla_decode_small.npz  B=2, 4 heads, latent 512 + rope 64 -> output before the final bf16 rounding, dense and with a
                        32-entry token selection per sequence
  gqa_prologue_small.npz 5 rows, 4q/2kv, d=128: per-head Gemma RMSNorm + split-half RoPE of Q and K, K/V quantized into pages
  gqa_prefill_small.npz prefix 200 + chunk 48, 8q/2kv, window 0 and 64 -> chunk outputs
  block_attention_small.npz 40 query rows over 100 KV rows, 8q/2kv, d=128: varlen segments (offsets Q [0, 7, 8, 40], KV [0, 50,
                        51, 100]) and free per-row ranges -> outputs of the block attention with explicit ranges
  mla_other_widths_small.npz B=2, 3 heads, latent 128 + rope 32, nope 64 / value 64, kv_b as W8A16 codes (groups of 64, bf16
                        scales) -> output before the final bf16 rounding
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle as O  # noqa: E402
from tests.cases import make_gqa_q8_case, oracle_gqa_decode  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def quantizer():
    rng = np.random.default_rng(100)
    x = rng.standard_normal((128, 256)).astype(np.float32)
    x[32:64] *= 1e-3
    x[64:96] *= 300.0
    x[96] = 0.0
    x[97, :64] = np.float32(127.0)
    out = {"input": x}
    table = np.arange(8, dtype=np.uint32)
    for name, rule, dtype in (("rocm_mla", O.RULE_ROCM_MLA, np.uint16), ("metal_gqa", O.RULE_METAL_GQA, np.uint16),
                              ("cuda_gqa", O.RULE_CUDA_GQA, np.float32)):
        codes = np.zeros((128, 256), dtype=np.int8)
        scales = np.zeros((128, 4), dtype=dtype)
        O.q8g64_append_paged(rule, x, codes, scales, table, 0, 16)
        out[name + "_codes"] = codes
        out[name + "_scales"] = scales
    np.savez_compressed(os.path.join(HERE, "q8g64_quantizer.npz"), **out)


def gqa_decode():
    case = make_gqa_q8_case(501, [130, 77, 300], 8, 2, 128, outliers=True, q_bf16=True)
    want = oracle_gqa_decode(case, 0.09)
    np.savez_compressed(os.path.join(HERE, "gqa_decode_small.npz"), q_bits=case["q_bits"], lens=case["lens"], tables=case["tables"],
                        score_scale=np.float32(0.09), expected=want, **case["planes"])


def mla_decode():
    from tests.test_gpu_mla_decode import make_mla_case, oracle_mla

    case = make_mla_case(502, [150, 41], 4)
    want, want_bf16 = oracle_mla(case)
    rng = np.random.default_rng(504)
    selection = np.stack([rng.choice(int(l), size=32, replace=False) for l in case["lens"]]).astype(np.uint32)
    selected, _ = oracle_mla(case, selection=selection)
    np.savez_compressed(os.path.join(HERE, "mla_decode_small.npz"), q_bits=case["q_bits"], kv_b_bits=case["kv_b_bits"], codes=case["codes"],
                        scales=case["scales"], rope=case["rope"], tables=case["tables"], lens=case["lens"], expected_f32=want,
                        expected_bf16=want_bf16, selection=selection, expected_selected_f32=selected)


def gqa_prologue():
    rng = np.random.default_rng(505)
    rows, hq, hkv, d, bt, position, rotary, eps = 5, 4, 2, 128, 16, 11, 64, 1e-6
    q = rng.standard_normal((rows, hq * d)).astype(np.float32) * 2
    k = rng.standard_normal((rows, hkv * d)).astype(np.float32)
    v = rng.standard_normal((rows, hkv * d)).astype(np.float32)
    qw = (rng.standard_normal(d) * 0.2).astype(np.float32)
    kw = (rng.standard_normal(d) * 0.2).astype(np.float32)
    half = rotary // 2
    angles = np.arange(position + rows, dtype=np.float64)[:, None] / 10000.0 ** (np.arange(half, dtype=np.float64)[None, :] / half)
    cos, sin = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
    table = rng.permutation(4)[:2].astype(np.uint32)
    out = {}
    for name, x, heads, w in (("q", q, hq, qw), ("k", k, hkv, kw)):
        rc, normed = O.rmsnorm_heads(x, heads, d, w, eps, 1.0)
        assert rc == 0
        rc, rotated = O.rope_apply(normed, heads, rotary, position, cos, sin, layout=0, placement=0)
        assert rc == 0
        out[name] = rotated
    planes = {n: np.zeros((4 * bt, hkv * d if "codes" in n else hkv * d // 64), dtype=np.int8 if "codes" in n else np.uint16)
              for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
    O.q8g64_append_paged(O.RULE_METAL_GQA, out["k"], planes["k_codes"], planes["k_scales"], table, position, bt)
    O.q8g64_append_paged(O.RULE_METAL_GQA, v, planes["v_codes"], planes["v_scales"], table, position, bt)
    np.savez_compressed(os.path.join(HERE, "gqa_prologue_small.npz"), q=q, k=k, v=v, q_norm=qw, k_norm=kw, cos=cos, sin=sin, table=table,
                        position=np.uint32(position), rotary=np.uint32(rotary), eps=np.float32(eps), expected_q=out["q"], **planes)


def gqa_prefill():
    rng = np.random.default_rng(503)
    hq, hkv, d, bt, prefix, chunk = 8, 2, 128, 16, 200, 48
    cols = hkv * d
    total = prefix + chunk
    table = rng.permutation(20)[: (total + bt - 1) // bt].astype(np.uint32)
    rows = 20 * bt
    planes = {n: np.zeros((rows, cols if "codes" in n else cols // 64), dtype=np.int8 if "codes" in n else np.uint16)
              for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
    k = rng.standard_normal((total, cols)).astype(np.float32)
    v = rng.standard_normal((total, cols)).astype(np.float32)
    O.q8g64_append_paged(O.RULE_METAL_GQA, k, planes["k_codes"], planes["k_scales"], table, 0, bt)
    O.q8g64_append_paged(O.RULE_METAL_GQA, v, planes["v_codes"], planes["v_scales"], table, 0, bt)
    q_bits = O.f32_to_bf16(rng.standard_normal((chunk, hq * d)).astype(np.float32))
    q = O.bf16_to_f32(q_bits)
    kd = O.gather_dequant_rows(O.FMT_Q8, planes["k_codes"], planes["k_scales"], O.SCALE_F16, table, bt, 0, total, cols)
    vd = O.gather_dequant_rows(O.FMT_Q8, planes["v_codes"], planes["v_scales"], O.SCALE_F16, table, bt, 0, total, cols)
    out = {}
    for window in (0, 64):
        rc, want = O.gqa_prefill_at_visible(q, kd, vd, 0, total, prefix, hq, hkv, d, window=window, score_scale=0.0884)
        assert rc == 0
        out[f"expected_window_{window}"] = want
    np.savez_compressed(os.path.join(HERE, "gqa_prefill_small.npz"), q_bits=q_bits, table=table, prefix=np.uint32(prefix),
                        score_scale=np.float32(0.0884), **planes, **out)


def block_attention():
    rng = np.random.default_rng(507)
    hq, hkv, d, bt, q_rows, kv_rows = 8, 2, 128, 16, 40, 100
    cols = hkv * d
    table = rng.permutation(12)[: (kv_rows + bt - 1) // bt].astype(np.uint32)
    planes = {n: np.zeros((12 * bt, cols if "codes" in n else cols // 64), dtype=np.int8 if "codes" in n else np.uint16)
              for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
    k = rng.standard_normal((kv_rows, cols)).astype(np.float32)
    v = rng.standard_normal((kv_rows, cols)).astype(np.float32)
    O.q8g64_append_paged(O.RULE_METAL_GQA, k, planes["k_codes"], planes["k_scales"], table, 0, bt)
    O.q8g64_append_paged(O.RULE_METAL_GQA, v, planes["v_codes"], planes["v_scales"], table, 0, bt)
    q_bits = O.f32_to_bf16(rng.standard_normal((q_rows, hq * d)).astype(np.float32))
    kd = O.gather_dequant_rows(O.FMT_Q8, planes["k_codes"], planes["k_scales"], O.SCALE_F16, table, bt, 0, kv_rows, cols)
    vd = O.gather_dequant_rows(O.FMT_Q8, planes["v_codes"], planes["v_scales"], O.SCALE_F16, table, bt, 0, kv_rows, cols)
    varlen = np.array([(0, 50)] * 7 + [(50, 51)] + [(51, 100)] * 32, dtype=np.uint32)
    starts = rng.integers(0, kv_rows, size=q_rows)
    free = np.stack([starts, starts + 1 + (rng.integers(0, kv_rows, size=q_rows) % (kv_rows - starts))], axis=1).astype(np.uint32)
    out = {}
    for name, visible in (("varlen", varlen), ("free", free)):
        rc, want = O.block_attention(O.bf16_to_f32(q_bits), kd, vd, hq, hkv, d, 0.0884, visible)
        assert rc == 0
        out[f"visible_{name}"] = visible
        out[f"expected_{name}"] = want
    np.savez_compressed(os.path.join(HERE, "block_attention_small.npz"), q_bits=q_bits, table=table, score_scale=np.float32(0.0884), **planes, **out)


def mla_other_widths():
    from tests.test_gpu_mla_decode import make_mla_case, oracle_mla, set_weight_form

    case = make_mla_case(509, [70, 33], 3, nope=64, rope=32, value=64, latent=128)
    set_weight_form(case, 8, group=64, scale_dtype=O.SCALE_BF16)
    want, _ = oracle_mla(case)
    form = case["kv_b_form"]
    np.savez_compressed(os.path.join(HERE, "mla_other_widths_small.npz"), q_bits=case["q_bits"], kv_b_words=form["data"], kv_b_scales=form["scales"],
                        kv_b_values=case["kv_b_f32"], codes=case["codes"], scales=case["scales"], rope=case["rope"], tables=case["tables"],
                        lens=case["lens"], expected_f32=want)


if __name__ == "__main__":
    block_attention()
    mla_other_widths()
    quantizer()
    gqa_decode()
    mla_decode()
    gqa_prefill()
    gqa_prologue()
    for name in sorted(os.listdir(HERE)):
        if name.endswith(".npz"):
            print(name, os.path.getsize(os.path.join(HERE, name)))

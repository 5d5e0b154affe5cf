"""Pins the CPU oracle against the known-answer tests the reference itself holds.

Every case below is a closed-form vector transcribed (as data: inputs and expected
outputs) from a `#[test]` in the reference; the citation names the test.
"""
import numpy as np
import pytest


def bf16(o, values):
    return o.f32_to_bf16(np.asarray(values, dtype=np.float32))


# ---- src/attention/gqa.rs:327-340 -------------------------------------------------------------
def test_key_range_known_answers(oracle):
    assert oracle.key_range(3, 4, 5) == (2, 5)
    assert oracle.key_range(3, 1, 2) == (0, 2)
    assert oracle.key_range(0, 4, 5) == (0, 5)
    assert oracle.key_range_with_visible_end(4, 2, 6, 5) == (0, 5)


def test_reference_prefill_is_causal(oracle):
    rc, out = oracle.gqa_prefill_at_visible([0.0, 0.0], [0.0, 0.0], [2.0, 6.0], 0, 2, 0, 1, 1, 1)
    assert rc == 0 and out.ravel().tolist() == [2.0, 4.0]


# ---- src/kernel/cpu/gqa.rs:33-69 --------------------------------------------------------------
def test_append_prefill_reads_prefix_values(oracle):
    rc, out = oracle.gqa_prefill_at_visible([0.0], [0.0, 0.0], [2.0, 6.0], 0, 2, 1, 1, 1, 1)
    assert rc == 0 and out.ravel().tolist() == [4.0]


def test_sliding_window_discards_old_values(oracle):
    rc, out = oracle.gqa_prefill_at_visible([0.0] * 3, [0.0] * 3, [2.0, 6.0, 10.0], 0, 3, 0, 1, 1, 1, window=2)
    assert rc == 0 and out.ravel().tolist() == [2.0, 4.0, 8.0]


def test_visual_block_reads_future_values(oracle):
    rc, out = oracle.gqa_prefill_at_visible([0.0] * 3, [0.0] * 3, [2.0, 6.0, 10.0], 0, 3, 0, 1, 1, 1, window=8,
                                            visible_ends=[3, 3, 3])
    assert rc == 0 and out.ravel().tolist() == [6.0, 6.0, 6.0]


# ---- src/attention/block.rs:125-141 -----------------------------------------------------------
def test_block_attention_known_answers(oracle):
    # varlen(3, 5, [0,2,3], [0,3,5]) expands to visible = [0..3, 0..3, 3..5]
    rc, out = oracle.block_attention([0.0] * 3, [0.0] * 5, [2.0, 4.0, 6.0, 20.0, 40.0], 1, 1, 1, 1.0,
                                     [0, 3, 0, 3, 3, 5])
    assert rc == 0 and out.ravel().tolist() == [4.0, 4.0, 30.0]
    rc, out = oracle.block_attention([0.0, 0.0], [0.0] * 3, [2.0, 6.0, 10.0], 1, 1, 1, 1.0, [0, 2, 1, 3])
    assert rc == 0 and out.ravel().tolist() == [4.0, 8.0]
    # empty or out-of-range visible intervals are rejected (block.rs:31-35)
    assert oracle.block_attention([0.0], [0.0] * 3, [1.0] * 3, 1, 1, 1, 1.0, [2, 2])[0] == -1
    assert oracle.block_attention([0.0], [0.0] * 3, [1.0] * 3, 1, 1, 1, 1.0, [0, 4])[0] == -1


# ---- src/attention/mla.rs:189-194 -------------------------------------------------------------
def test_mla_reference_single_token_returns_value(oracle):
    spec = oracle.MlaSpec(2, 2, 4, 4, 1)
    rc, out = oracle.mla_reference_attention([1.0, 0.0, 1.0, 0.0], [1.0, 0.0, 2.0, 4.0], [1.0, 0.0], [0], spec)
    assert rc == 0 and out.tolist() == [2.0, 4.0, 0.0, 0.0]


# ---- src/kernel/cpu/mla.rs:1082-1099 (running mean over 320 rows, 1e-3) ------------------------
def test_mla_uniform_scores_running_mean(oracle):
    rows = 320
    spec = oracle.MlaSpec(1, 2, 4, 4, 1)
    kv = np.zeros((rows, 4), dtype=np.float32)
    kv[:, 2] = np.arange(rows)
    kv[:, 3] = 2.0 * np.arange(rows)
    rope = np.zeros((rows, 2), dtype=np.float32)
    for token in (0, 1, 17, 319):
        rc, out = oracle.mla_reference_attention(np.zeros(4), kv[: token + 1], rope, np.arange(token + 1), spec)
        assert rc == 0
        assert abs(out[0] - token * 0.5) < 1e-3 and abs(out[1] - token) < 1e-3


# ---- src/kernel/cpu/mla.rs:1101-1111 ----------------------------------------------------------
def test_selected_bf16_history_uses_absolute_chunk_positions(oracle):
    spec = oracle.MlaSpec(1, 2, 4, 4, 1)
    projected = bf16(oracle, [0, 0, 1, 10, 0, 0, 2, 20, 0, 0, 3, 30, 0, 0, 4, 40])
    rc, out = oracle.mla_selected_bf16_history(spec, bf16(oracle, [0.0] * 8), 2, 2, projected, bf16(oracle, [0.0] * 8),
                                               4, selection=[0, 2, 1, 3], width=2)
    assert rc == 0
    assert oracle.bf16_to_f32(out).tolist() == [2.0, 20.0, 3.0, 30.0]


# ---- src/kernel/cpu/mla.rs:1197-1205 (causal chunk; same semantics through the scalar arm) ----
def test_chunk_uses_absolute_causal_prefix(oracle):
    spec = oracle.MlaSpec(1, 2, 4, 4, 1)
    projected = bf16(oracle, [0, 0, 1, 10, 0, 0, 2, 20, 0, 0, 3, 30, 0, 0, 4, 40])
    rc, out = oracle.mla_selected_bf16_history(spec, bf16(oracle, [0.0] * 8), 2, 2, projected, bf16(oracle, [0.0] * 8), 4)
    assert rc == 0
    assert oracle.bf16_to_f32(out).tolist() == [2.0, 20.0, 2.5, 25.0]


# ---- src/kernel/cpu/mla.rs:1136-1164 (absorbed-Q8 == expanded KV within 0.02) -----------------
def test_absorbed_q8_history_matches_expanded_kv_small(oracle):
    spec = oracle.MlaSpec(3, 2, 8, 8, 2)
    query = bf16(oracle, [0.5, -0.25, 0, 0, 1.0, 0.5, 0, 0, -0.5, 0.75, 0, 0, 0.25, -1.0, 0, 0])
    latent_values = np.array([1, 2, -1, 2, -1, 1, -1, 1, 2, 1, -2, 1], dtype=np.float32)
    codes = latent_values.astype(np.int8).view(np.uint8)
    scales = np.full(4, bf16(oracle, [1.0])[0], dtype=np.uint16)
    rope = bf16(oracle, [0.0] * 8)
    kv_b = np.array([1, 0, 0, 0, 1, 0, 1, 0, 0, 0, 1, 1, 0, 1, 0, 0, 0, 1, 1, 0, 1, -1, 0, 1], dtype=np.float32)
    projected = (latent_values.reshape(4, 3) @ kv_b.reshape(8, 3).T).astype(np.float32)
    sel = [0, 2, 1, 3]
    rc, expected = oracle.mla_selected_bf16_history(spec, query, 2, 2, bf16(oracle, projected), rope, 4, sel, 2)
    assert rc == 0
    rc, actual, _, _ = oracle.mla_absorbed_q8_history(spec, query, 2, 2, codes, scales, 3, rope, 4, kv_b, sel, 2)
    assert rc == 0
    assert np.abs(oracle.bf16_to_f32(actual) - oracle.bf16_to_f32(expected)).max() < 0.02


# ---- src/kernel/cpu/mla.rs:1166-1195 (same, integer-pattern recipe at rank 64) -----------------
def test_absorbed_q8_matches_expanded_kv_rank64(oracle):
    spec = oracle.MlaSpec(64, 32, 128, 128, 2)
    q_vals = np.array([(i % 11 - 5) * 0.03125 for i in range(2 * 128)], dtype=np.float32)
    query = bf16(oracle, q_vals)
    codes_i = np.array([(i * 7 % 31) - 15 for i in range(4 * 64)], dtype=np.int8)
    scales = np.full(4, bf16(oracle, [0.0625])[0], dtype=np.uint16)
    rope = bf16(oracle, [(i % 9 - 4) * 0.015625 for i in range(4 * 32)])
    kv_b = np.array([(i * 13 % 17 - 8) * 0.0078125 for i in range(128 * 64)], dtype=np.float32)
    latent = codes_i.astype(np.float32) * 0.0625
    projected = (latent.reshape(4, 64) @ kv_b.reshape(128, 64).T).astype(np.float32)
    sel = [0, 2, 1, 3]
    rc, expected = oracle.mla_selected_bf16_history(spec, query, 2, 2, bf16(oracle, projected), rope, 4, sel, 2)
    assert rc == 0
    rc, actual, _, _ = oracle.mla_absorbed_q8_history(spec, query, 2, 2, codes_i.view(np.uint8), scales, 64, rope, 4,
                                                      kv_b, sel, 2)
    assert rc == 0
    assert np.abs(oracle.bf16_to_f32(actual) - oracle.bf16_to_f32(expected)).max() < 0.02


# ---- src/kv_cache/mod.rs:615-625, 667-675, 690-710 ---------------------------------------------
def test_bytes_per_token_known_answers(oracle):
    assert oracle.bytes_per_token(0, 8, 4, 4) == 20
    assert oracle.bytes_per_token(1, 2, 4, 4) == 24
    assert oracle.bytes_per_token(0, 8, 4, 3) == 0  # group must divide (mod.rs:653-658)
    assert oracle.bytes_per_token(0, 0, 4, 4) == 0 and oracle.bytes_per_token(0, 8, 0, 4) == 0
    # src/backend/rocm/kv_cache.rs:3617-3624: 512 + 16 + 128 = 656
    assert oracle.bytes_per_token(0, 512, 64, 64) == 656
    # benchmark configs: C1 1,056 B; C2/C5 2,112 B
    assert oracle.bytes_per_token(1, 4, 128, 64) == 1056
    assert oracle.bytes_per_token(1, 8, 128, 64) == 2112


def test_cache_layout_computes_mla_offsets(oracle):
    total, off = oracle.layout_offsets(0, 8, 4, 4, 2, 3, 1)
    assert total == 120 and off[1] == 60 and off[2] == 84 and off[3] == 96


def test_ring_plan_known_answer(oracle):
    assert oracle.lib().zo_cache_capacity(3, 10) == 3 and oracle.lib().zo_cache_capacity(0, 10) == 10
    plan = oracle.ring_write_plan(3, 10, 0, 5)
    assert (plan["source_start"], plan["first_slot"], plan["first_count"], plan["second_count"]) == (2, 2, 1, 2)
    assert oracle.ring_write_plan(3, 10, 0, 0) is None
    assert oracle.ring_write_plan(3, 10, 8, 5) is None


# ---- src/backend/rocm/mod.rs:855-861 (bf16 bit patterns) ---------------------------------------
def test_bf16_bit_patterns(oracle):
    assert oracle.f32_to_bf16(np.array([1.0, 2.0, -1.0, 0.0], dtype=np.float32)).tolist() == [0x3F80, 0x4000, 0xBF80, 0]
    lib = oracle.lib()
    for v, b in [(1.0, 0x3F80), (2.0, 0x4000), (-1.0, 0xBF80), (0.0, 0)]:
        assert lib.zo_f32_to_bf16(v) == b and lib.zo_bf16_to_f32(b) == v


# ---- src/attention/rope.rs:171-201 -------------------------------------------------------------
def test_rope_known_answers(oracle):
    rc, out = oracle.rope_apply([1.0, 2.0, 3.0, 4.0], 1, 4, 0, [0.0, 0.0], [1.0, 1.0], layout=0, placement=0)
    assert rc == 0 and out.ravel().tolist() == [-3.0, -4.0, 1.0, 2.0]
    rc, out = oracle.rope_apply([1.0, 2.0, 3.0, 4.0], 1, 4, 0, [0.0, 0.0], [1.0, 1.0], layout=1, placement=0)
    assert rc == 0 and out.ravel().tolist() == [-2.0, 1.0, -4.0, 3.0]
    rc, _ = oracle.rope_apply([0.0] * 4, 1, 4, 1, [1.0, 1.0], [0.0, 0.0], layout=0, placement=1)
    assert rc == -1


# ---- src/kernel/cuda/attention.rs:1704-1747 (quantizer round-trip bound, append at offset) -----
@pytest.mark.parametrize("rule,sdt", [(0, 0), (1, 1), (2, 2)])
def test_q8g64_roundtrip_error_bounded(oracle, rule, sdt):
    rows, cols = 64, 1024
    x = np.array([((i * 37) % 199) * 0.021 - 2.1 for i in range(rows * cols)], dtype=np.float32).reshape(rows, cols)
    codes = np.zeros((rows, cols), dtype=np.int8)
    scales = np.zeros((rows, cols // 64), dtype=np.float32 if sdt == 2 else np.uint16)
    oracle.q8g64_append_paged(rule, x, codes, scales, None, 0, 64)
    deq = oracle.gather_dequant_rows(oracle.FMT_Q8, codes, scales, sdt, None, 64, 0, rows, cols)
    s = {0: oracle.bf16_to_f32, 1: oracle.f16_to_f32, 2: lambda a: a}[sdt](scales)
    bound = np.repeat(s, 64, axis=1) / 2 + 1e-6
    if sdt != 2:
        # a rounded 16-bit scale may clip the absmax element: allow the scale's rounding step
        bound = bound + np.repeat(s, 64, axis=1) * 127 * (2.0 ** -8 if sdt == 0 else 2.0 ** -11)
    assert (np.abs(deq - x) <= bound).all()
    assert np.abs(codes).max() <= 127


def test_q8g64_appends_at_position_offset(oracle):
    rows, cols = 8, 1024
    first = np.array([((i * 37) % 199) * 0.02 - 1.0 for i in range(rows * cols)], dtype=np.float32).reshape(rows, cols)
    second = np.array([((i * 53) % 211) * 0.03 + 0.5 for i in range(rows * cols)], dtype=np.float32).reshape(rows, cols)
    codes = np.zeros((2 * rows, cols), dtype=np.int8)
    scales = np.zeros((2 * rows, cols // 64), dtype=np.float32)
    oracle.q8g64_append_paged(2, first, codes, scales, None, 0, 64)
    keep = codes[:rows].copy()
    oracle.q8g64_append_paged(2, second, codes, scales, None, rows, 64)
    assert (codes[:rows] == keep).all()
    deq = codes[rows:].astype(np.float32) * np.repeat(scales[rows:], 64, axis=1)
    assert (np.abs(deq - second) <= np.repeat(scales[rows:], 64, axis=1) / 2 + 1e-6).all()


# ---- src/kernel/cpu/rmsnorm.rs:70-86 (Gemma weight reads as 1 + gamma) -----------------------------
def test_rmsnorm_heads_gemma_weight_is_one_plus_gamma(oracle):
    x = np.arange(1, 9, dtype=np.float32)
    w = np.array([[0.0, 0.5, -0.5, 1.0][i % 4] for i in range(8)], dtype=np.float32)
    rc, plain = oracle.rmsnorm_heads(x[None, :], 1, 8, w, 1.0e-6, 0.0)
    assert rc == 0
    rc, gemma = oracle.rmsnorm_heads(x[None, :], 1, 8, w, 1.0e-6, 1.0)
    assert rc == 0
    inv = 1.0 / np.sqrt((x.astype(np.float64) ** 2).mean() + 1.0e-6)
    assert np.abs(plain.ravel() - x * inv * w).max() < 1.0e-6
    assert np.abs(gemma.ravel() - x * inv * (1.0 + w)).max() < 1.0e-6


# ---- src/kernel/cpu/rmsnorm.rs:88-103 (length that is not a multiple of eight: scalar tail) --------
def test_rmsnorm_heads_scalar_tail(oracle):
    x = np.arange(1, 12, dtype=np.float32)
    w = (0.5 + np.arange(11) * 0.1).astype(np.float32)
    inv = 1.0 / np.sqrt((x.astype(np.float64) ** 2).mean() + 1.0e-6)
    for offset in (0.0, 1.0):
        rc, out = oracle.rmsnorm_heads(x[None, :], 1, 11, w, 1.0e-6, offset)
        assert rc == 0
        assert np.abs(out.ravel() - x * inv * (offset + w)).max() < 1.0e-5

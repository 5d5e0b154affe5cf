"""Pins the oracle against what the mathematics fixes, independently of its own code:
float64 NumPy softmax attention, closed forms, invariants and by-construction vectors."""
import numpy as np
import pytest


def softmax_attention_f64(q, k, v, scale, softcap=0.0):
    """q [Hq,d], k/v [L,Hkv,d] -> [Hq,d] in float64 (plain library math)."""
    hq, d = q.shape
    hkv = k.shape[1]
    g = hq // hkv
    out = np.zeros((hq, d))
    for h in range(hq):
        s = (k[:, h // g, :].astype(np.float64) @ q[h].astype(np.float64)) * scale
        if softcap > 0:
            s = softcap * np.tanh(s / softcap)
        p = np.exp(s - s.max())
        out[h] = (p / p.sum()) @ v[:, h // g, :].astype(np.float64)
    return out


@pytest.mark.parametrize("hq,hkv,d,L", [(4, 4, 64, 97), (16, 4, 128, 300), (8, 1, 32, 33)])
def test_gqa_matches_float64_library_math(oracle, hq, hkv, d, L):
    rng = np.random.default_rng(hq * 1000 + L)
    q = rng.standard_normal((hq, d)).astype(np.float32)
    k = rng.standard_normal((L, hkv, d)).astype(np.float32)
    v = rng.standard_normal((L, hkv, d)).astype(np.float32)
    scale = 1.0 / np.sqrt(d)
    rc, out = oracle.gqa_prefill_at_visible(q.reshape(1, -1), k.reshape(L, -1), v.reshape(L, -1), 0, L, L - 1, hq, hkv,
                                            d, score_scale=scale)
    assert rc == 0
    ref = softmax_attention_f64(q, k, v, scale)
    assert np.abs(out.reshape(hq, d) - ref).max() < 2e-5


def test_gqa_zero_query_is_mean_and_dominant_key_selects_row(oracle):
    rng = np.random.default_rng(5)
    L, hq, hkv, d = 50, 4, 2, 64
    k = rng.standard_normal((L, hkv * d)).astype(np.float32)
    v = rng.standard_normal((L, hkv * d)).astype(np.float32)
    rc, out = oracle.gqa_prefill_at_visible(np.zeros((1, hq * d)), k, v, 0, L, L - 1, hq, hkv, d, score_scale=0.125)
    mean = v.reshape(L, hkv, d).mean(0)
    assert np.abs(out.reshape(hq, d) - np.repeat(mean, hq // hkv, axis=0)).max() < 1e-5
    # one key aligned with a large query: softmax collapses onto it
    q = np.zeros((hq, d), dtype=np.float32)
    q[:, 0] = 200.0
    k2 = np.zeros((L, hkv, d), dtype=np.float32)
    k2[17, :, 0] = 1.0
    rc, out = oracle.gqa_prefill_at_visible(q.reshape(1, -1), k2.reshape(L, -1), v, 0, L, L - 1, hq, hkv, d,
                                            score_scale=1.0)
    assert np.abs(out.reshape(hq, d) - np.repeat(v.reshape(L, hkv, d)[17], hq // hkv, axis=0)).max() < 1e-5


def test_gqa_sliding_window_equals_full_attention_on_tail(oracle):
    rng = np.random.default_rng(6)
    L, hq, hkv, d, w = 120, 4, 2, 32, 37
    q = rng.standard_normal((1, hq * d)).astype(np.float32)
    k = rng.standard_normal((L, hkv * d)).astype(np.float32)
    v = rng.standard_normal((L, hkv * d)).astype(np.float32)
    rc, win = oracle.gqa_prefill_at_visible(q, k, v, 0, L, L - 1, hq, hkv, d, window=w, score_scale=0.2)
    rc2, tail = oracle.gqa_prefill_at_visible(q, k[L - w:], v[L - w:], 0, w, w - 1, hq, hkv, d, score_scale=0.2)
    assert rc == 0 and rc2 == 0 and np.array_equal(win, tail)
    # window-evicted prefix: kv_start shifts the dense rows (cpu/attention.rs:517-548)
    rc3, shifted = oracle.gqa_prefill_at_visible(q, k[L - w:], v[L - w:], L - w, L, L - 1, hq, hkv, d, window=w,
                                                 score_scale=0.2)
    assert rc3 == 0 and np.array_equal(win, shifted)


def test_gqa_multi_row_chunk_is_causal(oracle):
    """Chunked prefill: row t of the chunk sees [0, position + t + 1)."""
    rng = np.random.default_rng(7)
    prefix, T, hq, hkv, d = 40, 9, 4, 2, 32
    L = prefix + T
    q = rng.standard_normal((T, hq, d)).astype(np.float32)
    k = rng.standard_normal((L, hkv, d)).astype(np.float32)
    v = rng.standard_normal((L, hkv, d)).astype(np.float32)
    rc, out = oracle.gqa_prefill_at_visible(q.reshape(T, -1), k.reshape(L, -1), v.reshape(L, -1), 0, L, prefix, hq,
                                            hkv, d, score_scale=0.25)
    assert rc == 0
    for t in range(T):
        ref = softmax_attention_f64(q[t], k[: prefix + t + 1], v[: prefix + t + 1], 0.25)
        assert np.abs(out[t].reshape(hq, d) - ref).max() < 2e-5


def test_softcap_definition(oracle):
    rng = np.random.default_rng(8)
    L, hq, hkv, d = 64, 2, 1, 16
    q = (rng.standard_normal((hq, d)) * 6).astype(np.float32)
    k = rng.standard_normal((L, hkv, d)).astype(np.float32)
    v = rng.standard_normal((L, hkv, d)).astype(np.float32)
    args = (q.reshape(1, -1), k.reshape(L, -1), v.reshape(L, -1), 0, L, L - 1, hq, hkv, d)
    _, capped = oracle.gqa_prefill_at_visible(*args, score_scale=0.5, softcap=5.0)
    assert np.abs(capped.reshape(hq, d) - softmax_attention_f64(q, k, v, 0.5, softcap=5.0)).max() < 2e-5
    _, plain = oracle.gqa_prefill_at_visible(*args, score_scale=0.5)
    _, huge = oracle.gqa_prefill_at_visible(*args, score_scale=0.5, softcap=1e9)
    assert np.abs(plain - huge).max() < 1e-5
    assert np.abs(plain - capped).max() > 1e-3  # the cap actually bites on these logits


def test_fully_masked_rows_are_zero_not_nan(oracle):
    q = np.ones((1, 4), dtype=np.float32)
    kv = np.ones((3, 4), dtype=np.float32)
    rc, out = oracle.gqa_prefill_at_visible(q, kv, kv, 0, 0, 0, 1, 1, 4)  # kv_end = 0 -> empty range
    assert rc == -2 and not np.isnan(out).any() and (out == 0).all()


# ---------------------------------------------------------------------------- quantizer
@pytest.mark.parametrize("rule,sdt", [(0, 0), (1, 1), (2, 2)])
def test_quantizer_by_construction(oracle, rule, sdt):
    """x = code * 2^-k with |code| reaching 127: the scale is exactly 2^-k in every storage
    dtype, so the codes must come back exactly."""
    rng = np.random.default_rng(11)
    codes_true = rng.integers(-127, 128, size=(5, 128)).astype(np.int8)
    codes_true[:, 0] = 127
    codes_true[:, 64] = -127
    scale_true = np.array([[2.0 ** -3, 2.0 ** -7]] * 5, dtype=np.float32)
    x = codes_true.astype(np.float32) * np.repeat(scale_true, 64, axis=1)
    codes = np.zeros_like(codes_true)
    scales = np.zeros((5, 2), dtype=np.float32 if sdt == 2 else np.uint16)
    oracle.q8g64_append_paged(rule, x, codes, scales, None, 0, 16)
    dec = {0: oracle.bf16_to_f32, 1: oracle.f16_to_f32, 2: lambda a: a}[sdt](scales)
    if rule == 0:
        assert np.array_equal(dec, scale_true)  # bf16(127*s*fl(1/127)) == s
    else:
        assert np.allclose(dec, scale_true, rtol=2e-7 if sdt == 2 else 1e-3)
    assert np.array_equal(codes, codes_true)


@pytest.mark.parametrize("rule,sdt", [(0, 0), (1, 1), (2, 2)])
def test_quantizer_invariants(oracle, rule, sdt):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((33, 256)).astype(np.float32)
    x[:, 5] *= 8  # outlier channel
    x[3, 64:128] = 0.0  # all-zero group
    codes = np.zeros(x.shape, dtype=np.int8)
    scales = np.zeros((33, 4), dtype=np.float32 if sdt == 2 else np.uint16)
    oracle.q8g64_append_paged(rule, x, codes, scales, None, 0, 16)
    dec = {0: oracle.bf16_to_f32, 1: oracle.f16_to_f32, 2: lambda a: a}[sdt](scales)
    assert dec[3, 1] == 1.0 and (codes[3, 64:128] == 0).all()
    xg = x.reshape(33, 4, 64)
    cg = codes.reshape(33, 4, 64)
    amax_idx = np.abs(xg).argmax(axis=2)
    picked = np.take_along_axis(cg, amax_idx[..., None], axis=2)[..., 0]
    nz = np.abs(xg).max(axis=2) > 0
    assert (np.abs(picked[nz]) >= 126).all()  # absmax element maps to +-127 (126 only via a scale rounded up)
    assert (np.sign(picked[nz]) == np.sign(np.take_along_axis(xg, amax_idx[..., None], axis=2)[..., 0][nz])).all()
    ideal = np.abs(xg).max(axis=2) / 127.0
    assert np.allclose(dec[nz], ideal[nz], rtol={0: 2.0 ** -8, 1: 2.0 ** -11, 2: 1e-6}[sdt])
    # rule 1/2 derive codes from the UNROUNDED scale: |x - code * ideal| <= ideal / 2
    if rule != 0:
        err = np.abs(xg - cg * ideal[..., None])
        assert (err <= ideal[..., None] / 2 * (1 + 1e-5) + 1e-9).all()
    else:
        err = np.abs(xg - cg * dec[..., None])
        inside = np.abs(xg) <= 127 * dec[..., None]
        assert (err[inside] <= dec[..., None].repeat(64, 2)[inside] / 2 * (1 + 1e-5)).all()


def test_rule0_uses_rounded_scale_rule1_does_not(oracle):
    """The two conventions differ observably: pick absmax so bf16(scale) rounds down by a lot."""
    x = np.zeros((1, 64), dtype=np.float32)
    x[0, 0] = 127.0 * 1.00389  # scale ~1.00389 -> bf16 rounds to 1.0
    x[0, 1] = 100.6
    c0 = np.zeros((1, 64), dtype=np.int8)
    s0 = np.zeros((1, 1), dtype=np.uint16)
    oracle.q8g64_append_paged(0, x, c0, s0, None, 0, 16)
    c1 = np.zeros((1, 64), dtype=np.int8)
    s1 = np.zeros((1, 1), dtype=np.uint16)
    oracle.q8g64_append_paged(1, x, c1, s1, None, 0, 16)
    assert oracle.bf16_to_f32(s0)[0, 0] == 1.0
    assert c0[0, 1] == 101 and c1[0, 1] == 100  # 100.6/1.0 -> 101 ; 100.6/1.00389 = 100.21 -> 100
    assert c0[0, 0] == 127 and c1[0, 0] == 127


# ---------------------------------------------------------------------------- paging
def test_paged_gather_invariants(oracle):
    rng = np.random.default_rng(13)
    B, nblk, cols = 16, 9, 32
    L = B * nblk - 5
    x = rng.standard_normal((L, cols)).astype(np.float32)
    perm = rng.permutation(nblk + 4).astype(np.uint32)[:nblk]
    pool_rows = (nblk + 4) * B
    codes_p = np.zeros((pool_rows, cols), dtype=np.int8)
    scales_p = np.zeros((pool_rows, cols // 16), dtype=np.uint16)
    oracle.q8g64_append_paged(1, x, codes_p, scales_p, perm, 0, B, group=16)
    codes_i = np.zeros((pool_rows, cols), dtype=np.int8)
    scales_i = np.zeros((pool_rows, cols // 16), dtype=np.uint16)
    oracle.q8g64_append_paged(1, x, codes_i, scales_i, None, 0, B, group=16)
    # closed form of paged_row, and identity table == no table (source.hip:52)
    for t in (0, 15, 16, 77, L - 1):
        assert oracle.paged_row(perm, t, B) == int(perm[t // B]) * B + t % B
        assert oracle.paged_row(None, t, B) == t
        assert oracle.paged_row(np.arange(nblk, dtype=np.uint32), t, B) == t
    got = oracle.gather_rows_bytes(codes_p, perm, B, 0, L, cols)
    assert np.array_equal(got, codes_i[:L].view(np.uint8))
    got_s = oracle.gather_rows_bytes(scales_p, perm, B, 0, L, cols // 16 * 2)
    assert np.array_equal(got_s, scales_i[:L].view(np.uint8).reshape(L, -1))
    # brute force: row by row through the closed form
    for t in range(L):
        phys = int(perm[t // B]) * B + t % B
        assert np.array_equal(codes_p[phys], codes_i[t])


def test_ring_addressing(oracle):
    """slot = token % capacity (cuda/attention.rs:82-88): the last `cap` tokens survive."""
    rng = np.random.default_rng(14)
    cap, cols, total = 8, 16, 21
    x = rng.standard_normal((total, cols)).astype(np.float32)
    cache = np.zeros((cap, cols), dtype=np.uint16)
    oracle.half_append_paged(1, x, cache, None, 0, 4, ring_capacity=cap)
    got = oracle.gather_dequant_rows(oracle.FMT_F16, cache, None, 0, None, 4, total - cap, cap, cols,
                                     ring_capacity=cap)
    assert np.array_equal(got, x[total - cap:].astype(np.float16).astype(np.float32))


# ---------------------------------------------------------------------------- MLA
def mla_absorbed_f64(spec, q, codes, scales, rope, kv_b):
    """Independent float64 evaluation of absorbed MLA == expanded MLA (one query row, causal over all rows)."""
    H, qh, nope = spec.num_heads, spec.q_head_dim, spec.nope
    kvh, vd, R = spec.kv_head_dim, spec.value_dim, spec.kv_lora_rank
    latent = codes.astype(np.float64) * np.repeat(scales.astype(np.float64), R // scales.shape[1], axis=1)
    W = kv_b.astype(np.float64).reshape(H, kvh, R)
    out = np.zeros((H, vd))
    for h in range(H):
        kv = latent @ W[h].T  # expanded [L, kvh]
        s = (kv[:, :nope] @ q[h, :nope] + rope.astype(np.float64) @ q[h, nope:]) / np.sqrt(qh)
        p = np.exp(s - s.max())
        out[h] = (p / p.sum()) @ kv[:, nope:]
    return out


def test_mla_absorbed_equals_expanded_float64(oracle):
    rng = np.random.default_rng(21)
    H, nope, rope_d, vd, R, L, g = 4, 32, 16, 24, 128, 70, 64
    spec = oracle.MlaSpec(R, rope_d, H * (nope + rope_d), H * (nope + vd), H)
    q = rng.standard_normal((H, nope + rope_d)).astype(np.float32)
    q_bits = oracle.f32_to_bf16(q)
    qf = oracle.bf16_to_f32(q_bits)
    latent = rng.standard_normal((L, R)).astype(np.float32)
    codes = np.zeros((L, R), dtype=np.int8)
    scales = np.zeros((L, R // g), dtype=np.uint16)
    oracle.q8g64_append_paged(0, latent, codes, scales, None, 0, 16, group=g)
    rope_bits = oracle.f32_to_bf16(rng.standard_normal((L, rope_d)).astype(np.float32))
    kv_b = (rng.standard_normal((H * (nope + vd), R)) / np.sqrt(R)).astype(np.float32)
    rc, out_b, out_f, weighted = oracle.mla_absorbed_q8_history(spec, q_bits.reshape(1, -1), 1, L - 1, codes, scales, g,
                                                                rope_bits, L, kv_b, want_weighted=True)
    assert rc == 0
    ref = mla_absorbed_f64(spec, qf, codes, oracle.bf16_to_f32(scales), oracle.bf16_to_f32(rope_bits), kv_b)
    # the only non-f32 step in O7 before the output is the bf16 rounding of the absorbed query (rel 2^-9)
    assert np.abs(out_f.reshape(H, vd) - ref).max() < 5e-3
    assert np.abs(oracle.bf16_to_f32(out_b) - out_f).max() <= np.abs(out_f).max() * 2.0 ** -8
    # and against the reference's own non-absorbed formulation O6 on the expanded KV
    lat_hat = codes.astype(np.float32) * np.repeat(oracle.bf16_to_f32(scales), g, axis=1)
    projected = lat_hat @ kv_b.T
    rc, o6 = oracle.mla_reference_attention(qf.reshape(-1), projected, oracle.bf16_to_f32(rope_bits), np.arange(L), spec)
    assert rc == 0
    o6 = o6.reshape(H, nope + rope_d)[:, :vd]
    assert np.abs(o6 - ref).max() < 1e-4
    assert np.abs(o6 - out_f.reshape(H, vd)).max() < 5e-3
    # weighted latent is a convex combination of dequantised rows
    assert weighted.reshape(H, R).max() <= lat_hat.max() + 1e-5


def test_mla_zero_query_gives_mean_latent_projection(oracle):
    rng = np.random.default_rng(22)
    H, nope, rope_d, vd, R, L = 2, 16, 8, 16, 64, 40
    spec = oracle.MlaSpec(R, rope_d, H * (nope + rope_d), H * (nope + vd), H)
    codes = rng.integers(-100, 100, size=(L, R)).astype(np.int8)
    scales = np.full((L, 1), oracle.f32_to_bf16(np.float32(0.03125)), dtype=np.uint16)
    rope_bits = oracle.f32_to_bf16(rng.standard_normal((L, rope_d)).astype(np.float32))
    kv_b = rng.standard_normal((H * (nope + vd), R)).astype(np.float32)
    rc, _, out_f, _ = oracle.mla_absorbed_q8_history(spec, np.zeros((1, spec.q_projection_size), np.uint16), 1, L - 1,
                                                     codes, scales, 64, rope_bits, L, kv_b)
    mean_latent = (codes.astype(np.float64) * 0.03125).mean(0)
    ref = np.stack([kv_b.reshape(H, nope + vd, R)[h, nope:] @ mean_latent for h in range(H)])
    assert rc == 0 and np.abs(out_f.reshape(H, vd) - ref).max() < 1e-3


def test_absorbed_q8_selection_equals_dense_attention_over_the_gathered_rows(oracle):
    """Attention over listed positions is attention over those rows laid out densely in list order: pins the
    `selected` arm of the absorbed-Q8 oracle (src/kernel/cpu/mla.rs:958-1076) against its dense arm."""
    rng = np.random.default_rng(11)
    heads, latent, rope, nope, value, rows, width = 3, 128, 16, 32, 24, 50, 9
    spec = oracle.MlaSpec(latent, rope, heads * (nope + rope), heads * (nope + value), heads)
    q = oracle.f32_to_bf16(rng.standard_normal((1, heads * (nope + rope))).astype(np.float32))
    codes = rng.integers(-127, 128, size=(rows, latent), dtype=np.int8)
    scales = oracle.f32_to_bf16((rng.random((rows, latent // 64)) * 0.05 + 0.01).astype(np.float32))
    rope_rows = oracle.f32_to_bf16(rng.standard_normal((rows, rope)).astype(np.float32))
    kv_b = oracle.bf16_to_f32(oracle.f32_to_bf16((rng.standard_normal((heads * (nope + value), latent)) / 8).astype(np.float32)))
    sel = rng.choice(rows, size=width, replace=False).astype(np.uint32)
    rc, _, picked, _ = oracle.mla_absorbed_q8_history(spec, q, 1, rows - 1, codes, scales, 64, rope_rows, rows, kv_b,
                                                      selection=sel, width=width)
    assert rc == 0
    rc, _, dense, _ = oracle.mla_absorbed_q8_history(spec, q, 1, width - 1, codes[sel], scales[sel], 64, rope_rows[sel], width, kv_b)
    assert rc == 0
    np.testing.assert_array_equal(picked, dense)
    # a position at or past the query row is rejected (mla.rs:965-975)
    bad = sel.copy()
    bad[0] = rows
    assert oracle.mla_absorbed_q8_history(spec, q, 1, rows - 1, codes, scales, 64, rope_rows, rows, kv_b, selection=bad, width=width)[0] != 0


def test_rmsnorm_heads_and_sigmoid_gate_against_float64(oracle):
    """Heads are normalised independently (a scaled copy of a head normalises to the same vector), every head of unit
    weight has mean square 1 - eps-ish, and the gate is the logistic function."""
    rng = np.random.default_rng(5)
    rows, heads, dim = 3, 4, 128
    x = rng.standard_normal((rows, heads * dim)).astype(np.float32)
    x[:, dim:2 * dim] = 7.5 * x[:, :dim]
    w = (rng.standard_normal(dim) * 0.1).astype(np.float32)
    rc, out = oracle.rmsnorm_heads(x, heads, dim, w, 1e-6, 1.0)
    assert rc == 0
    x64 = x.astype(np.float64).reshape(rows, heads, dim)
    want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * (1.0 + w.astype(np.float64))
    assert np.abs(out.reshape(rows, heads, dim) - want).max() < 2e-6
    assert np.abs(out[:, :dim] - out[:, dim:2 * dim]).max() < 5e-6  # eps is not scaled with the head
    gate = rng.standard_normal((rows, heads * dim)).astype(np.float32) * 4
    rc, gated = oracle.sigmoid_gate(out, gate)
    assert rc == 0
    assert np.abs(gated - out / (1.0 + np.exp(-gate.astype(np.float64)))).max() < 1e-6
    rc, per_row = oracle.sigmoid_gate(out, gate[:, :1])
    assert rc == 0
    assert np.abs(per_row - out / (1.0 + np.exp(-gate[:, :1].astype(np.float64)))).max() < 1e-6


def test_gqa_decode_direct_over_q8_equals_dequantise_then_f32(oracle):
    """The second CPU mode (values formed from the codes on the fly, src/kernel/cpu/mla.rs:771-829 style) against the
    pinned dequantise-then-f32 routine and against float64 NumPy: same products, so they agree to f32 summation order.
    A dropped scale, a wrong head offset or a shifted visible range would not."""
    rng = np.random.default_rng(17)
    for hq, hkv, d, length, first, sdt, rule, softcap in [(8, 2, 128, 300, 0, oracle.SCALE_F16, oracle.RULE_METAL_GQA, 0.0),
                                                          (4, 4, 64, 77, 13, oracle.SCALE_BF16, oracle.RULE_ROCM_MLA, 0.0),
                                                          (16, 8, 256, 150, 100, oracle.SCALE_F16, oracle.RULE_METAL_GQA, 50.0)]:
        cols = hkv * d
        k = rng.standard_normal((length, cols)).astype(np.float32)
        v = rng.standard_normal((length, cols)).astype(np.float32)
        planes = {n: np.zeros((length, cols if "codes" in n else cols // 64), dtype=np.int8 if "codes" in n else np.uint16)
                  for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
        oracle.q8g64_append_paged(rule, k, planes["k_codes"], planes["k_scales"], None, 0, 1)
        oracle.q8g64_append_paged(rule, v, planes["v_codes"], planes["v_scales"], None, 0, 1)
        q = rng.standard_normal(hq * d).astype(np.float32)
        scale = 1.0 / np.sqrt(d)
        rc, direct = oracle.gqa_decode_q8_direct(q, planes["k_codes"], planes["k_scales"], planes["v_codes"], planes["v_scales"], sdt, first,
                                                 length, hq, hkv, d, scale, softcap)
        assert rc == 0
        kd = oracle.gather_dequant_rows(oracle.FMT_Q8, planes["k_codes"], planes["k_scales"], sdt, None, 1, 0, length, cols)
        vd = oracle.gather_dequant_rows(oracle.FMT_Q8, planes["v_codes"], planes["v_scales"], sdt, None, 1, 0, length, cols)
        window = length - first if first else 0
        rc, two_step = oracle.gqa_prefill_at_visible(q[None, :], kd, vd, 0, length, length - 1, hq, hkv, d, window=window, score_scale=scale,
                                                     softcap=softcap)
        assert rc == 0
        np.testing.assert_allclose(direct, two_step[0], rtol=0, atol=2e-6)
        # float64, from the definition
        want = np.zeros(hq * d)
        for h in range(hq):
            kh = kd[first:, (h // (hq // hkv)) * d:(h // (hq // hkv) + 1) * d].astype(np.float64)
            vh = vd[first:, (h // (hq // hkv)) * d:(h // (hq // hkv) + 1) * d].astype(np.float64)
            s = kh @ q[h * d:(h + 1) * d].astype(np.float64) * scale
            if softcap:
                s = softcap * np.tanh(s / softcap)
            p = np.exp(s - s.max())
            want[h * d:(h + 1) * d] = (p / p.sum()) @ vh
        np.testing.assert_allclose(direct, want, rtol=0, atol=5e-6)

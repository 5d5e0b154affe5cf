"""Parity of absorbed MLA decode (absorb -> split-KV partial -> LSE merge -> project) with the CPU oracle
`mla_attention_absorbed_q8_history` (src/kernel/cpu/mla.rs:958-1076), through the C ABI.

The oracle's final result is bf16-rounded; the kernel's f32 output is compared with the oracle's value before that
rounding (max-abs 2e-3, relative 1e-2), and its bf16 output must be within one bf16 step of the oracle's bits.
"""
import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, draw_tables, to_torch_bf16, upload

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def make_mla_case(seed, lens, heads, nope=128, rope=64, value=128, latent=512, block_tokens=16, layout="random", w_std=None,
                  poison=False, latent_gain=1.0):
    rng = np.random.default_rng(seed)
    tables, pool_blocks = draw_tables(rng, lens, block_tokens, layout=layout)
    rows = pool_blocks * block_tokens
    codes = np.zeros((rows, latent), dtype=np.int8)
    scales = np.zeros((rows, latent // 64), dtype=np.uint16)
    rope_cache = np.zeros((rows, rope), dtype=np.uint16)
    if poison:  # rows no sequence has written yet: NaN scales and rope, extreme codes
        codes[:] = -128
        scales[:] = 0x7FC0
        rope_cache[:] = 0x7FC0
    for b, l in enumerate(lens):
        # latent_gain: one factor, or one per token of the longest sequence (magnitude tests)
        gain = np.reshape(np.asarray(latent_gain, dtype=np.float32), (-1, 1))
        lat = rng.standard_normal((l, latent)).astype(np.float32) * (gain if gain.shape[0] == 1 else gain[:l])
        kr = rng.standard_normal((l, rope)).astype(np.float32)
        O.q8g64_append_paged(O.RULE_ROCM_MLA, lat, codes, scales, tables[b], 0, block_tokens)
        O.half_append_paged(0, kr, rope_cache, tables[b], 0, block_tokens)
    q = rng.standard_normal((len(lens), heads * (nope + rope))).astype(np.float32)
    q_bits = O.f32_to_bf16(q)
    w_std = w_std if w_std is not None else 1.0 / np.sqrt(latent)
    kv_b_bits = O.f32_to_bf16((rng.standard_normal((heads * (nope + value), latent)) * w_std).astype(np.float32))
    spec = O.MlaSpec(latent, rope, heads * (nope + rope), heads * (nope + value), heads)
    return dict(q_bits=q_bits, kv_b_bits=kv_b_bits, codes=codes, scales=scales, rope=rope_cache, tables=tables,
                lens=np.array(lens, dtype=np.uint32), spec=spec, heads=heads, nope=nope, rope_dim=rope, value=value,
                latent=latent, block_tokens=block_tokens)


def weights_f32(case):
    """kv_b as the oracle takes it: the f32 values of whatever form the device reads (bf16 unless the case says otherwise)."""
    return case["kv_b_f32"] if "kv_b_f32" in case else O.bf16_to_f32(case["kv_b_bits"])


def weight_args(case):
    """(device tensor of kv_b, keyword arguments naming its form) for ops.mla_decode: bf16, or what set_weight_form left."""
    if "kv_b_form" not in case:
        return upload(case["kv_b_bits"]), {}
    form = case["kv_b_form"]
    kw = dict(kv_b_bits=form["bits"])
    if form["bits"] in (4, 8):
        kw.update(kv_b_scales=upload(form["scales"]), kv_b_group=form["group"], kv_b_scale_dtype=form["scale_dtype"])
    return upload(form["data"]), kw


def set_weight_form(case, bits, group=128, scale_dtype=O.SCALE_BF16):
    """Re-express the case's kv_b as f32 (bits 32) or as 8- / 4-bit codes with a scale per row and `group` columns, the
    W8A16 / W4A16 layout of paged_weight (src/kernel/rocm/hip/attention/paged_mla/source.hip:2-26): codes packed low
    bits first into 32-bit words, value = (code - 128 | code - 8) * scale.  The oracle gets the values the codes stand for."""
    w = O.bf16_to_f32(case["kv_b_bits"]).astype(np.float32)
    rows, cols = w.shape
    if bits == 32:
        rng = np.random.default_rng(rows + cols)
        w = (w * (1.0 + 1e-3 * rng.standard_normal(w.shape))).astype(np.float32)  # not bf16-representable any more
        case["kv_b_form"], case["kv_b_f32"] = dict(bits=32, data=w), w
        return case
    top = 127 if bits == 8 else 7
    grouped = w.reshape(rows, cols // group, group)
    scale = np.abs(grouped).max(axis=2) / top
    scale[scale == 0] = 1.0
    if scale_dtype == O.SCALE_BF16:
        stored = O.f32_to_bf16(scale.astype(np.float32))
        scale = O.bf16_to_f32(stored)
    elif scale_dtype == O.SCALE_F16:
        stored = scale.astype(np.float16).view(np.uint16)
        scale = stored.view(np.float16).astype(np.float32)
    else:
        stored = scale.astype(np.float32)
        scale = stored
    centred = np.clip(np.rint(grouped / scale[:, :, None]), -top - 1, top).astype(np.int32)
    codes = (centred + (128 if bits == 8 else 8)).astype(np.uint32).reshape(rows, cols)
    per_word = 32 // bits
    words = np.zeros((rows, cols // per_word), dtype=np.uint32)
    for i in range(per_word):
        words |= codes[:, i::per_word] << np.uint32(i * bits)
    case["kv_b_form"] = dict(bits=bits, data=words, scales=np.ascontiguousarray(stored), group=group, scale_dtype=scale_dtype)
    case["kv_b_f32"] = (centred.astype(np.float32) * scale[:, :, None].astype(np.float32)).reshape(rows, cols)
    return case


def oracle_mla(case, head_subset=None, selection=None, counts=None):
    """`selection` [batch, top_k]: the reference's rule (paged_mla/source.hip:4761-4764) -- a sequence longer than top_k
    attends to its first count listed positions, a shorter one stays dense."""
    spec, bt = case["spec"], case["block_tokens"]
    kv_b = weights_f32(case)
    outs_f, outs_b = [], []
    for b, l in enumerate(case["lens"]):
        l = int(l)
        codes = O.gather_rows_bytes(case["codes"], case["tables"][b], bt, 0, l, case["latent"])
        scales = O.gather_rows_bytes(case["scales"], case["tables"][b], bt, 0, l, case["latent"] // 64 * 2).view(np.uint16)
        rope = O.gather_rows_bytes(case["rope"], case["tables"][b], bt, 0, l, case["rope_dim"] * 2).view(np.uint16)
        sel, width = None, 0
        if selection is not None and selection.shape[1] < l:
            width = int(counts[b]) if counts is not None else selection.shape[1]
            sel = selection[b, :width]
        rc, ob, of, _ = O.mla_absorbed_q8_history(spec, case["q_bits"][b:b + 1], 1, l - 1, codes, scales, 64, rope, l, kv_b,
                                                  selection=sel, width=width)
        assert rc == 0
        outs_f.append(of)
        outs_b.append(ob)
    return np.stack(outs_f), np.stack(outs_b)


def run_mla(case, out_dtype=None, compact=True, q_f32=False, max_ctx_len=None, selection=None, counts=None, total_ctx_tokens=0,
            wide_tiles=False):
    from zllm_amd import ops

    out_dtype = out_dtype or torch.float32
    q = upload(O.bf16_to_f32(case["q_bits"])) if q_f32 else to_torch_bf16(case["q_bits"], "cuda")
    kv_b, weight_kw = weight_args(case)
    out = ops.mla_decode(q, kv_b, upload(case["codes"]), upload(case["scales"]), upload(case["rope"]),
                         upload(case["tables"]), upload(case["lens"]), case["heads"], case["nope"] + case["rope_dim"],
                         case["nope"] + case["value"], case["latent"], case["rope_dim"], case["block_tokens"],
                         max_ctx_len or int(case["lens"].max()), out_dtype=out_dtype, out_compact=compact,
                         selection=None if selection is None else upload(selection),
                         selection_counts=None if counts is None else upload(counts), total_ctx_tokens=total_ctx_tokens,
                         wide_tiles=wide_tiles, **weight_kw)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("heads,lens", [(128, [700, 2300]), (16, [100]), (64, [1025, 33]), (32, [1]),
                                        # one, two and three 32-token steps exactly and off by one; head counts that leave a
                                        # value wave with one live head tile (40 = 2.5 tiles) or a partial tile (20)
                                        (40, [31, 32, 33, 64, 65, 96]), (20, [5, 97])])
def test_mla_decode_matches_oracle(heads, lens):
    case = make_mla_case(heads + len(lens), lens, heads)
    want_f, want_b = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    print("mla", heads, lens, assert_attention_close(got, want_f, f"MLA heads={heads} lens={lens}"))


def test_mla_decode_config4_shape_at_oracle_size():
    """Benchmark config 4 geometry (B=4, 128 heads, latent 512 + rope 64, q_head 192, kv_head 256) at a context the
    scalar oracle finishes in seconds; the full 65,536-token case is covered by the split-invariance property below."""
    case = make_mla_case(4, [4096, 3000, 4096, 257], 128)
    want_f, want_b = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    print("config4-small", assert_attention_close(got, want_f, "config 4 (small)"))
    # bf16 output: within one bf16 step of the oracle's rounded bits
    got_b = run_mla(case, out_dtype=torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16)
    diff = np.abs(O.bf16_to_f32(got_b).astype(np.float64) - O.bf16_to_f32(want_b))
    step = np.maximum(np.abs(O.bf16_to_f32(want_b)), 2.0 ** -126) * 2.0 ** -7
    assert (diff <= step + 2e-3).all()


def test_mla_output_layouts_and_f32_query():
    case = make_mla_case(9, [500], 32)
    want_f, _ = oracle_mla(case)
    compact = run_mla(case).cpu().numpy()
    strided = run_mla(case, compact=False).cpu().numpy()  # row stride q_head_dim, only value_dim written (mla.rs:134)
    assert strided.shape == (1, 32 * 192)
    assert np.array_equal(strided.reshape(32, 192)[:, :128], compact.reshape(32, 128))
    assert (strided.reshape(32, 192)[:, 128:] == 0).all()
    f32q = run_mla(case, q_f32=True).cpu().numpy()
    assert np.array_equal(f32q, compact)  # the f32 query holds bf16-representable values
    assert_attention_close(compact, want_f, "layouts")


@pytest.mark.parametrize("block_tokens,layout", [(64, "identity"), (128, "reversed"), (1, "random"), (48, "random")])
def test_mla_page_sizes(block_tokens, layout):
    """The reference ships 64-token identity pages and tests a reversed table with 128-token pages
    (src/kernel/rocm/hip/attention/paged_mla.rs:6157-6222)."""
    case = make_mla_case(block_tokens, [900], 16, block_tokens=block_tokens, layout=layout)
    want_f, _ = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    assert_attention_close(got, want_f, f"block_tokens={block_tokens}")


@pytest.mark.parametrize("block_tokens", [32, 64, 16])
def test_mla_rows_past_the_end_of_a_page_are_ignored(block_tokens):
    """A sequence ends in the middle of a page; whatever the rest of the page holds (here NaN scales, NaN rope and
    the code -128) must not reach the result.  With pages of a multiple of 32 tokens the kernel loads whole
    32-row steps from a page, so the rows past the end are really read."""
    lens = [70, 1, 33, 96, 2049]
    case = make_mla_case(100 + block_tokens, lens, 32, block_tokens=block_tokens, poison=True)
    want_f, _ = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    assert np.isfinite(got).all()
    assert_attention_close(got, want_f, f"poisoned tail, block_tokens={block_tokens}")


@pytest.mark.parametrize("exponent", [30, -30, 12])
def test_mla_latent_magnitudes(exponent):
    """Latent rows far from unit magnitude (the kernel carries P' = p * scale as f16 inside an exponent window that follows
    the largest scale met so far), with kv_b scaled the other way so that scores and outputs keep their size."""
    heads, lens = 32, [900, 130]
    flat, w_std = float(2.0 ** exponent), float(2.0 ** -exponent) / np.sqrt(512)
    case = make_mla_case(300 + exponent, lens, heads, w_std=w_std, latent_gain=flat)
    want, _ = oracle_mla(case)
    print("uniform", assert_attention_close(run_mla(case).cpu().numpy(), want, f"latent * 2^{exponent}"))
    # rows of mixed magnitude: a large row also has large scores, so it takes the whole softmax when it is visible
    for name, rows in (("large first", slice(0, 20)), ("large last", slice(800, 900)), ("spike", slice(444, 445))):
        gain = np.full(max(lens), flat, dtype=np.float32)
        gain[rows] = flat * 64.0
        case = make_mla_case(310 + exponent, lens, heads, w_std=w_std, latent_gain=gain)
        want, _ = oracle_mla(case)
        top = float(np.abs(want).max())  # outputs are 64 times larger here: the absolute bound scales with them
        print(name, top, assert_attention_close(run_mla(case).cpu().numpy() / top, want / top, f"{name}, 2^{exponent}"))


def draw_selection(rng, lens, top_k, sort):
    """Per sequence: top_k distinct visible positions (repeats only when the context is shorter than top_k, where the
    list is ignored anyway)."""
    sel = np.zeros((len(lens), top_k), dtype=np.uint32)
    for b, l in enumerate(lens):
        picks = rng.choice(l, size=top_k, replace=l < top_k)
        sel[b] = np.sort(picks) if sort else picks
    return sel


@pytest.mark.parametrize("top_k,sort,block_tokens", [(200, False, 16), (2048, True, 64), (33, False, 1), (1, True, 16)])
def test_mla_selected_tokens(top_k, sort, block_tokens):
    """The `selection` arm (paged_mla.rs:3092-3105): sequences longer than top_k attend to the listed positions, in
    list order; shorter ones stay dense.  Lengths straddle top_k on purpose."""
    rng = np.random.default_rng(500 + top_k)
    lens = [max(top_k * 3, 40), top_k + 1, max(top_k // 2, 1), 2500]
    case = make_mla_case(600 + top_k, lens, 32, block_tokens=block_tokens, poison=True)
    sel = draw_selection(rng, lens, top_k, sort)
    want_f, _ = oracle_mla(case, selection=sel)
    got = run_mla(case, selection=sel).cpu().numpy()
    assert_attention_close(got, want_f, f"top_k={top_k}")
    dense_f, _ = oracle_mla(case)
    if top_k > 1:
        assert np.abs(want_f[0] - dense_f[0]).max() > 1e-3  # the list really changes the long sequences' result
    np.testing.assert_array_equal(np.abs(want_f[2] - dense_f[2]).max(), 0.0)  # and not the short one's


def test_mla_selected_tokens_with_counts_and_repeats():
    """selection_counts shortens a row's list; a position listed twice counts twice, as in the reference's loop over
    slots (src/kernel/cpu/mla.rs:582-686)."""
    rng = np.random.default_rng(77)
    lens = [1500, 700, 64]
    top_k = 256
    case = make_mla_case(78, lens, 16, block_tokens=16)
    sel = draw_selection(rng, lens, top_k, False)
    sel[0, 10:20] = sel[0, 0]  # repeats
    counts = np.array([256, 100, 256], dtype=np.uint32)
    want_f, _ = oracle_mla(case, selection=sel, counts=counts)
    got = run_mla(case, selection=sel, counts=counts).cpu().numpy()
    assert_attention_close(got, want_f, "counts + repeats")


def test_mla_split_invariance_and_zero_query():
    case = make_mla_case(11, [6000], 16)
    case["tables"] = np.pad(case["tables"], ((0, 0), (0, 40000 - case["tables"].shape[1])))
    a = run_mla(case, max_ctx_len=6000).cpu().numpy()
    b = run_mla(case, max_ctx_len=600000).cpu().numpy()
    assert np.abs(a - b).max() < 2e-4
    # zero query: uniform attention -> the projected mean latent
    case["q_bits"][:] = 0
    got = run_mla(case, max_ctx_len=6000).cpu().numpy().reshape(16, 128)
    lat = O.gather_dequant_rows(O.FMT_Q8, case["codes"], case["scales"], O.SCALE_BF16, case["tables"][0], 16, 0, 6000, 512)
    w = O.bf16_to_f32(case["kv_b_bits"]).reshape(16, 256, 512)[:, 128:, :]
    want = np.einsum("hvc,c->hv", w.astype(np.float64), lat.astype(np.float64).mean(0))
    assert np.abs(got - want).max() < 2e-3


@pytest.mark.parametrize("heads,ctx", [(64, 1357), (32, 768), (32, 2048), (32, 16384), (64, 16384)])
def test_mla_reference_split_test_recipe(heads, ctx):
    """Integer-pattern recipe of `mla_decode_split_matches_serial_and_reports_latency`
    (src/kernel/rocm/hip/attention/paged_mla.rs:6226-6342): q_head 256, kv_head 448, latent 512, rope 64, 64 heads and
    the 32 of a GPU's half, 128-token identity pages, scales 0x3b80, contexts from that test's list; checked against the
    CPU oracle at that test's 5e-3 bound.  (32 heads run the narrow layout of the partial kernel; 16,384 tokens are cut
    into a split per compute unit, merged by the wide merge; the value width of 256 takes the projection's general path.)"""
    q_head, kv_head, latent, rope, bt = 256, 448, 512, 64, 128
    q = np.array([((i % 257) - 128) / 256.0 for i in range(heads * q_head)], dtype=np.float32)
    weight = np.array([(((i * 17) % 127) - 63) / 4096.0 for i in range(heads * kv_head * latent)], dtype=np.float32)
    codes = np.array([((i * 29 + i // latent * 7) % 63 + 1) for i in range(ctx * latent)], dtype=np.uint8).view(np.int8)
    scales = np.full((ctx, latent // 64), 0x3B80, dtype=np.uint16)
    rope_vals = np.array([(((i * 13) % 127) - 63) / 128.0 for i in range(ctx * rope)], dtype=np.float32)
    table = np.arange((ctx + bt - 1) // bt, dtype=np.uint32)
    rows = len(table) * bt
    codes_p = np.zeros((rows, latent), dtype=np.int8)
    codes_p[:ctx] = codes.reshape(ctx, latent)
    scales_p = np.full((rows, latent // 64), 0x3B80, dtype=np.uint16)
    rope_p = np.zeros((rows, rope), dtype=np.uint16)
    rope_p[:ctx] = (rope_vals.view(np.uint32) >> 16).astype(np.uint16).reshape(ctx, rope)  # exact: values are bf16-representable
    q_bits = O.f32_to_bf16(q)
    w_bits = (weight.view(np.uint32) >> 16).astype(np.uint16)  # the test truncates; these values are exact in bf16
    spec = O.MlaSpec(latent, rope, heads * q_head, heads * kv_head, heads)
    case = dict(q_bits=q_bits.reshape(1, -1), kv_b_bits=w_bits.reshape(heads * kv_head, latent), codes=codes_p, scales=scales_p,
                rope=rope_p, tables=table.reshape(1, -1), lens=np.array([ctx], dtype=np.uint32), spec=spec, heads=heads,
                nope=q_head - rope, rope_dim=rope, value=kv_head - (q_head - rope), latent=latent, block_tokens=bt)
    want_f, _ = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    assert np.abs(got - want_f).max() <= 5e-3


def test_mla_layer_snapshot_round_trip_and_rollback():
    """Download a layer through its block table (gather), put it on the wire as the reference's MlaLayerSerde record,
    parse it, upload it into differently placed pages (scatter): decode over the restored cache is bit-identical.  Then
    rollback as truncate_layer_rows does it (src/backend/rocm/kv_cache.rs:509-586): only the logical length moves, and an
    append after it overwrites the tail."""
    import ctypes as C

    from oracle import wire
    from zllm_amd import capi, ops

    lens = [333]
    case = make_mla_case(901, lens, 16, block_tokens=16)
    bt, rows = 16, lens[0]
    dev = {n: upload(case[n]) for n in ("codes", "scales", "rope")}
    table = upload(case["tables"][0])
    row_bytes = {"codes": 512, "scales": 16, "rope": 128}
    host = {n: ops.gather_rows(dev[n].view(torch.uint8) if dev[n].dtype != torch.uint8 else dev[n], table, 0, rows, row_bytes[n], bt).cpu().numpy().tobytes()
            for n in dev}
    record = wire.MlaLayerSerde(rows, "Full", 512, 64, 64, host["codes"], host["scales"], host["rope"])
    lib = capi.load()
    keep = []
    rec = capi.MlaLayerRecord()
    rec.rows, rec.ownership, rec.latent_cols, rec.rope_cols, rec.latent_group_size = rows, 0, 512, 64, 64
    for name, field in (("codes", "latent"), ("scales", "latent_scales"), ("rope", "rope")):
        buf = (C.c_uint8 * len(host[name])).from_buffer_copy(host[name])
        keep.append(buf)
        setattr(rec, field, C.cast(buf, C.c_void_p))
        setattr(rec, field + "_bytes", len(host[name]))
    need = lib.zllm_kv_mla_layer_wire_bytes(C.byref(rec))
    out = (C.c_uint8 * need)()
    written = C.c_uint64(0)
    assert lib.zllm_kv_mla_layer_write(C.byref(rec), C.cast(out, C.c_void_p), need, C.byref(written)) == 0
    assert bytes(out) == wire.write_mla_layer(record)  # what the reference's reader would be handed
    parsed, used = capi.MlaLayerRecord(), C.c_uint64(0)
    assert lib.zllm_kv_mla_layer_read(C.cast(out, C.c_void_p), need, C.byref(parsed), C.byref(used)) == 0
    # restore into other pages
    rng = np.random.default_rng(902)
    tables2, pool_blocks2 = draw_tables(rng, lens, bt, layout="reversed")
    pool_rows2 = pool_blocks2 * bt
    restored = {"codes": torch.zeros((pool_rows2, 512), dtype=torch.uint8, device="cuda"),
                "scales": torch.zeros((pool_rows2, 16), dtype=torch.uint8, device="cuda"),
                "rope": torch.zeros((pool_rows2, 128), dtype=torch.uint8, device="cuda")}
    table2 = upload(tables2[0])
    for name, field in (("codes", "latent"), ("scales", "latent_scales"), ("rope", "rope")):
        blob = np.frombuffer(C.string_at(getattr(parsed, field), getattr(parsed, field + "_bytes")), dtype=np.uint8)
        ops.scatter_rows(restored[name], upload(blob.reshape(rows, row_bytes[name]).copy()), table2, 0, bt)
    before = run_mla(case).cpu().numpy()
    case2 = dict(case, codes=restored["codes"].view(torch.int8).cpu().numpy(), scales=restored["scales"].cpu().numpy().view(np.uint16),
                 rope=restored["rope"].cpu().numpy().view(np.uint16), tables=tables2)
    after = run_mla(case2).cpu().numpy()
    assert np.array_equal(before, after)
    # rollback to 300 rows, then append 10 other rows at position 300: the oracle over 310 rows must agree
    keep_rows, extra = 300, 10
    lat = rng.standard_normal((extra, 512)).astype(np.float32)
    kr = rng.standard_normal((extra, 64)).astype(np.float32)
    codes_t, scales_t, rope_t = (restored["codes"].view(torch.int8), restored["scales"].view(torch.int16), restored["rope"].view(torch.int16))
    ops.mla_append(upload(lat), upload(kr), codes_t, scales_t, rope_t, table2, keep_rows, bt)
    torch.cuda.synchronize()
    ref = dict(case2)
    ref["codes"], ref["scales"], ref["rope"] = case2["codes"].copy(), case2["scales"].copy(), case2["rope"].copy()
    O.q8g64_append_paged(O.RULE_ROCM_MLA, lat, ref["codes"], ref["scales"], tables2[0], keep_rows, bt)
    O.half_append_paged(0, kr, ref["rope"], tables2[0], keep_rows, bt)
    ref["lens"] = np.array([keep_rows + extra], dtype=np.uint32)
    want_f, _ = oracle_mla(ref)
    live = dict(ref, codes=codes_t.cpu().numpy(), scales=scales_t.cpu().numpy().view(np.uint16), rope=rope_t.cpu().numpy().view(np.uint16))
    assert np.array_equal(live["codes"], ref["codes"]) and np.array_equal(live["scales"], ref["scales"])
    got = run_mla(live).cpu().numpy()
    assert_attention_close(got, want_f, "rollback + append")


def _oracle_mla_heads(case, b, heads_picked):
    """The oracle on a few heads of one sequence: heads are independent, so slicing the query and kv_b rows of those heads
    gives exactly what the full call computes for them."""
    qd, kd = case["nope"] + case["rope_dim"], case["nope"] + case["value"]
    q = case["q_bits"][b].reshape(case["heads"], qd)[heads_picked].reshape(1, -1)
    w = case["kv_b_bits"].reshape(case["heads"], kd, case["latent"])[heads_picked].reshape(-1, case["latent"])
    n = len(heads_picked)
    sub = dict(case, q_bits=q, kv_b_bits=w, lens=case["lens"][b:b + 1], tables=case["tables"][b:b + 1], heads=n,
               spec=O.MlaSpec(case["latent"], case["rope_dim"], n * qd, n * kd, n))
    want_f, want_b = oracle_mla(sub)
    return want_f[0].reshape(n, case["value"])


@pytest.mark.parametrize("block_tokens", [64, 16])
def test_config4_full_size(block_tokens):
    """Benchmark config 4 at its own size: B = 4, 128 heads, 65,536 tokens, with the reference's 64-token pages (the
    instantiation the bench times: whole 32-row steps from one page) and with 16-token pages (per-row table lookups).
    The oracle runs on heads 0, 63, 64, 127 -- both 64-head blocks of a workgroup pair, first and last column -- of two
    sequences sliced out of the full call's output; a zero query at full length must give the projected mean latent."""
    ctx = 65536
    case = make_mla_case(4, [ctx, ctx, ctx - 37, ctx], 128, block_tokens=block_tokens)
    got = run_mla(case).cpu().numpy().reshape(4, 128, 128)
    picks = [0, 63, 64, 127]
    for b in (1, 2):
        want = _oracle_mla_heads(case, b, picks)
        print("config4 full", block_tokens, b, assert_attention_close(got[b][picks], want, f"config 4 full size, sequence {b}"))
    case["q_bits"][:] = 0
    zero = run_mla(case).cpu().numpy().reshape(4, 128, 128)
    lat = O.gather_dequant_rows(O.FMT_Q8, case["codes"], case["scales"], O.SCALE_BF16, case["tables"][2], block_tokens, 0, ctx - 37, 512)
    w = O.bf16_to_f32(case["kv_b_bits"]).reshape(128, 256, 512)[:, 128:, :]
    want = np.einsum("hvc,c->hv", w.astype(np.float64), lat.astype(np.float64).mean(0))
    assert np.abs(zero[2] - want).max() < 2e-3


# ---- prefill chunks: several query rows per sequence --------------------------------------------------------------

def make_mla_chunk_case(seed, lens, rows, heads, **kw):
    """An MLA case whose sequences end in a chunk of `rows` query rows (already in the cache): queries [batch * rows, ...]."""
    case = make_mla_case(seed, lens, heads, **kw)
    rng = np.random.default_rng(seed + 1000)
    q = rng.standard_normal((len(lens) * rows, heads * (case["nope"] + case["rope_dim"]))).astype(np.float32)
    case["q_bits"] = O.f32_to_bf16(q)
    case["rows"] = rows
    return case


def oracle_mla_chunk(case, selection=None):
    """The oracle's own query_rows > 1 arm (src/kernel/cpu/mla.rs:958-1076): row r of a chunk at query_start sees
    query_start + r + 1 tokens.  Returns f32 and bf16-bit outputs [batch * rows, heads * value_dim]."""
    spec, bt, rows = case["spec"], case["block_tokens"], case["rows"]
    kv_b = weights_f32(case)
    outs_f, outs_b = [], []
    for b, l in enumerate(case["lens"]):
        l = int(l)
        codes = O.gather_rows_bytes(case["codes"], case["tables"][b], bt, 0, l, case["latent"])
        scales = O.gather_rows_bytes(case["scales"], case["tables"][b], bt, 0, l, case["latent"] // 64 * 2).view(np.uint16)
        rope = O.gather_rows_bytes(case["rope"], case["tables"][b], bt, 0, l, case["rope_dim"] * 2).view(np.uint16)
        sel, width = None, 0
        if selection is not None:
            sel, width = selection[b * rows:(b + 1) * rows], selection.shape[1]
        rc, ob, of, _ = O.mla_absorbed_q8_history(spec, case["q_bits"][b * rows:(b + 1) * rows], rows, l - rows, codes, scales, 64,
                                                  rope, l, kv_b, selection=sel, width=width)
        assert rc == 0
        outs_f.append(of.reshape(rows, -1))
        outs_b.append(ob.reshape(rows, -1))
    return np.concatenate(outs_f), np.concatenate(outs_b)


def run_mla_chunk(case, out_dtype=None, selection=None, compact=True, q_kind="bf16", wide_tiles=False):
    from zllm_amd import ops

    q = to_torch_bf16(case["q_bits"], "cuda")
    if q_kind != "bf16":  # the same bf16-representable values carried as f32 or f16 (f16 holds them after a second rounding)
        q = upload(O.bf16_to_f32(case["q_bits"]))
        q = q.to(torch.float16) if q_kind == "f16" else q
    kv_b, weight_kw = weight_args(case)
    out = ops.mla_decode(q, kv_b, upload(case["codes"]), upload(case["scales"]),
                         upload(case["rope"]), upload(case["tables"]), upload(case["lens"]), case["heads"],
                         case["nope"] + case["rope_dim"], case["nope"] + case["value"], case["latent"], case["rope_dim"],
                         case["block_tokens"], int(case["lens"].max()), out_dtype=out_dtype or torch.float32, out_compact=compact,
                         selection=None if selection is None else upload(selection), query_rows=case["rows"], wide_tiles=wide_tiles,
                         **weight_kw)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("heads,lens,rows,block_tokens", [(16, [40], 8, 16), (128, [700, 300], 5, 16), (32, [1300, 64, 129], 64, 64),
                                                          (20, [33, 97], 33, 16), (64, [2500], 3, 48)])
def test_mla_prefill_chunk_matches_oracle(heads, lens, rows, block_tokens):
    """Chunked MLA prefill: `rows` query rows per sequence, causal inside the chunk, f32 and bf16 output
    (the reference returns bf16 for more than one row, src/backend/rocm/attention.rs:17-19)."""
    case = make_mla_chunk_case(heads + rows, lens, rows, heads, block_tokens=block_tokens)
    want_f, want_b = oracle_mla_chunk(case)
    got = run_mla_chunk(case).cpu().numpy()
    print("mla chunk", heads, lens, rows, assert_attention_close(got, want_f, f"MLA chunk heads={heads} lens={lens} rows={rows}"))
    got_b = run_mla_chunk(case, out_dtype=torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16)
    diff = np.abs(O.bf16_to_f32(got_b).astype(np.float64) - O.bf16_to_f32(want_b))
    step = np.maximum(np.abs(O.bf16_to_f32(want_b)), 2.0 ** -126) * 2.0 ** -7
    assert (diff <= step + 2e-3).all()


def test_mla_ragged_batch_with_the_token_count_hint():
    """One long sequence among short ones: with the sum of the lengths as a hint the plan cuts short splits (the long
    sequence then has many workgroups), without it every sequence is planned as the longest.  Same results either way."""
    from zllm_amd import capi
    import ctypes as C

    lens = [4000, 100, 64, 700, 33, 1]
    case = make_mla_case(57, lens, 32)
    want_f, _ = oracle_mla(case)
    plain = run_mla(case).cpu().numpy()
    hinted = run_mla(case, total_ctx_tokens=sum(lens)).cpu().numpy()
    assert_attention_close(plain.reshape(want_f.shape), want_f, "MLA ragged batch")
    assert_attention_close(hinted.reshape(want_f.shape), want_f, "MLA ragged batch with the hint")
    args = capi.MlaDecodeArgs()
    args.batch, args.heads, args.q_head_dim, args.kv_head_dim, args.latent_dim, args.rope_dim = len(lens), 32, 192, 256, 512, 64
    args.block_tokens, args.max_ctx_len, args.q_dtype, args.out_dtype, args.out_compact = 16, max(lens), capi.DTYPE_BF16, capi.DTYPE_F32, 1
    lib = capi.load()
    plain_plan, hinted_plan = capi.SplitRecordLayout(), capi.SplitRecordLayout()
    assert lib.zllm_attn_mla_decode_record_layout(C.byref(args), C.byref(plain_plan)) == 0
    args.total_ctx_tokens = sum(lens)
    assert lib.zllm_attn_mla_decode_record_layout(C.byref(args), C.byref(hinted_plan)) == 0
    assert hinted_plan.chunk_tokens < plain_plan.chunk_tokens and hinted_plan.dense == 1  # more, shorter splits; records over the live ones


@pytest.mark.parametrize("heads,lens", [(16, [20000]), (32, [9000, 70]), (64, [17000]), (32, [8300, 8200])])
def test_mla_few_rows_of_many_splits_take_the_wide_merge(heads, lens):
    """One or two sequences of few heads are cut into a split per compute unit, 128 or 256 records per (row, head): the
    merge then runs as eight workgroups per pair, without the sequence lengths (a short sequence beside a long one has
    records that say "empty"), and the projection as a kernel of its own.  f32 and bf16 output."""
    case = make_mla_case(91 + heads, lens, heads, block_tokens=64)
    want_f, want_b = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    print("mla wide merge", heads, lens, assert_attention_close(got.reshape(want_f.shape), want_f, f"MLA heads={heads} lens={lens}"))
    got_b = run_mla(case, out_dtype=torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16)
    diff = np.abs(O.bf16_to_f32(got_b).astype(np.float64).reshape(want_f.shape) - O.bf16_to_f32(want_b).reshape(want_f.shape))
    assert (diff <= np.maximum(np.abs(want_f), 2.0 ** -126) * 2.0 ** -7 + 2e-3).all()


@pytest.mark.parametrize("heads", [16, 20])
def test_mla_short_and_peaked_rows_in_the_narrow_layout(heads):
    """Calls of at most 32 heads score the two token halves of a step in waves of their own.  A row that sees one key, or a
    few, must come out as precisely as in the wide layout: its largest probability is exactly 1 and numerator and
    denominator carry the same rounded weights (a reference moved to whole numbers cost these rows half their margin:
    1.2e-3 to 1.45e-3 against the 2e-3 bound).  Checked at half the usual bound, and a one-key selection at a twentieth of it."""
    lens = [1, 2, 31, 32, 33, 65, 511]
    case = make_mla_case(400 + heads, lens, heads, block_tokens=64)
    want, _ = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    print("mla narrow short rows", heads, assert_attention_close(got.reshape(want.shape), want, f"MLA narrow heads={heads}", atol=1e-3))
    selection = draw_selection(np.random.default_rng(5), lens, 1, True)
    want_s, _ = oracle_mla(case, selection=selection)
    got_s = run_mla(case, selection=selection).cpu().numpy()
    print("mla narrow one key", heads, assert_attention_close(got_s.reshape(want_s.shape), want_s, f"MLA narrow one key heads={heads}", atol=1e-4))


def test_mla_batched_decode_on_the_matrix_core_stages():
    """A decode batch of sixteen rows and more takes the matrix-core absorb and projection (one query row per sequence
    here; chunks take them through test_mla_prefill_chunk_matches_oracle): 40 ragged sequences, strided and compact
    output, and the query as bf16 and as f32 (one block of sixteen rows is partly empty: 40 = 2.5 blocks)."""
    rng = np.random.default_rng(41)
    lens = [int(x) for x in rng.integers(1, 900, size=40)]
    case = make_mla_case(41, lens, 32)
    want_f, want_b = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    print("mla batch 40", assert_attention_close(got.reshape(want_f.shape), want_f, "MLA batch of 40"))
    got32 = run_mla(case, q_f32=True).cpu().numpy()
    assert np.array_equal(got, got32)  # the f32 query holds bf16-representable values
    strided = run_mla(case, compact=False).cpu().numpy().reshape(40, 32, 192)[:, :, :128]
    assert np.array_equal(strided.reshape(got.shape), got)


def test_mla_matrix_core_stages_at_192_query_and_256_value_columns():
    """The reference's decode test has 192 query columns next to the rope and 256 value columns
    (src/kernel/rocm/hip/attention/paged_mla.rs:6226-6233).  The matrix-core absorb then stages half the latent columns
    a workgroup, and the projection runs sixteen waves: a decode batch of 20 rows (split merge, then projection from
    merged rows), a chunk of 40 rows (one record a row) and a chunk of 200 rows (sixteen-wave absorb)."""
    case = make_mla_case(301, [int(x) for x in np.random.default_rng(301).integers(1, 700, size=20)], 16, nope=192, value=256)
    want_f, _ = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    print("mla 192/256 batch", assert_attention_close(got.reshape(want_f.shape), want_f, "MLA 192/256 batch of 20"))
    for rows, lens in ((40, [300, 120]), (200, [260])):
        chunk = make_mla_chunk_case(302 + rows, lens, rows, 16, nope=192, value=256)
        want_c, _ = oracle_mla_chunk(chunk)
        got_c = run_mla_chunk(chunk).cpu().numpy()
        print("mla 192/256 chunk", rows, assert_attention_close(got_c.reshape(want_c.shape), want_c, f"MLA 192/256 chunk of {rows}"))


def test_mla_chunk_query_types_on_the_matrix_core_absorb():
    case = make_mla_chunk_case(9, [300, 120], 20, 16)
    want_f, _ = oracle_mla_chunk(case)
    for q_kind in ("bf16", "f32"):
        got = run_mla_chunk(case, q_kind=q_kind).cpu().numpy()
        assert_attention_close(got, want_f, f"MLA chunk q as {q_kind}")


@pytest.mark.parametrize("rows", [4, 11])
def test_mla_prefill_chunk_rows_equal_single_row_calls(rows):
    """Row r of a chunk is the decode step of a sequence that ends at that row.  With 8 query rows the call runs the
    decode kernels: same bits.  With 22 it runs absorb and projection on the matrix cores, sixteen rows a workgroup: the
    f32 sums run in another order, an absorbed query differs from the single-row one by a bf16 step in a few elements
    out of a million, and the outputs agree to 5e-4."""
    case = make_mla_chunk_case(77, [600, 90], rows, 32)
    got = run_mla_chunk(case).cpu().numpy()
    for b, l in enumerate(case["lens"]):
        for r in range(rows):
            single = dict(case)
            single["lens"] = np.array([int(l) - (rows - 1) + r], dtype=np.uint32)
            single["tables"] = case["tables"][b:b + 1]
            single["q_bits"] = case["q_bits"][b * rows + r:b * rows + r + 1]
            one = run_mla(single, max_ctx_len=int(case["lens"].max())).cpu().numpy()
            if rows == 4:
                assert np.array_equal(one[0], got[b * rows + r]), (b, r)
            else:
                assert np.abs(one[0] - got[b * rows + r]).max() <= 5e-4, (b, r)


def test_mla_prefill_chunk_zero_query_is_the_running_mean():
    """The reference's chunk vector (src/kernel/cpu/mla.rs:1197-1205: zero queries, two rows at position 2 of four
    tokens whose values are 1/10, 2/20, 3/30, 4/40 -> [2, 20, 2.5, 25]) on this kernel's shape: zero queries make
    every row the mean of the value projections of the tokens it sees, here 4 tokens and a chunk of 2 rows."""
    heads = 16
    case = make_mla_chunk_case(5, [4], 2, heads)
    case["q_bits"][:] = 0
    # latent column 0 carries t + 1 and column 64 (another scale group) 10 (t + 1); the value weights pick them out
    lat = np.zeros((4, 512), dtype=np.float32)
    lat[:, 0] = [1, 2, 3, 4]
    lat[:, 64] = [10, 20, 30, 40]
    case["codes"][:] = 0
    case["scales"][:] = 0
    O.q8g64_append_paged(O.RULE_ROCM_MLA, lat, case["codes"], case["scales"], case["tables"][0], 0, case["block_tokens"])
    w = np.zeros((heads, 256, 512), dtype=np.float32)
    w[:, 128, 0] = 1.0   # value column 0 <- latent column 0
    w[:, 129, 64] = 1.0  # value column 1 <- latent column 64
    case["kv_b_bits"] = O.f32_to_bf16(w.reshape(heads * 256, 512))
    got = run_mla_chunk(case).cpu().numpy().reshape(2, heads, 128)
    want_f, _ = oracle_mla_chunk(case)
    assert_attention_close(got.reshape(2, -1), want_f, "zero-query chunk")
    # 1, 2, 3 (and 10, 20, 30) are exact in Q8 with these scales up to the bf16 rounding of the scale: compare at 1e-2
    np.testing.assert_allclose(got[0, :, 0], 2.0, rtol=1e-2)
    np.testing.assert_allclose(got[0, :, 1], 20.0, rtol=1e-2)
    np.testing.assert_allclose(got[1, :, 0], 2.5, rtol=1e-2)
    np.testing.assert_allclose(got[1, :, 1], 25.0, rtol=1e-2)
    assert (got[:, :, 2:] == 0).all()


def test_mla_prefill_chunk_with_per_row_selection():
    """Selected-token prefill: one list per query row, positions inside the row's causal prefix
    (src/kernel/cpu/mla.rs:1008-1018)."""
    rows, top_k = 4, 64
    case = make_mla_chunk_case(31, [500, 300], rows, 16)
    rng = np.random.default_rng(32)
    sel = np.zeros((2 * rows, top_k), dtype=np.uint32)
    for b, l in enumerate(case["lens"]):
        for r in range(rows):
            sel[b * rows + r] = rng.choice(int(l) - rows + r + 1, size=top_k, replace=False)
    want_f, _ = oracle_mla_chunk(case, selection=sel)
    got = run_mla_chunk(case, selection=sel).cpu().numpy()
    assert_attention_close(got, want_f, "selected chunk")

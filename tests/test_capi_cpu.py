"""CPU-only checks of the C-ABI library: it loads, exports every declared symbol, and its host-side
layout arithmetic reproduces the reference's known answers (no GPU call is made here)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from zllm_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(capi.LIB_PATH):
        from zllm_amd.build import build_library

        build_library()
    return capi.load()


def test_every_declared_symbol_is_exported(lib):
    header = open(os.path.join(ROOT, "include", "zllm_attn.h")).read()
    declared = set(re.findall(r"\b(zllm_(?:attn|kv)_[a-z0-9_]+)\s*\(", header))
    assert declared == set(capi.SYMBOLS), declared ^ set(capi.SYMBOLS)
    for name in declared:
        assert getattr(lib, name) is not None


def test_struct_sizes_follow_the_header():
    # pointers first, then 32-bit fields: natural alignment, no surprises for an FFI binding
    assert C.sizeof(capi.Q8AppendArgs) == 5 * 8 + 7 * 4 + 4
    assert C.sizeof(capi.GqaDecodeArgs) == 10 * 8 + 8 + 9 * 4 + 2 * 4 + 3 * 4 + 4 + 4 + 8 + 4 + 4  # + padding, gate fields
    # stage_mask, top_k, selection pointers, query_rows, total_ctx_tokens; then the kv_b scales pointer, three 32-bit fields + padding
    assert C.sizeof(capi.MlaDecodeArgs) == 9 * 8 + 8 + 9 * 4 + 3 * 4 + 4 + 4 + 2 * 8 + 4 + 4 + 8 + 3 * 4 + 4


def test_key_range_known_answers(lib):
    # src/attention/gqa.rs:334-339
    def kr(w, q, e):
        s, t = C.c_uint64(), C.c_uint64()
        lib.zllm_attn_key_range(w, q, e, C.byref(s), C.byref(t))
        return s.value, t.value

    assert kr(3, 4, 5) == (2, 5) and kr(3, 1, 2) == (0, 2) and kr(0, 4, 5) == (0, 5)
    assert kr(1024, 8191, 8192) == (7168, 8192)


def test_layout_known_answers(lib, oracle):
    # src/kv_cache/mod.rs:615-625, 667-675; src/backend/rocm/kv_cache.rs:3617-3624
    assert lib.zllm_kv_bytes_per_token(0, 8, 4, 4) == 20
    assert lib.zllm_kv_bytes_per_token(1, 2, 4, 4) == 24
    assert lib.zllm_kv_bytes_per_token(0, 512, 64, 64) == 656
    assert lib.zllm_kv_bytes_per_token(1, 8, 128, 64) == 2112
    assert lib.zllm_kv_bytes_per_token(0, 8, 4, 3) == 0
    off = (C.c_uint64 * 5)()
    assert lib.zllm_kv_layout_offsets(0, 8, 4, 4, 2, 3, 1, off) == 120
    assert (off[1], off[2], off[3]) == (60, 84, 96)
    # agrees with the oracle's restatement on a sweep
    for kind, a, b, g, layers, cap, layer in [(1, 8, 128, 64, 3, 1000, 2), (0, 512, 64, 64, 4, 77, 1), (1, 4, 128, 64, 1, 4096, 0)]:
        total = lib.zllm_kv_layout_offsets(kind, a, b, g, layers, cap, layer, off)
        t2, o2 = oracle.layout_offsets(kind, a, b, g, layers, cap, layer)
        n = 4 if kind == 0 else 5
        assert total == t2 and list(off)[:n] == [int(v) for v in o2[:n]]


def test_ring_plan_known_answers(lib, oracle):
    plan = (C.c_uint64 * 6)()
    assert lib.zllm_kv_ring_write_plan(3, 10, 0, 5, plan) == 0
    assert (plan[1], plan[3], plan[4], plan[5]) == (2, 2, 1, 2)  # src/kv_cache/mod.rs:705-709
    assert lib.zllm_kv_ring_write_plan(3, 10, 0, 0, plan) == -1
    assert lib.zllm_kv_ring_write_plan(3, 10, 8, 5, plan) == -1
    assert b"ring write plan" in lib.zllm_attn_last_error()
    rng = np.random.default_rng(0)
    for _ in range(200):
        cap, pos, cnt = int(rng.integers(1, 40)), int(rng.integers(0, 100)), int(rng.integers(1, 60))
        rc = lib.zllm_kv_ring_write_plan(cap, 200, pos, cnt, plan)
        ref = oracle.ring_write_plan(cap, 200, pos, cnt)
        assert (rc == 0) == (ref is not None)
        if ref:
            assert list(plan) == [ref[k] for k in ("end", "source_start", "token_count", "first_slot", "first_count", "second_count")]


def test_invalid_shapes_are_reported_without_a_gpu(lib):
    args = capi.GqaDecodeArgs()
    assert lib.zllm_attn_gqa_decode_workspace_bytes(C.byref(args)) == 0
    assert lib.zllm_attn_gqa_decode(C.byref(args), None) == -1
    assert b"invalid shape" in lib.zllm_attn_last_error()
    args.batch, args.num_heads, args.num_kv_heads, args.head_dim = 1, 16, 3, 128  # heads % kv_heads != 0
    assert lib.zllm_attn_gqa_decode(C.byref(args), None) == -1
    args.num_kv_heads, args.head_dim = 4, 96
    assert lib.zllm_attn_gqa_decode(C.byref(args), None) == -1
    args.head_dim, args.block_tokens, args.max_kv_len, args.score_scale = 128, 16, 4096, 0.0
    assert lib.zllm_attn_gqa_decode(C.byref(args), None) == -1
    assert b"score_scale" in lib.zllm_attn_last_error()
    args.score_scale = 0.088
    args.kv_format, args.scale_dtype, args.q_dtype = capi.KV_Q8G64, capi.SCALE_F16, capi.DTYPE_F32
    assert lib.zllm_attn_gqa_decode_workspace_bytes(C.byref(args)) > 0
    assert lib.zllm_attn_gqa_decode(C.byref(args), None) == -1  # null pointers
    assert b"null pointer" in lib.zllm_attn_last_error()
    q8 = capi.Q8AppendArgs()
    assert lib.zllm_attn_q8g64_append(C.byref(q8), None) == -1
    # MLA decode: shape, selection and alignment errors come back before anything touches a device
    mla = capi.MlaDecodeArgs()
    assert lib.zllm_attn_mla_decode(C.byref(mla), None) == -1
    mla.batch, mla.heads, mla.q_head_dim, mla.kv_head_dim, mla.latent_dim, mla.rope_dim = 1, 16, 192, 256, 512, 64
    mla.block_tokens, mla.max_ctx_len, mla.q_dtype, mla.out_dtype = 64, 4096, capi.DTYPE_BF16, capi.DTYPE_F32
    assert lib.zllm_attn_mla_decode_workspace_bytes(C.byref(mla)) > 0
    mla.selection, mla.top_k = 0x1000, 0
    assert lib.zllm_attn_mla_decode_workspace_bytes(C.byref(mla)) == 0 and b"top_k" in lib.zllm_attn_last_error()
    mla.top_k = 2048
    dense = capi.MlaDecodeArgs.from_buffer_copy(mla)
    dense.selection, dense.top_k = None, 0
    # a selection bounds every sequence by top_k tokens: fewer splits, smaller workspace
    assert lib.zllm_attn_mla_decode_workspace_bytes(C.byref(mla)) < lib.zllm_attn_mla_decode_workspace_bytes(C.byref(dense))
    for name in ("q", "kv_b", "latent_codes", "latent_scales", "rope_cache", "ctx_lens", "out", "workspace"):
        setattr(mla, name, 0x10000)
    mla.workspace_bytes = 1 << 30
    mla.rope_cache = 0x10008
    assert lib.zllm_attn_mla_decode(C.byref(mla), None) == -1 and b"aligned" in lib.zllm_attn_last_error()
    prologue = capi.GqaPrologueArgs()
    assert lib.zllm_attn_gqa_prologue(C.byref(prologue), None) == -1


def test_cpp_host_layer_builds_and_exports_the_backend_methods():
    """The C++ mirror of the reference's backend traits (zllm_amd/host) is a shared library next to the C ABI."""
    import os
    import subprocess

    lib = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "zllm_amd", "libzllm_backend.so")
    assert os.path.exists(lib), "run __graft_entry__.build()"
    names = subprocess.run(["nm", "-DC", "--defined-only", lib], capture_output=True, text=True, check=True).stdout
    for method in ("zllm_amd::RocmContext::gqa_prefill_attention_cached", "zllm_amd::RocmContext::append_mla(",
                   "zllm_amd::RocmContext::append_mla_rope", "zllm_amd::RocmContext::mla_decode_attention",
                   "zllm_amd::CausalWindow::key_range", "zllm_amd::RocmKvCache::new_gqa", "zllm_amd::RocmKvCache::new_mla",
                   "zllm_amd::RocmContext::gqa_prefill_attention_cached_visible", "zllm_amd::RocmContext::gqa_prefill_attention_cached_from",
                   "zllm_amd::RocmContext::mla_prefill_attention(", "zllm_amd::RocmContext::mla_prefill_attention_rope",
                   "zllm_amd::committed_cache_rows"):
        assert method in names, method


def test_split_plan_covers_the_host_bound_and_sizes_the_workspace(lib):
    """The split plan is a function of the host arguments: max_chunks splits of chunk_tokens tokens cover max_kv_len and
    nothing more, which is the bound a recorded graph stays valid under (a longer kv_lens[b] on the device is read up
    to max_chunks * chunk_tokens tokens only)."""
    rng = np.random.default_rng(5)
    for _ in range(300):
        args = capi.GqaDecodeArgs()
        args.batch = int(rng.integers(1, 65))
        args.num_kv_heads = int(rng.choice([1, 2, 4, 8]))
        args.num_heads = args.num_kv_heads * int(rng.choice([1, 2, 4, 8, 16]))
        args.head_dim = int(rng.choice([64, 128, 256]))
        args.max_kv_len = int(rng.integers(1, 200000))
        args.block_tokens = int(rng.choice([1, 16, 64]))
        args.score_scale = 0.1
        args.kv_format, args.scale_dtype, args.q_dtype = capi.KV_Q8G64, capi.SCALE_F16, capi.DTYPE_F32
        if rng.random() < 0.5:  # a ragged batch: the hint may only shorten the splits, never drop coverage
            args.total_kv_tokens = int(rng.integers(1, args.batch * args.max_kv_len + 1) % (1 << 32))
        chunk, chunks = C.c_uint32(), C.c_uint32()
        assert lib.zllm_attn_gqa_decode_split_plan(C.byref(args), C.byref(chunk), C.byref(chunks)) == 0
        assert chunk.value % 32 == 0 and chunk.value >= 64 and chunks.value >= 1
        assert chunk.value * chunks.value >= args.max_kv_len
        assert chunk.value * (chunks.value - 1) < args.max_kv_len  # no split lies wholly beyond the bound
        # the record layout: [sequence][max_chunks] rows for a plan of equal lengths; a ragged plan numbers its records over
        # the live splits, so their bytes follow the tokens there are and not batch x longest sequence
        layout = capi.SplitRecordLayout()
        assert lib.zllm_attn_gqa_decode_record_layout(C.byref(args), C.byref(layout)) == 0
        assert (layout.chunk_tokens, layout.max_chunks) == (chunk.value, chunks.value)
        align = lambda n: (n + 255) // 256 * 256
        if layout.dense:
            assert args.total_kv_tokens and layout.record_rows < args.batch * chunks.value
            assert layout.record_rows == args.total_kv_tokens // chunk.value + 2 * args.batch
            # every sequence's splits fit: sum of ceil((len + 31) / chunk) over any lengths that add up to the total
            assert layout.record_rows >= -(-args.total_kv_tokens // chunk.value) + args.batch
        else:
            assert layout.record_rows == args.batch * chunks.value and layout.first_rows_offset == 0
        records = layout.record_rows * args.num_heads
        assert layout.partial_offset == 0 and layout.stats_offset == align(records * args.head_dim * 4)
        size = layout.stats_offset + align(records * 8)
        if layout.dense:
            assert layout.first_rows_offset == size
            size += align(args.batch * 4)
        assert lib.zllm_attn_gqa_decode_workspace_bytes(C.byref(args)) == size
    bad = capi.GqaDecodeArgs()
    assert lib.zllm_attn_gqa_decode_split_plan(C.byref(bad), None, None) == -1
    assert lib.zllm_attn_gqa_decode_record_layout(C.byref(bad), C.byref(capi.SplitRecordLayout())) == -1


def test_ragged_mla_records_follow_the_tokens_not_the_longest_sequence(lib):
    """One 1M-token context among 31 of 2,000 tokens: records numbered over the live splits stay a few MiB where
    [row][max_chunks] rows would take most of a gigabyte; a plan of equal lengths keeps the rows that need no lookup."""
    args = capi.MlaDecodeArgs()
    args.batch, args.heads, args.q_head_dim, args.kv_head_dim = 32, 64, 192, 256
    args.latent_dim, args.rope_dim, args.block_tokens = 512, 64, 64
    args.max_ctx_len, args.total_ctx_tokens = 1 << 20, (1 << 20) + 31 * 2000
    args.q_dtype, args.out_dtype = capi.DTYPE_BF16, capi.DTYPE_F32
    layout = capi.SplitRecordLayout()
    assert lib.zllm_attn_mla_decode_record_layout(C.byref(args), C.byref(layout)) == 0
    assert layout.dense == 1 and layout.record_rows == args.total_ctx_tokens // layout.chunk_tokens + args.batch
    assert layout.record_rows < 400 and layout.max_chunks * layout.chunk_tokens >= args.max_ctx_len
    assert lib.zllm_attn_mla_decode_workspace_bytes(C.byref(args)) < 64 << 20
    assert args.batch * layout.max_chunks * args.heads * 512 * 4 > 512 << 20  # what the rows by sequence would have taken
    args.total_ctx_tokens = 0
    assert lib.zllm_attn_mla_decode_record_layout(C.byref(args), C.byref(layout)) == 0
    assert layout.dense == 0 and layout.first_rows_offset == 0 and layout.record_rows == args.batch * layout.max_chunks


def test_split_plan_fills_whole_rounds_of_the_compute_units(lib):
    """A batch that does not divide the 256 CUs must not leave a few workgroups for a round of their own: with uniform
    lengths the launch's rounds are at least 4/5 full whenever a sequence has keys to spare, and a head_dim-128
    Q8g64 split stays within the 127 pages whose table entries the page-streaming kernel keeps in registers."""
    for batch in (1, 2, 3, 5, 7, 8, 12, 13, 24, 31, 48, 64):
        for max_len in (4096, 16384, 32768, 65536, 131072):
            args = capi.GqaDecodeArgs()
            args.batch, args.num_kv_heads, args.num_heads, args.head_dim = batch, 8, 64, 128
            args.max_kv_len, args.block_tokens, args.score_scale = max_len, 16, 0.1
            args.kv_format, args.scale_dtype, args.q_dtype = capi.KV_Q8G64, capi.SCALE_F16, capi.DTYPE_BF16
            chunk, chunks = C.c_uint32(), C.c_uint32()
            assert lib.zllm_attn_gqa_decode_split_plan(C.byref(args), C.byref(chunk), C.byref(chunks)) == 0
            groups = batch * chunks.value  # one workgroup per (sequence, split): all eight KV heads ride in it
            rounds = -(-groups // 256)
            if chunk.value > 64:  # at the shortest split there are no more keys to spread
                assert groups >= rounds * 256 * 4 // 5, (batch, max_len, chunk.value, chunks.value)
            assert chunk.value <= 127 * 16, (batch, max_len, chunk.value)


def test_prefill_workspace_covers_few_row_chunks_and_kv_splits(lib):
    """One workspace size serves whichever route the call takes: a chunk of one row over a long prefix runs as a decode
    item (row ranges + split records), a short chunk is cut into KV splits (records per row and part), a chunk of a
    workgroup per compute unit and more needs none."""
    pre = capi.GqaPrefillArgs()
    pre.num_heads, pre.num_kv_heads, pre.head_dim, pre.block_tokens = 32, 8, 128, 16
    pre.score_scale, pre.kv_format, pre.scale_dtype, pre.q_dtype = 0.1, capi.KV_Q8G64, capi.SCALE_F16, capi.DTYPE_BF16
    sizes = {}
    for rows, position in ((1, 32768), (2, 32768), (64, 32768), (2048, 50000), (1, 100)):
        pre.rows, pre.position = rows, position
        sizes[rows, position] = lib.zllm_attn_gqa_prefill_workspace_bytes(C.byref(pre))
    assert sizes[1, 32768] > 256 and sizes[2, 32768] > sizes[1, 32768]  # a row's records beside its ranges
    assert sizes[64, 32768] >= 64 * 32 * 128 * 4 * 2                     # at least two parts of f32 records a row
    assert sizes[2048, 50000] == 0
    assert sizes[1, 100] > 0                                            # still a decode item (its records are small)


def test_prefill_and_mla_argument_checks_without_a_gpu(lib):
    pre = capi.GqaPrefillArgs()
    pre.rows, pre.num_heads, pre.num_kv_heads, pre.head_dim, pre.block_tokens = 8, 8, 2, 128, 16
    pre.score_scale, pre.kv_format, pre.scale_dtype = 0.1, capi.KV_Q8G64, capi.SCALE_F16
    for name in ("q", "k_plane", "k_scales", "v_plane", "v_scales", "out"):
        setattr(pre, name, 0x10000)
    pre.k_plane = 0x10008  # codes are read as 16-byte vectors
    assert lib.zllm_attn_gqa_prefill_chunk(C.byref(pre), None) == -1 and b"aligned" in lib.zllm_attn_last_error()
    pre.k_plane, pre.k_scales = 0x10000, 0x10002  # scales as 4-byte words
    assert lib.zllm_attn_gqa_prefill_chunk(C.byref(pre), None) == -1 and b"aligned" in lib.zllm_attn_last_error()
    pre.k_scales = 0x10000
    pre.table, pre.table_stride, pre.position = 0x20000, 3, 48  # 3 pages of 16 tokens < 48 + 8
    assert lib.zllm_attn_gqa_prefill_chunk(C.byref(pre), None) == -1 and b"cannot cover" in lib.zllm_attn_last_error()
    assert lib.zllm_attn_gqa_prefill_workspace_bytes(C.byref(pre)) == 0
    pre.table_stride = 4
    pre.head_dim = 256  # this geometry runs its rows through the decode kernels and needs their split records
    assert lib.zllm_attn_gqa_prefill_workspace_bytes(C.byref(pre)) > 8 * 8
    assert lib.zllm_attn_gqa_prefill_chunk(C.byref(pre), None) == -1 and b"workspace" in lib.zllm_attn_last_error()
    # a chunk whose rows run as decode items is a decode call of that many rows: more than the merge's grid can index is
    # refused before anything is launched, and so is a decode batch of that size
    pre.rows, pre.q_dtype, pre.table = 70000, capi.DTYPE_F32, None
    assert lib.zllm_attn_gqa_prefill_chunk(C.byref(pre), None) == -1 and b"65535" in lib.zllm_attn_last_error()
    dec = capi.GqaDecodeArgs()
    dec.batch, dec.num_heads, dec.num_kv_heads, dec.head_dim, dec.block_tokens, dec.max_kv_len = 70000, 8, 2, 128, 16, 64
    dec.score_scale, dec.kv_format, dec.scale_dtype = 0.1, capi.KV_Q8G64, capi.SCALE_F16
    assert lib.zllm_attn_gqa_decode_workspace_bytes(C.byref(dec)) == 0 and b"65535" in lib.zllm_attn_last_error()
    # MLA: value part and query-row limits
    mla = capi.MlaDecodeArgs()
    mla.batch, mla.heads, mla.q_head_dim, mla.kv_head_dim, mla.latent_dim, mla.rope_dim = 1, 16, 192, 128, 512, 64
    mla.block_tokens, mla.max_ctx_len, mla.q_dtype, mla.out_dtype = 64, 4096, capi.DTYPE_BF16, capi.DTYPE_F32
    assert lib.zllm_attn_mla_decode_workspace_bytes(C.byref(mla)) == 0 and b"value_dim" in lib.zllm_attn_last_error()  # nope == kv_head_dim
    mla.kv_head_dim, mla.q_head_dim, mla.rope_dim = 600, 192, 64  # value 472 > q_head_dim with strided output
    assert lib.zllm_attn_mla_decode_workspace_bytes(C.byref(mla)) == 0 and b"value_dim" in lib.zllm_attn_last_error()
    mla.out_compact = 1
    assert lib.zllm_attn_mla_decode_workspace_bytes(C.byref(mla)) > 0
    mla.kv_head_dim = 256
    mla.batch, mla.query_rows = 40, 2048
    assert lib.zllm_attn_mla_decode_workspace_bytes(C.byref(mla)) == 0 and b"65535" in lib.zllm_attn_last_error()
    mla.batch, mla.query_rows = 2, 64
    one = capi.MlaDecodeArgs.from_buffer_copy(mla)
    one.query_rows = 0
    assert lib.zllm_attn_mla_decode_workspace_bytes(C.byref(mla)) > lib.zllm_attn_mla_decode_workspace_bytes(C.byref(one)) > 0


def test_mla_widths_and_weight_forms_are_validated_on_the_host(lib):
    """Latent widths are multiples of 64 up to 1,024, rope widths even up to 256, kv_b is bf16 / f32 or 8- / 4-bit codes with
    scales and a group size that divides the latent width: everything else is refused before a workspace size is named."""
    def args(**kw):
        a = capi.MlaDecodeArgs()
        a.batch, a.heads, a.q_head_dim, a.kv_head_dim, a.latent_dim, a.rope_dim = 2, 4, 96, 128, 128, 32
        a.block_tokens, a.max_ctx_len, a.q_dtype, a.out_dtype = 16, 500, capi.DTYPE_BF16, capi.DTYPE_F32
        for k, v in kw.items():
            setattr(a, k, v)
        return a

    size = lib.zllm_attn_mla_decode_workspace_bytes
    assert size(C.byref(args())) > 0
    assert size(C.byref(args(latent_dim=1024, rope_dim=256, q_head_dim=320))) > 0
    assert size(C.byref(args(kv_b_bits=32))) > 0
    scales = C.c_void_p(0x1000)  # never read on the host
    assert size(C.byref(args(kv_b_bits=8, kv_b_scales=scales, kv_b_group=64, kv_b_scale_dtype=capi.SCALE_F16))) > 0
    assert size(C.byref(args(kv_b_bits=4, kv_b_scales=scales, kv_b_group=128))) > 0
    for bad, word in ((dict(latent_dim=96), "multiple of 64"), (dict(latent_dim=1088), "multiple of 64"), (dict(rope_dim=31), "even"),
                      (dict(rope_dim=258, q_head_dim=322), "even"), (dict(kv_b_bits=5), "kv_b_bits"),
                      (dict(kv_b_bits=8, kv_b_group=64), "scales"), (dict(kv_b_bits=8, kv_b_scales=scales, kv_b_group=48), "group size"),
                      (dict(kv_b_bits=4, kv_b_scales=scales, kv_b_group=64, kv_b_scale_dtype=7), "scale dtype")):
        assert size(C.byref(args(**bad))) == 0
        assert word in capi.last_error(), (bad, capi.last_error())


def test_head_dim_192_is_taken_over_q8g64_only(lib):
    a = capi.GqaDecodeArgs()
    a.batch, a.num_heads, a.num_kv_heads, a.head_dim, a.max_kv_len, a.block_tokens, a.score_scale = 2, 12, 3, 192, 4000, 16, 0.07
    a.kv_format, a.scale_dtype, a.q_dtype = capi.KV_Q8G64, capi.SCALE_F16, capi.DTYPE_BF16
    assert lib.zllm_attn_gqa_decode_workspace_bytes(C.byref(a)) > 0
    a.kv_format = capi.KV_F16
    assert lib.zllm_attn_gqa_decode_workspace_bytes(C.byref(a)) == 0 and "f16 KV supports head_dim 128 and 256" in capi.last_error()
    a.kv_format, a.head_dim = capi.KV_Q8G64, 96
    assert lib.zllm_attn_gqa_decode_workspace_bytes(C.byref(a)) == 0
    pre = capi.GqaPrefillArgs()
    pre.rows, pre.position, pre.num_heads, pre.num_kv_heads, pre.head_dim, pre.block_tokens, pre.score_scale = 64, 500, 12, 3, 192, 16, 0.07
    pre.kv_format, pre.scale_dtype, pre.q_dtype = capi.KV_Q8G64, capi.SCALE_F16, capi.DTYPE_BF16
    assert lib.zllm_attn_gqa_prefill_workspace_bytes(C.byref(pre)) > 0  # its rows run as decode items: ranges and split records


def test_planning_entry_points_survive_arbitrary_argument_blocks(lib):
    """The entry points that run on the host alone (workspace sizes, split plans, record layouts) take argument blocks
    whose numbers are zero, huge or inconsistent: each answers 0 / -1 with a message, or a size, and never divides by zero
    or walks a null pointer.  Pointers stay null: nothing here reads device memory."""
    rng = np.random.default_rng(4242)
    edge = [0, 1, 2, 3, 15, 16, 31, 32, 33, 63, 64, 65, 127, 128, 192, 255, 256, 512, 576, 1024, 4096, 65535, 65536, 1 << 20, (1 << 31) - 1,
            1 << 31, (1 << 32) - 1]

    def fill(args, skip=()):
        for name, ctype in args._fields_:
            if name in skip or ctype is C.c_void_p:
                continue
            if ctype is C.c_float:
                setattr(args, name, float(rng.choice([0.0, -1.0, 0.09, 1e30, float("inf"), float("nan")])))
            elif ctype is C.c_uint64:
                setattr(args, name, int(rng.choice(edge)) * int(rng.choice([1, 1 << 20])))
            elif ctype is C.c_int:
                setattr(args, name, int(rng.choice([-1, 0, 1, 2, 3, 7])))
            else:
                setattr(args, name, int(rng.choice(edge)))

    for _ in range(3000):
        g = capi.GqaDecodeArgs()
        fill(g)
        if rng.random() < 0.7:  # mostly near-valid blocks: the plans' arithmetic is what is under test
            g.kv_format, g.scale_dtype, g.q_dtype, g.score_scale = capi.KV_Q8G64, capi.SCALE_F16, capi.DTYPE_BF16, 0.1
            g.num_kv_heads = int(rng.choice([1, 2, 3, 8]))
            g.num_heads = g.num_kv_heads * int(rng.choice([1, 4, 16, 17, 64]))
            g.head_dim = int(rng.choice([64, 128, 192, 256]))
            g.block_tokens = int(rng.choice([1, 16, 48, 64, 1 << 20]))
        need = lib.zllm_attn_gqa_decode_workspace_bytes(C.byref(g))
        chunk, chunks, layout = C.c_uint32(), C.c_uint32(), capi.SplitRecordLayout()
        rc = lib.zllm_attn_gqa_decode_split_plan(C.byref(g), C.byref(chunk), C.byref(chunks))
        assert lib.zllm_attn_gqa_decode_record_layout(C.byref(g), C.byref(layout)) == rc
        assert (need > 0) == (rc == 0)
        if rc == 0:
            assert chunk.value >= 32 and chunks.value >= 1 and layout.record_rows >= 1
        p = capi.GqaPrefillArgs()
        fill(p)
        if rng.random() < 0.7:
            p.kv_format, p.scale_dtype, p.q_dtype, p.out_dtype, p.score_scale = capi.KV_Q8G64, capi.SCALE_F16, capi.DTYPE_BF16, capi.DTYPE_F32, 0.1
            p.num_kv_heads = int(rng.choice([1, 2, 8]))
            p.num_heads = p.num_kv_heads * int(rng.choice([1, 4, 16, 200]))
            p.head_dim = int(rng.choice([64, 128, 192, 256]))
            p.block_tokens = int(rng.choice([1, 16, 48, 64]))
            p.rows = int(rng.choice([1, 2, 16, 17, 300, 5000]))
            p.position = int(rng.choice([0, 1, 1000, 50000, 1 << 22]))
            p.gate_cols, p.softcap = 0, 0.0
        lib.zllm_attn_gqa_prefill_workspace_bytes(C.byref(p))
        m = capi.MlaDecodeArgs()
        fill(m)
        if rng.random() < 0.7:
            m.q_dtype, m.out_dtype = capi.DTYPE_BF16, capi.DTYPE_F32
            m.heads = int(rng.choice([1, 16, 33, 128]))
            m.latent_dim, m.rope_dim = int(rng.choice([64, 512, 1024])), int(rng.choice([2, 64, 256]))
            nope, value = int(rng.choice([16, 128])), int(rng.choice([16, 128, 192]))
            m.q_head_dim, m.kv_head_dim = nope + m.rope_dim, nope + value
            m.block_tokens = int(rng.choice([1, 16, 48, 64]))
            m.kv_b_bits, m.stage_mask, m.top_k = 0, 0, 0
            m.batch, m.query_rows = int(rng.choice([1, 4, 33, 3000])), int(rng.choice([0, 1, 5, 512]))
        need = lib.zllm_attn_mla_decode_workspace_bytes(C.byref(m))
        rc = lib.zllm_attn_mla_decode_record_layout(C.byref(m), C.byref(layout))
        assert (need > 0) == (rc == 0)

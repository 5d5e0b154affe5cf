"""Split records numbered over the live splits (a ragged plan: `total_kv_tokens` / `total_ctx_tokens` given): a long
sequence among short ones keeps a small workspace and the results of the plan for equal lengths; a caller that asks for
ZLLM_STAGE_PARTIAL finds the records where zllm_attn_gqa_decode_record_layout says they are and combines them itself
(the shard form of the reference, src/kernel/rocm/hip/attention/paged_mla.rs:3642; record sizing :2987-2994,3248-3257)."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, make_gqa_q8_case, oracle_gqa_decode, to_torch_bf16, upload
from tests.test_gpu_mla_decode import make_mla_case, oracle_mla, run_mla

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def decode_call(case, score_scale, total_kv_tokens, window=0):
    from zllm_amd import capi, ops

    pl, lens = case["planes"], case["lens"]
    q = to_torch_bf16(case["q_bits"], "cuda") if case["q_bits"] is not None else upload(case["q"])
    first = None
    if window:
        first = upload(np.array([O.key_range(window, int(l) - 1, int(l))[0] if l else 0 for l in lens], dtype=np.uint32))
    keep = [q, first] + [upload(pl[n]) for n in ("k_codes", "k_scales", "v_codes", "v_scales")] + [upload(case["tables"]), upload(lens)]
    args, out, ws = ops.gqa_decode_args(q, keep[2], keep[3], keep[4], keep[5], keep[6], keep[7], case["hq"], case["hkv"], case["d"],
                                        case["block_tokens"], score_scale, max(int(lens.max()), 1), first_visible=first,
                                        kv_format=capi.KV_Q8G64, scale_dtype=case["scale_dtype"], total_kv_tokens=total_kv_tokens)
    return args, out, ws, keep  # the argument block holds addresses only: `keep` owns the tensors behind them


@pytest.mark.parametrize("hq,hkv,d,long_len,window", [(16, 4, 128, 150_000, 0), (8, 1, 128, 60_000, 0), (8, 2, 256, 40_000, 0),
                                                      (8, 2, 64, 50_000, 0), (16, 4, 128, 90_000, 3000)])
def test_one_long_sequence_among_short_ones(hq, hkv, d, long_len, window):
    """The records of the ragged plan follow the tokens there are: a workspace well below what [sequence][max_chunks]
    rows would take, and the oracle's output for the long sequence, a short one, an empty one and the last."""
    from zllm_amd import capi

    rng = np.random.default_rng(long_len + hq)
    lens = [int(x) for x in rng.integers(1, 900, size=24)]
    lens[5], lens[11], lens[-1] = long_len, 0, 65
    case = make_gqa_q8_case(long_len % 1000 + d, lens, hq, hkv, d, outliers=True)
    visible = [min(l, window) if window else l for l in lens]
    args, out, ws, keep = decode_call(case, 0.09, sum(visible), window=window)
    layout = capi.SplitRecordLayout()
    assert capi.load().zllm_attn_gqa_decode_record_layout(C.byref(args), C.byref(layout)) == 0
    if not window:
        assert layout.dense == 1 and layout.record_rows * 4 < len(lens) * layout.max_chunks
    capi.check(capi.load().zllm_attn_gqa_decode(C.byref(args), None))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    want = oracle_gqa_decode(case, 0.09, window=window)
    print("dense records", hq, hkv, d, long_len, window, "rows", layout.record_rows, "of", len(lens) * layout.max_chunks,
          assert_attention_close(got, want, f"ragged {hq}/{hkv} d={d} long={long_len} window={window}"))
    assert (got[11] == 0).all()


def test_partial_stage_records_are_where_the_layout_says():
    """ZLLM_STAGE_PARTIAL leaves un-merged (partial, max, sum) records; combining them on the host with the documented
    indexing -- row g * max_chunks + c for a plan of equal lengths, first_rows[g] + c for a ragged one -- gives the
    call's own merged output.  Exponents are base 2 of the scaled scores; a record's partial is its un-normalised sum."""
    from zllm_amd import capi

    lens = [5000, 130, 0, 2200, 64, 700, 31, 1]
    hq, hkv, d = 8, 2, 128
    case = make_gqa_q8_case(321, lens, hq, hkv, d, outliers=True)
    lib = capi.load()
    for hint in (0, sum(lens)):
        args, out, ws, keep = decode_call(case, 0.09, hint)
        layout = capi.SplitRecordLayout()
        assert lib.zllm_attn_gqa_decode_record_layout(C.byref(args), C.byref(layout)) == 0
        assert layout.dense == (1 if hint else 0)
        capi.check(lib.zllm_attn_gqa_decode(C.byref(args), None))
        torch.cuda.synchronize()
        whole = out.cpu().numpy().copy()
        ws.fill_(0x7f)  # whatever the partial stage does not write must not be needed
        out.fill_(7.0)
        args.stages = capi.STAGE_PARTIAL
        capi.check(lib.zllm_attn_gqa_decode(C.byref(args), None))
        torch.cuda.synchronize()
        assert (out == 7.0).all()  # the partial stage writes records only
        raw = ws.cpu().numpy()
        rows = layout.record_rows
        partial = raw[layout.partial_offset:layout.partial_offset + rows * hq * d * 4].view(np.float32).reshape(rows, hq, d)
        stats = raw[layout.stats_offset:layout.stats_offset + rows * hq * 8].view(np.float32).reshape(rows, hq, 2)
        first_rows = raw[layout.first_rows_offset:layout.first_rows_offset + len(lens) * 4].view(np.uint32) if layout.dense else None
        mine = np.zeros((len(lens), hq, d), dtype=np.float64)
        for g, n in enumerate(lens):
            splits = min(layout.max_chunks, -(-n // layout.chunk_tokens))
            if splits == 0:
                continue
            base = int(first_rows[g]) if layout.dense else g * layout.max_chunks
            mx = stats[base:base + splits, :, 0].astype(np.float64)
            sm = stats[base:base + splits, :, 1].astype(np.float64)
            top = mx.max(axis=0)
            w = np.where(sm > 0, np.exp2(mx - top), 0.0)
            mine[g] = (partial[base:base + splits].astype(np.float64) * w[:, :, None]).sum(0) / (sm * w).sum(0)[:, None]
        np.testing.assert_allclose(mine.reshape(len(lens), -1), whole, rtol=2e-5, atol=2e-6)
        if layout.dense:  # rows in sequence order, one run per sequence with splits
            live = [g for g, n in enumerate(lens) if n]
            counts = [min(layout.max_chunks, -(-lens[g] // layout.chunk_tokens)) for g in live]
            assert [int(first_rows[g]) for g in live] == [int(x) for x in np.cumsum([0] + counts[:-1])]
        # ZLLM_STAGE_MERGE over the records in the workspace gives the whole call's output again
        args.stages = capi.STAGE_MERGE
        capi.check(lib.zllm_attn_gqa_decode(C.byref(args), None))
        torch.cuda.synchronize()
        assert (out.cpu().numpy() == whole).all()


@pytest.mark.parametrize("heads,wide_tiles,page", [(32, False, 16), (64, False, 64), (128, True, 64), (16, False, 64)])
def test_mla_one_long_sequence_among_short_ones(heads, wide_tiles, page):
    """MLA decode with the token-count hint: records over the live splits (the workspace stays small whatever the longest
    context), both split-KV kernels, against the oracle."""
    from zllm_amd import capi

    lens = [300, 33, 9000 if heads > 64 else 30_000, 1, 64, 700, 1500, 2]
    case = make_mla_case(700 + heads, lens, heads, block_tokens=page)
    want, _ = oracle_mla(case)
    got = run_mla(case, total_ctx_tokens=sum(lens), wide_tiles=wide_tiles).cpu().numpy()
    print("mla dense records", heads, assert_attention_close(got.reshape(want.shape), want, f"MLA ragged heads={heads}"))
    args = capi.MlaDecodeArgs()
    args.batch, args.heads, args.q_head_dim, args.kv_head_dim, args.latent_dim, args.rope_dim = len(lens), heads, 192, 256, 512, 64
    args.block_tokens, args.max_ctx_len, args.q_dtype, args.out_dtype, args.out_compact = page, max(lens), capi.DTYPE_BF16, capi.DTYPE_F32, 1
    args.total_ctx_tokens = sum(lens)
    layout = capi.SplitRecordLayout()
    assert capi.load().zllm_attn_mla_decode_record_layout(C.byref(args), C.byref(layout)) == 0
    assert layout.dense == 1 and layout.record_rows * 2 < len(lens) * layout.max_chunks


def test_a_hint_below_the_real_sum_drops_splits_but_stays_in_bounds():
    """`total_kv_tokens` sizes the record rows of a ragged plan.  Given a sum below the real one, the splits past the rows it
    sized find nothing to do and write nothing: the sequences whose splits all fit are still right, and the same buffers
    serve a correct call afterwards."""
    from zllm_amd import capi

    lens = [3000, 2000, 4000, 100]
    case = make_gqa_q8_case(17, lens, 16, 4, 128)
    want = oracle_gqa_decode(case, 0.09)
    args, out, ws, keep = decode_call(case, 0.09, 3000)
    layout = capi.SplitRecordLayout()
    assert capi.load().zllm_attn_gqa_decode_record_layout(C.byref(args), C.byref(layout)) == 0
    splits = [-(-l // layout.chunk_tokens) for l in lens]
    assert layout.dense == 1 and splits[0] <= layout.record_rows < sum(splits)  # the first sequence fits, the batch does not
    guard = torch.full((1 << 20,), 0x5A, dtype=torch.uint8, device="cuda")  # whatever follows the workspace stays untouched
    ws.zero_()
    capi.check(capi.load().zllm_attn_gqa_decode(C.byref(args), None))
    torch.cuda.synchronize()
    assert_attention_close(out[:1].cpu().numpy(), want[:1], "the sequence whose splits fit")
    assert bool((guard == 0x5A).all())
    args, out, ws, keep = decode_call(case, 0.09, sum(lens))
    capi.check(capi.load().zllm_attn_gqa_decode(C.byref(args), None))
    torch.cuda.synchronize()
    assert_attention_close(out.cpu().numpy(), want, "the same call with an honest hint")

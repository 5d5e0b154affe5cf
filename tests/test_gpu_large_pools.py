"""Pools whose planes pass 4 GiB: physical rows whose byte offsets need 64 bits, as a serving pool on this GPU's 288 GB has
them (the reference widens to u64 for the same reason, src/kernel/rocm/hip/attention/paged_mla/source.hip:46-54).  The
Q8g64 decode kernels have such cases in tests/test_gpu_gqa_decode.py; here are the MLA cache (append, both split-KV
kernels, the selected-token arm, a chunk of rows), the chunk kernels of GQA prefill over Q8g64 and f16 rows, and f16 decode.
Every case builds the same rows in a compact pool and in a far one and asks for the same bits from both, then checks the
far result against the oracle."""
import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, to_torch_bf16, upload
from tests.test_gpu_mla_decode import make_mla_case, make_mla_chunk_case, oracle_mla, oracle_mla_chunk

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def far_ids(rng, used_blocks, far_blocks):
    """Block ids all over a pool of `far_blocks`, both ends included, for the compact ids 0..used_blocks-1."""
    ids = rng.choice(far_blocks, size=used_blocks, replace=False).astype(np.int64)
    ids[0], ids[-1] = far_blocks - 1, 0
    return ids


def move_pages(compact, ids, far_blocks, block_rows):
    """A device plane of far_blocks pages (never cleared) holding page c of `compact` at page ids[c]."""
    compact = compact if isinstance(compact, torch.Tensor) else upload(compact)
    cols = compact.shape[1]
    far = torch.empty((far_blocks * block_rows, cols), dtype=compact.dtype, device="cuda")
    pages = compact.shape[0] // block_rows
    far.view(far_blocks, block_rows * cols)[torch.from_numpy(ids[:pages]).cuda()] = compact.view(pages, block_rows * cols)
    return far


def mla_call(case, planes, tables, **kw):
    from zllm_amd import ops

    rows = case.get("rows", 1)
    out = ops.mla_decode(to_torch_bf16(case["q_bits"], "cuda"), upload(case["kv_b_bits"]), planes[0], planes[1], planes[2], upload(tables),
                         upload(case["lens"]), case["heads"], case["nope"] + case["rope_dim"], case["nope"] + case["value"], case["latent"],
                         case["rope_dim"], case["block_tokens"], int(case["lens"].max()), query_rows=rows, **kw)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("heads,page,lens,rows", [(128, 64, [3000, 700, 65], 1), (16, 16, [2500, 33], 1), (64, 64, [1500, 300], 6)])
def test_mla_cache_beyond_4_gib(heads, page, lens, rows):
    """A latent-code plane of 6 GiB (12.6 M rows; rope plane 1.5 GiB, scales 190 MiB) with the sequences' pages anywhere
    in it: decode through both split-KV kernels, the selected-token arm and a chunk of query rows give the bits of the
    compact pool and meet the oracle; a row appended through the far table lands where the table says."""
    from zllm_amd import ops

    rng = np.random.default_rng(heads + page)
    case = make_mla_chunk_case(900 + heads, lens, rows, heads, block_tokens=page) if rows > 1 else make_mla_case(900 + heads, lens, heads, block_tokens=page)
    used = case["codes"].shape[0] // page
    far_blocks = (6 << 30) // (512 * page)
    ids = far_ids(rng, used, far_blocks)
    torch.cuda.empty_cache()
    near = [upload(case[n]) for n in ("codes", "scales", "rope")]
    far = [move_pages(case[n], ids, far_blocks, page) for n in ("codes", "scales", "rope")]
    far_tables = ids[case["tables"].astype(np.int64)].astype(np.uint32)
    assert int(far_tables.max()) * page * 512 > (4 << 30)
    want, _ = oracle_mla_chunk(case) if rows > 1 else oracle_mla(case)
    variants = [dict()] if rows > 1 else [dict(), dict(total_ctx_tokens=int(sum(lens)))]
    if heads > 32 and page % 32 == 0:
        variants.append(dict(wide_tiles=True))
    for kw in variants:
        a = mla_call(case, near, case["tables"], **kw)
        b = mla_call(case, far, far_tables, **kw)
        assert np.array_equal(a, b), kw
        assert_attention_close(b.reshape(want.shape), want, f"MLA far pool heads={heads} page={page} {kw}")
    if rows == 1:
        top_k = 64
        selection = np.stack([rng.permutation(max(int(l), top_k))[:top_k] % int(l) for l in lens]).astype(np.uint32)
        a = mla_call(case, near, case["tables"], selection=upload(selection))
        b = mla_call(case, far, far_tables, selection=upload(selection))
        assert np.array_equal(a, b)
        # one more token per sequence, appended through the far table: the bytes the oracle's quantizer writes, at the far row
        for s, l in enumerate(lens):
            lat = rng.standard_normal((1, 512)).astype(np.float32)
            kr = rng.standard_normal((1, 64)).astype(np.float32)
            if l % page == 0:
                continue  # the next row would open a page the case did not draw
            ops.mla_append(upload(lat), upload(kr), far[0], far[1], far[2], upload(far_tables[s]), l, page)
            torch.cuda.synchronize()
            row = int(far_tables[s][l // page]) * page + l % page
            codes = np.zeros((1, 512), dtype=np.int8)
            scales = np.zeros((1, 8), dtype=np.uint16)
            O.q8g64_append_paged(O.RULE_ROCM_MLA, lat, codes, scales, None, 0, 1)
            assert np.array_equal(far[0][row].cpu().numpy(), codes[0])
            assert np.array_equal(far[1][row].cpu().numpy().view(np.uint16), scales[0])
            assert np.array_equal(far[2][row].cpu().numpy().view(np.uint16), O.f32_to_bf16(kr)[0])
    del far, near
    torch.cuda.empty_cache()


@pytest.mark.parametrize("kv,d,hq,hkv,prefix,chunk", [("q8", 128, 32, 8, 3000, 300), ("q8", 256, 8, 2, 1500, 100), ("q8", 64, 16, 4, 2000, 64),
                                                      ("f16", 128, 16, 8, 2000, 200), ("f16", 256, 8, 2, 1000, 70)])
def test_gqa_prefill_and_f16_decode_beyond_4_gib(kv, d, hq, hkv, prefix, chunk):
    """The chunk kernels (and, for f16 rows, the decode kernel) over planes of 5 GiB: a chunk's output is that of the same
    rows in a compact pool, bit for bit, and meets the oracle."""
    from zllm_amd import capi, ops

    rng = np.random.default_rng(d + hq)
    bt = 16
    cols = hkv * d
    total = prefix + chunk
    blocks = (total + bt - 1) // bt
    k = rng.standard_normal((total, cols)).astype(np.float32)
    v = rng.standard_normal((total, cols)).astype(np.float32)
    q_bits = O.f32_to_bf16(rng.standard_normal((chunk, hq * d)).astype(np.float32))
    scale = 1.0 / np.sqrt(d)
    compact_table = rng.permutation(blocks).astype(np.uint32)
    if kv == "q8":
        planes = {n: np.zeros((blocks * bt, cols if "codes" in n else cols // 64), dtype=np.int8 if "codes" in n else np.uint16)
                  for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
        O.q8g64_append_paged(O.RULE_METAL_GQA, k, planes["k_codes"], planes["k_scales"], compact_table, 0, bt)
        O.q8g64_append_paged(O.RULE_METAL_GQA, v, planes["v_codes"], planes["v_scales"], compact_table, 0, bt)
        kd = O.gather_dequant_rows(O.FMT_Q8, planes["k_codes"], planes["k_scales"], O.SCALE_F16, compact_table, bt, 0, total, cols)
        vd = O.gather_dequant_rows(O.FMT_Q8, planes["v_codes"], planes["v_scales"], O.SCALE_F16, compact_table, bt, 0, total, cols)
        order = ("k_codes", "k_scales", "v_codes", "v_scales")
        fmt, code_bytes = capi.KV_Q8G64, cols
    else:
        planes = {n: np.zeros((blocks * bt, cols), dtype=np.uint16) for n in ("k", "v")}
        O.half_append_paged(1, k, planes["k"], compact_table, 0, bt)
        O.half_append_paged(1, v, planes["v"], compact_table, 0, bt)
        kd, vd = k.astype(np.float16).astype(np.float32), v.astype(np.float16).astype(np.float32)
        order = ("k", None, "v", None)
        fmt, code_bytes = capi.KV_F16, cols * 2
    far_blocks = (5 << 30) // (code_bytes * bt)
    ids = far_ids(rng, blocks, far_blocks)
    far_table = ids[compact_table.astype(np.int64)].astype(np.uint32)
    assert int(far_table.max()) * bt * code_bytes > (4 << 30)
    torch.cuda.empty_cache()

    def as_device(n, far):
        if n is None:
            return None
        t = move_pages(planes[n], ids, far_blocks, bt) if far else upload(planes[n])
        return t.view(torch.float16) if kv == "f16" else t

    outs, decodes = {}, {}
    for name, table in (("near", compact_table), ("far", far_table)):
        dev = [as_device(n, name == "far") for n in order]
        out = ops.gqa_prefill_chunk(to_torch_bf16(q_bits, "cuda"), dev[0], dev[1], dev[2], dev[3], upload(table), prefix, hq, hkv, d, bt, scale,
                                    kv_format=fmt)
        torch.cuda.synchronize()
        outs[name] = out.cpu().numpy()
        if kv == "f16":
            dec = ops.gqa_decode(to_torch_bf16(q_bits[-1:], "cuda"), dev[0], None, dev[2], None, upload(table).view(1, -1),
                                 upload(np.array([total], dtype=np.uint32)), hq, hkv, d, bt, scale, total, kv_format=capi.KV_F16)
            torch.cuda.synchronize()
            decodes[name] = dec.cpu().numpy()
        del dev
        torch.cuda.empty_cache()
    assert np.array_equal(outs["near"], outs["far"])
    rc, want = O.gqa_prefill_at_visible(O.bf16_to_f32(q_bits), kd, vd, 0, total, prefix, hq, hkv, d, score_scale=scale)
    assert rc == 0
    assert_attention_close(outs["far"], want, f"prefill over a far pool, {kv} d={d}")
    if kv == "f16":
        assert np.array_equal(decodes["near"], decodes["far"])
        assert_attention_close(decodes["far"], want[-1:], f"f16 decode over a far pool, d={d}")

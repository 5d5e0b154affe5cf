"""Calls at the edges of what the argument checks accept: the largest batches, one row, one head, one token, a hundred and
more query heads on one KV head, pages of one token and of 65,536 -- each against the CPU oracle (on a sample of the rows
where the call has tens of thousands)."""
import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, make_gqa_q8_case, oracle_gqa_decode
from tests.test_gpu_gqa_decode import run_decode
from tests.test_gpu_gqa_prefill import run_case
from tests.test_gpu_mla_decode import make_mla_case, oracle_mla, run_mla

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.mark.parametrize("batch,hq,hkv,d,length", [(65535, 1, 1, 64, 1), (65535, 2, 1, 128, 3), (20000, 8, 1, 128, 17), (4096, 16, 2, 256, 40)])
def test_decode_batches_up_to_the_row_limit(batch, hq, hkv, d, length):
    """65,535 sequences is what a decode call takes (the merge numbers rows with a grid dimension); with and without the
    token-count hint, 40 sampled rows against the oracle."""
    rng = np.random.default_rng(batch + d)
    case = make_gqa_q8_case(5, [length] * batch, hq, hkv, d, block_tokens=16)
    sub = rng.choice(batch, size=40, replace=False)
    small = dict(case)
    small["lens"], small["tables"], small["q"] = case["lens"][sub], case["tables"][sub], case["q"][sub]
    want = oracle_gqa_decode(small, 0.09)
    for hint in (0, length * batch):
        got = run_decode(case, 0.09, total_kv_tokens=hint)
        assert_attention_close(got[sub], want, f"decode batch={batch} {hq}/{hkv} d={d} hint={hint}")


@pytest.mark.parametrize("batch,heads,length", [(65535, 1, 1), (8000, 16, 5), (300, 128, 33)])
def test_mla_batches_up_to_the_row_limit(batch, heads, length):
    rng = np.random.default_rng(batch)
    case = make_mla_case(6, [length] * batch, heads, block_tokens=16)
    got = run_mla(case).cpu().numpy()
    sub = rng.choice(batch, size=12, replace=False)
    small = dict(case)
    small["lens"], small["tables"], small["q_bits"] = case["lens"][sub], case["tables"][sub], case["q_bits"][sub]
    want, _ = oracle_mla(small)
    assert_attention_close(got.reshape(batch, -1)[sub], want.reshape(len(sub), -1), f"MLA batch={batch} heads={heads}")


@pytest.mark.parametrize("prefix,chunk,hq,hkv,d", [(0, 1, 8, 2, 128), (0, 1, 1, 1, 64), (1000, 40, 128, 1, 128), (500, 5, 200, 1, 128),
                                                   (300, 3, 256, 1, 256), (0, 700, 136, 1, 256)])
def test_prefill_of_one_row_and_of_many_heads_on_one_kv_head(prefix, chunk, hq, hkv, d):
    """A first token alone; 128 query heads on a KV head (a row tile of two rows); 136 to 256 on one (more columns than a
    row tile has: the rows run as decode items)."""
    out, want = run_case(7, prefix, chunk, hq, hkv, d=d)
    assert_attention_close(out.cpu().numpy(), want, f"prefill prefix={prefix} chunk={chunk} {hq}/{hkv} d={d}")


@pytest.mark.parametrize("page,lens", [(1, [9000, 5]), (1 << 16, [70000, 3])])
def test_pages_of_one_token_and_of_65536(page, lens):
    case = make_gqa_q8_case(8, lens, 8, 2, 128, block_tokens=page, pool_blocks=len(lens) + 2 if page > 4096 else None)
    got = run_decode(case, 0.09)
    assert_attention_close(got, oracle_gqa_decode(case, 0.09), f"pages of {page}")

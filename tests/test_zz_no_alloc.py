"""zllm_attn_gqa_decode_static (split records in the library's static device array) against zllm_attn_gqa_decode
(split records in a workspace of the caller's): same kernels, so the outputs are compared bit for bit, and both
against the CPU oracle within the attention tolerance.  Two calls in a row, the second smaller than the first, so
that records left in the array by the first call lie beside and beyond the second call's."""
import ctypes as C

import numpy as np
import pytest

from tests.cases import assert_attention_close, make_gqa_q8_case, oracle_gqa_decode, to_torch_bf16, upload

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def _device_inputs(case):
    pl = case["planes"]
    q = to_torch_bf16(case["q_bits"], "cuda") if case["q_bits"] is not None else upload(case["q"])
    return (q, upload(pl["k_codes"]), upload(pl["k_scales"]), upload(pl["v_codes"]), upload(pl["v_scales"]), upload(case["tables"]),
            upload(case["lens"]), case["hq"], case["hkv"], case["d"], case["block_tokens"])


def _both(case, score_scale):
    from zllm_amd import capi, ops

    inputs = _device_inputs(case)
    max_len = max(int(case["lens"].max()), 1)
    kw = dict(kv_format=capi.KV_Q8G64, scale_dtype=case["scale_dtype"])
    want = ops.gqa_decode(*inputs, score_scale, max_len, **kw)
    out = torch.empty_like(want)
    ops.gqa_decode_static(*inputs, score_scale, max_len, out=out, **kw)  # warm-up: code objects and the array's address are in place
    torch.cuda.synchronize()
    out.zero_()
    held = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]  # the driver's count: sees a hipMalloc that bypasses torch's allocator
    got = ops.gqa_decode_static(*inputs, score_scale, max_len, out=out, **kw)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == held  # nothing was taken from torch's allocator by the call
    assert torch.cuda.mem_get_info()[0] == free_before, "the static-scratch call changed the device's free memory"
    return got.cpu().numpy(), want.cpu().numpy()


def test_static_scratch_decode_matches_workspace_decode_twice():
    from zllm_amd import ops

    ops.init(0)
    scale = 1.0 / np.sqrt(128.0)
    # first call: eight sequences, many splits; second call: fewer and shorter sequences, other head geometry
    first = make_gqa_q8_case(41, [4000, 1200, 3333, 17, 2500, 64, 900, 4096], 64, 8, 128, q_bf16=True, outliers=True)
    second = make_gqa_q8_case(42, [700, 33, 0], 16, 4, 128)
    for name, case in (("first", first), ("second (smaller)", second)):
        got, want = _both(case, scale)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"{name}: static-scratch output differs from the workspace call"
        assert_attention_close(got, oracle_gqa_decode(case, scale), f"static scratch, {name} call")


def test_static_scratch_rejects_calls_beyond_its_size():
    from zllm_amd import capi, ops

    ops.init(0)
    lib = capi.load()
    limit = lib.zllm_attn_static_scratch_bytes()
    assert limit == 16 << 20
    # 256 sequences x 128 heads x 256 dims: the split records alone pass the array's size; nothing may be launched
    args = capi.GqaDecodeArgs()
    args.batch, args.num_heads, args.num_kv_heads, args.head_dim = 256, 128, 8, 256
    args.max_kv_len, args.block_tokens, args.table_stride = 4096, 16, 256
    args.score_scale = 0.1
    args.kv_format, args.scale_dtype, args.q_dtype = capi.KV_Q8G64, capi.SCALE_F16, capi.DTYPE_F32
    assert lib.zllm_attn_gqa_decode_workspace_bytes(C.byref(args)) > limit
    rc = lib.zllm_attn_gqa_decode_static(C.byref(args), None)
    assert rc < 0 and "static" in capi.last_error()

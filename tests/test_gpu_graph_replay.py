"""The C-ABI calls under HIP graph capture: a captured call is replayed several times with the device inputs changed and
ordinary eager work in between, and every replay must give what the same call gives when launched directly."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, make_gqa_q8_case, oracle_gqa_decode, to_torch_bf16, upload
from tests.test_gpu_mla_decode import make_mla_case, oracle_mla

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def _capture(fn):
    """Warm up on a side stream (as torch asks before a capture), then record `fn` into a graph."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    return graph


def _eager_noise():
    a = torch.randn((256, 256), device="cuda")
    (a @ a).sum().item()  # unrelated work and a synchronization between the replays


def test_gqa_decode_replays_follow_the_device_inputs():
    from zllm_amd import capi, ops

    case = make_gqa_q8_case(700, [900, 2100, 64], 16, 4, 128)
    pl = case["planes"]
    dev = {k: upload(v) for k, v in pl.items()}
    tables, lens = upload(case["tables"]), upload(case["lens"])
    q = upload(case["q"])
    args, out, workspace = ops.gqa_decode_args(q, dev["k_codes"], dev["k_scales"], dev["v_codes"], dev["v_scales"], tables, lens, 16, 4, 128,
                                               case["block_tokens"], 0.088, int(case["lens"].max()), kv_format=capi.KV_Q8G64,
                                               scale_dtype=case["scale_dtype"])
    lib = capi.load()

    def call():
        capi.check(lib.zllm_attn_gqa_decode(C.byref(args), C.c_void_p(torch.cuda.current_stream().cuda_stream)))

    graph = _capture(call)
    rng = np.random.default_rng(701)
    for replay in range(4):
        new_q = rng.standard_normal(case["q"].shape).astype(np.float32)
        new_lens = np.maximum(case["lens"].astype(np.int64) - 37 * replay, 1).astype(np.uint32)
        q.copy_(upload(new_q))
        lens.copy_(upload(new_lens))
        _eager_noise()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.cpu().numpy().copy()
        out.zero_()
        call()
        torch.cuda.synchronize()
        assert np.array_equal(replayed, out.cpu().numpy()), f"replay {replay} differs from the direct launch"
        check = dict(case, q=new_q, q_bits=None, lens=new_lens)
        assert_attention_close(replayed, oracle_gqa_decode(check, 0.088), f"replay {replay}")


def test_mla_decode_replays_follow_the_device_inputs():
    from zllm_amd import capi, ops

    case = make_mla_case(710, [700, 1300], 32)
    q = to_torch_bf16(case["q_bits"], "cuda")
    lens = upload(case["lens"])
    # the argument record holds raw pointers: the tensors behind them have to stay alive with it
    kv_b, codes, scales, rope, tables = (upload(case[k]) for k in ("kv_b_bits", "codes", "scales", "rope", "tables"))
    args, out, workspace = ops.mla_decode_args(q, kv_b, codes, scales, rope, tables, lens, case["heads"], case["nope"] + case["rope_dim"],
                                               case["nope"] + case["value"], case["latent"], case["rope_dim"], case["block_tokens"],
                                               int(case["lens"].max()))
    lib = capi.load()

    def call():
        capi.check(lib.zllm_attn_mla_decode(C.byref(args), C.c_void_p(torch.cuda.current_stream().cuda_stream)))

    graph = _capture(call)
    rng = np.random.default_rng(711)
    for replay in range(3):
        bits = O.f32_to_bf16(rng.standard_normal(case["q_bits"].shape).astype(np.float32))
        new_lens = np.maximum(case["lens"].astype(np.int64) - 101 * replay, 1).astype(np.uint32)
        q.copy_(to_torch_bf16(bits, "cuda"))
        lens.copy_(upload(new_lens))
        _eager_noise()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.float().cpu().numpy().copy()
        out.zero_()
        call()
        torch.cuda.synchronize()
        assert np.array_equal(replayed, out.float().cpu().numpy()), f"replay {replay} differs from the direct launch"
        want, _ = oracle_mla(dict(case, q_bits=bits, lens=new_lens))
        assert_attention_close(replayed.reshape(want.shape), want, f"MLA replay {replay}")


def test_append_then_prefill_in_one_graph():
    """A chunk's K/V append and its attention recorded together (the order a prefill step issues them in)."""
    from zllm_amd import ops

    rng = np.random.default_rng(720)
    hq, hkv, d, bt, prefix, chunk = 8, 2, 128, 16, 300, 70
    cols, total = hkv * d, prefix + chunk
    table = upload(np.arange((total + bt - 1) // bt + 2, dtype=np.uint32)[::-1].copy())
    rows = (len(table)) * bt
    planes = {n: torch.zeros((rows, cols if "codes" in n else cols // 64), dtype=torch.int8 if "codes" in n else torch.int16, device="cuda")
              for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
    k0 = to_torch_bf16(O.f32_to_bf16(rng.standard_normal((prefix, cols)).astype(np.float32)), "cuda")
    v0 = to_torch_bf16(O.f32_to_bf16(rng.standard_normal((prefix, cols)).astype(np.float32)), "cuda")
    ops.q8g64_append(k0, planes["k_codes"], planes["k_scales"], table, 0, bt, O.RULE_METAL_GQA)
    ops.q8g64_append(v0, planes["v_codes"], planes["v_scales"], table, 0, bt, O.RULE_METAL_GQA)
    q = torch.zeros((chunk, hq * d), dtype=torch.bfloat16, device="cuda")
    kc, vc = torch.zeros((chunk, cols), dtype=torch.bfloat16, device="cuda"), torch.zeros((chunk, cols), dtype=torch.bfloat16, device="cuda")
    result = {}

    def step():
        ops.q8g64_append(kc, planes["k_codes"], planes["k_scales"], table, prefix, bt, O.RULE_METAL_GQA)
        ops.q8g64_append(vc, planes["v_codes"], planes["v_scales"], table, prefix, bt, O.RULE_METAL_GQA)
        result["out"] = ops.gqa_prefill_chunk(q, planes["k_codes"], planes["k_scales"], planes["v_codes"], planes["v_scales"], table, prefix,
                                              hq, hkv, d, bt, 0.088, scale_dtype=O.SCALE_F16)

    graph = _capture(step)
    captured_out = result["out"]
    for replay in range(3):
        for t in (q, kc, vc):
            t.copy_(torch.randn(t.shape, device="cuda").to(torch.bfloat16))
        _eager_noise()
        graph.replay()
        torch.cuda.synchronize()
        replayed = captured_out.cpu().numpy().copy()
        step()
        torch.cuda.synchronize()
        assert np.array_equal(replayed, result["out"].cpu().numpy()), f"replay {replay} differs from the direct launch"
        assert np.isfinite(replayed).all() and np.abs(replayed).max() > 0

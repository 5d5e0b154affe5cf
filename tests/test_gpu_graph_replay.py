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
    """A chunk's K/V append and its attention recorded together (the order a prefill step issues them in); every replay is
    held against the direct launch and against the oracle over the pages as the oracle's own append leaves them."""
    from zllm_amd import ops

    rng = np.random.default_rng(720)
    hq, hkv, d, bt, prefix, chunk = 8, 2, 128, 16, 300, 70
    cols, total = hkv * d, prefix + chunk
    host_table = np.arange((total + bt - 1) // bt + 2, dtype=np.uint32)[::-1].copy()
    table = upload(host_table)
    rows = (len(table)) * bt
    planes = {n: torch.zeros((rows, cols if "codes" in n else cols // 64), dtype=torch.int8 if "codes" in n else torch.int16, device="cuda")
              for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
    ref = {n: np.zeros((rows, cols if "codes" in n else cols // 64), dtype=np.int8 if "codes" in n else np.uint16) for n in planes}
    k0_bits = O.f32_to_bf16(rng.standard_normal((prefix, cols)).astype(np.float32))
    v0_bits = O.f32_to_bf16(rng.standard_normal((prefix, cols)).astype(np.float32))
    ops.q8g64_append(to_torch_bf16(k0_bits, "cuda"), planes["k_codes"], planes["k_scales"], table, 0, bt, O.RULE_METAL_GQA)
    ops.q8g64_append(to_torch_bf16(v0_bits, "cuda"), planes["v_codes"], planes["v_scales"], table, 0, bt, O.RULE_METAL_GQA)
    O.q8g64_append_paged(O.RULE_METAL_GQA, O.bf16_to_f32(k0_bits), ref["k_codes"], ref["k_scales"], host_table, 0, bt)
    O.q8g64_append_paged(O.RULE_METAL_GQA, O.bf16_to_f32(v0_bits), ref["v_codes"], ref["v_scales"], host_table, 0, bt)
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
        bits = {n: O.f32_to_bf16(rng.standard_normal(t.shape).astype(np.float32)) for n, t in (("q", q), ("k", kc), ("v", vc))}
        for n, t in (("q", q), ("k", kc), ("v", vc)):
            t.copy_(to_torch_bf16(bits[n], "cuda"))
        _eager_noise()
        graph.replay()
        torch.cuda.synchronize()
        replayed = captured_out.cpu().numpy().copy()
        step()
        torch.cuda.synchronize()
        assert np.array_equal(replayed, result["out"].cpu().numpy()), f"replay {replay} differs from the direct launch"
        # the oracle's append into its own copy of the pages, then the oracle's attention over the gathered rows
        O.q8g64_append_paged(O.RULE_METAL_GQA, O.bf16_to_f32(bits["k"]), ref["k_codes"], ref["k_scales"], host_table, prefix, bt)
        O.q8g64_append_paged(O.RULE_METAL_GQA, O.bf16_to_f32(bits["v"]), ref["v_codes"], ref["v_scales"], host_table, prefix, bt)
        for n in planes:
            got = planes[n].cpu().numpy()
            assert np.array_equal(got.view(ref[n].dtype), ref[n]), f"replay {replay}: plane {n} differs from the oracle's append"
        k = O.gather_dequant_rows(O.FMT_Q8, ref["k_codes"], ref["k_scales"], O.SCALE_F16, host_table, bt, 0, total, cols)
        v = O.gather_dequant_rows(O.FMT_Q8, ref["v_codes"], ref["v_scales"], O.SCALE_F16, host_table, bt, 0, total, cols)
        rc, want = O.gqa_prefill_at_visible(O.bf16_to_f32(bits["q"]), k, v, 0, total, prefix, hq, hkv, d, score_scale=0.088)
        assert rc == 0
        assert_attention_close(replayed, want, f"append + prefill replay {replay}")


def test_mla_append_then_decode_in_one_graph_with_positions_on_the_device():
    """One decode step of an MLA layer as the reference's graph replay records it: the fused append reads the cache row and
    the rope row from device memory (paged_cache_append_mla_f32_q8_bf16_indirect, paged_mla/source.hip:787-807), the
    attention reads the context length from device memory, and the step itself advances both words.  Recorded once, replayed
    for consecutive tokens (a page boundary is crossed); every replay is held against the oracle's append and attention."""
    from zllm_amd import capi, ops

    start, steps, heads, bt = 302, 5, 16, 16
    case = make_mla_case(730, [start + steps + 3], heads, block_tokens=bt)
    host_table = case["tables"][0]
    rng = np.random.default_rng(731)
    half = case["rope_dim"] // 2
    angles = rng.uniform(0, 6.28, size=(start + steps + 8, half)).astype(np.float32)
    cos, sin = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
    ref = {k: case[k].copy() for k in ("codes", "scales", "rope")}
    kv_b, codes, scales, rope, tables = (upload(case[k]) for k in ("kv_b_bits", "codes", "scales", "rope", "tables"))
    dev_cos, dev_sin = upload(cos), upload(sin)
    q = to_torch_bf16(case["q_bits"], "cuda")
    latent = torch.zeros((1, case["latent"]), dtype=torch.float32, device="cuda")
    k_rope = torch.zeros((1, case["rope_dim"]), dtype=torch.float32, device="cuda")
    positions = upload(np.array([start, start], dtype=np.uint32))  # [cache row, rope-table row]
    lens = upload(np.array([start + 1], dtype=np.uint32))  # the context the query sees once its own row is appended
    args, out, workspace = ops.mla_decode_args(q, kv_b, codes, scales, rope, tables, lens, heads, case["nope"] + case["rope_dim"],
                                               case["nope"] + case["value"], case["latent"], case["rope_dim"], bt, start + steps + 3)
    lib = capi.load()

    def step():
        # host-side position / rope_position are wrong on purpose: the device words decide
        ops.mla_append(latent, k_rope, codes, scales, rope, tables[0], 7, bt, cos=dev_cos, sin=dev_sin, rotary_dim=case["rope_dim"],
                       rotary_layout=capi.ROTARY_SPLIT_HALF, rope_position=9, positions=positions)
        capi.check(lib.zllm_attn_mla_decode(C.byref(args), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        positions.add_(1)
        lens.add_(1)

    graph = _capture(step)
    # the warm-up before the capture ran one step at `start` and advanced the words; put them back
    positions.copy_(upload(np.array([start, start], dtype=np.uint32)))
    lens.copy_(upload(np.array([start + 1], dtype=np.uint32)))
    for replay in range(steps):
        position = start + replay
        new_latent = rng.standard_normal((1, case["latent"])).astype(np.float32)
        new_rope = rng.standard_normal((1, case["rope_dim"])).astype(np.float32)
        bits = O.f32_to_bf16(rng.standard_normal(case["q_bits"].shape).astype(np.float32))
        latent.copy_(upload(new_latent))
        k_rope.copy_(upload(new_rope))
        q.copy_(to_torch_bf16(bits, "cuda"))
        _eager_noise()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert positions.cpu().tolist() == [position + 1, position + 1] and lens.cpu().tolist() == [position + 2]
        O.q8g64_append_paged(O.RULE_ROCM_MLA, new_latent, ref["codes"], ref["scales"], host_table, position, bt)
        rc, rotated = O.rope_apply(new_rope, 1, case["rope_dim"], position, cos, sin, layout=0, placement=1)
        assert rc == 0
        O.half_append_paged(0, rotated, ref["rope"], host_table, position, bt)
        assert np.array_equal(codes.cpu().numpy(), ref["codes"]), f"replay {replay}: latent codes differ"
        assert np.array_equal(scales.cpu().numpy().view(np.uint16), ref["scales"]), f"replay {replay}: scale bits differ"
        assert np.array_equal(rope.cpu().numpy().view(np.uint16), ref["rope"]), f"replay {replay}: rope bits differ"
        want, _ = oracle_mla(dict(case, q_bits=bits, lens=np.array([position + 1], dtype=np.uint32), **ref))
        assert_attention_close(out.cpu().numpy().reshape(want.shape), want, f"MLA append + decode replay {replay}")

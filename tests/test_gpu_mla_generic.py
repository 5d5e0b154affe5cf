"""Absorbed MLA decode at latent / rope widths other than 512 / 64 and with kv_b in the other forms the reference's weight
loader reads (f32, W8A16, W4A16: paged_weight, src/kernel/rocm/hip/attention/paged_mla/source.hip:2-26), against the CPU
oracle -- starting with the reference's own rank-64 recipe (src/kernel/cpu/mla.rs:1166-1195), which the device now runs."""
import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, to_torch_bf16, upload
from tests.test_gpu_mla_decode import (make_mla_case, make_mla_chunk_case, oracle_mla, oracle_mla_chunk, run_mla, run_mla_chunk,
                                       set_weight_form)

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.mark.parametrize("weights", ["bf16", "f32"])
def test_reference_rank64_recipe(weights):
    """src/kernel/cpu/mla.rs:1166-1195: rank 64, rope 32, two heads of 32 + 32 query and 32 + 32 KV columns, four cached
    rows of integer-pattern codes with the scale 0.0625, two query rows at position 2, each attending to its two listed
    rows ([0, 2] and [1, 3]).  The device's rows agree with the oracle's absorbed arm to the attention tolerance and,
    as the reference's test asks, with attention over the expanded K/V to 0.02."""
    from zllm_amd import ops

    spec = O.MlaSpec(64, 32, 128, 128, 2)
    q_vals = np.array([(i % 11 - 5) * 0.03125 for i in range(2 * 128)], dtype=np.float32)
    q_bits = O.f32_to_bf16(q_vals).reshape(2, 128)
    codes = np.array([(i * 7 % 31) - 15 for i in range(4 * 64)], dtype=np.int8).reshape(4, 64)
    scales = np.full((4, 1), O.f32_to_bf16(np.array([0.0625], dtype=np.float32))[0], dtype=np.uint16)
    rope = O.f32_to_bf16(np.array([(i % 9 - 4) * 0.015625 for i in range(4 * 32)], dtype=np.float32)).reshape(4, 32)
    kv_b = np.array([(i * 13 % 17 - 8) * 0.0078125 for i in range(128 * 64)], dtype=np.float32).reshape(128, 64)
    selection = np.array([[0, 2], [1, 3]], dtype=np.uint32)
    rc, want_b, want_f, _ = O.mla_absorbed_q8_history(spec, q_bits, 2, 2, codes.view(np.uint8), scales, 64, rope, 4, kv_b,
                                                      selection=selection.reshape(-1), width=2)
    assert rc == 0
    projected = (codes.astype(np.float32) * 0.0625) @ kv_b.T
    rc, expanded = O.mla_selected_bf16_history(spec, q_bits, 2, 2, O.f32_to_bf16(projected.astype(np.float32)), rope, 4,
                                               selection.reshape(-1).tolist(), 2)
    assert rc == 0
    if weights == "bf16":  # multiples of 2^-7 below 1/8: exact in bf16
        kv_b_dev, kw = upload(O.f32_to_bf16(kv_b)), {}
    else:
        kv_b_dev, kw = upload(kv_b), dict(kv_b_bits=32)
    out = ops.mla_decode(to_torch_bf16(q_bits, "cuda"), kv_b_dev, upload(codes), upload(scales), upload(rope), None,
                         upload(np.array([4], dtype=np.uint32)), 2, 64, 64, 64, 32, 64, 4, out_dtype=torch.float32,
                         selection=upload(selection), query_rows=2, **kw)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    print("rank-64 recipe", weights, assert_attention_close(got, want_f.reshape(got.shape), "rank-64 recipe vs the absorbed oracle"))
    assert np.abs(got.reshape(-1) - O.bf16_to_f32(expanded).reshape(-1)).max() < 0.02


@pytest.mark.parametrize("latent,rope,nope,value,heads,lens,page", [
    (64, 32, 32, 32, 2, [4, 1, 70], 16), (128, 64, 64, 64, 5, [300, 33], 16), (192, 32, 96, 128, 3, [129, 640], 64),
    (256, 128, 128, 64, 8, [1000], 48), (576, 64, 128, 128, 4, [257, 64, 31], 16), (1024, 256, 64, 192, 2, [90, 400], 1),
    (512, 32, 128, 128, 6, [700], 16), (448, 2, 16, 16, 1, [65], 16)])
def test_other_widths_match_oracle(latent, rope, nope, value, heads, lens, page):
    """Latent widths from one Q8g64 group to sixteen, rope widths from 2 to 256, value widths other than the nope width,
    pages of 1 to 64 tokens; one row per sequence, f32 and bf16 output, with and without the token-count hint."""
    case = make_mla_case(latent + rope + heads, lens, heads, nope=nope, rope=rope, value=value, latent=latent, block_tokens=page,
                         poison=True)
    want_f, want_b = oracle_mla(case)
    what = f"MLA latent={latent} rope={rope} nope={nope} value={value} heads={heads} lens={lens}"
    got = run_mla(case).cpu().numpy()
    print(what, assert_attention_close(got.reshape(want_f.shape), want_f, what))
    hinted = run_mla(case, total_ctx_tokens=int(sum(lens))).cpu().numpy()
    assert_attention_close(hinted.reshape(want_f.shape), want_f, what + " with the hint")
    got_b = run_mla(case, out_dtype=torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16)
    diff = np.abs(O.bf16_to_f32(got_b).astype(np.float64).reshape(want_f.shape) - O.bf16_to_f32(want_b).reshape(want_f.shape))
    assert (diff <= np.maximum(np.abs(want_f), 2.0 ** -126) * 2.0 ** -7 + 2e-3).all()


def test_other_widths_selected_tokens_and_chunks():
    """The sparse arm (a list of positions per row, with counts) and several query rows per sequence at other widths."""
    rng = np.random.default_rng(8)
    lens = [500, 40, 1300]
    case = make_mla_case(77, lens, 4, nope=64, rope=32, value=64, latent=128, block_tokens=16)
    top_k = 64
    selection = np.stack([rng.permutation(max(l, top_k))[:top_k] % l for l in lens]).astype(np.uint32)
    counts = np.array([64, 64, 37], dtype=np.uint32)
    want, _ = oracle_mla(case, selection=selection, counts=counts)
    got = run_mla(case, selection=selection, counts=counts).cpu().numpy()
    assert_attention_close(got.reshape(want.shape), want, "other widths, selected tokens")
    chunk = make_mla_chunk_case(78, [300, 64, 1000], 7, 3, nope=32, rope=64, value=96, latent=320, block_tokens=64)
    want_f, _ = oracle_mla_chunk(chunk)
    got = run_mla_chunk(chunk).cpu().numpy()
    print("other widths chunk", assert_attention_close(got, want_f, "other widths, seven query rows per sequence"))


@pytest.mark.parametrize("bits,group,scale_dtype,heads,lens", [(32, 0, 0, 16, [300, 1000]), (8, 128, O.SCALE_BF16, 128, [700, 40]),
                                                               (8, 64, O.SCALE_F16, 32, [2500]), (8, 512, O.SCALE_F32, 20, [64, 65]),
                                                               (4, 128, O.SCALE_BF16, 64, [900]), (4, 32, O.SCALE_F16, 8, [33, 200])])
def test_weight_forms_at_the_usual_widths(bits, group, scale_dtype, heads, lens):
    """kv_b as f32, W8A16 and W4A16 at latent 512 + rope 64: the split-KV stage stays on the matrix cores (it never reads
    kv_b), absorb and projection read the codes.  The oracle gets the f32 values the codes stand for."""
    case = make_mla_case(bits * 100 + heads, lens, heads, block_tokens=64)
    set_weight_form(case, bits, group=group or 128, scale_dtype=scale_dtype)
    want, _ = oracle_mla(case)
    got = run_mla(case).cpu().numpy()
    what = f"MLA kv_b {bits}-bit group={group} scales={scale_dtype} heads={heads} lens={lens}"
    print(what, assert_attention_close(got.reshape(want.shape), want, what))


def test_weight_forms_at_other_widths_and_chunks():
    case = make_mla_chunk_case(91, [200, 64], 5, 6, nope=64, rope=32, value=64, latent=256, block_tokens=16)
    set_weight_form(case, 8, group=64, scale_dtype=O.SCALE_BF16)
    want_f, _ = oracle_mla_chunk(case)
    got = run_mla_chunk(case).cpu().numpy()
    print("w8 other widths chunk", assert_attention_close(got, want_f, "W8 kv_b, latent 256, five query rows"))


def test_unsupported_widths_and_forms_are_refused():
    from zllm_amd import capi

    case = make_mla_case(5, [40], 2, nope=32, rope=32, value=32, latent=64)
    for field, value, word in (("latent", 96, "multiple of 64"), ("latent", 1088, "multiple of 64"), ("rope_dim", 33, "even")):
        bad = dict(case)
        bad[field] = value
        with pytest.raises(capi.ZllmAttnError, match=word):
            run_mla(bad)
    bad = dict(case)
    bad["kv_b_form"] = dict(bits=8, data=np.zeros((128, 16), dtype=np.uint32), scales=np.zeros((128, 1), dtype=np.uint16), group=48,
                            scale_dtype=O.SCALE_BF16)
    with pytest.raises(capi.ZllmAttnError, match="group size"):
        run_mla(bad)
    bad["kv_b_form"] = dict(bits=5, data=np.zeros((128, 16), dtype=np.uint32))
    with pytest.raises(capi.ZllmAttnError, match="kv_b_bits"):
        run_mla(bad)

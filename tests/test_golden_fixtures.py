"""The committed fixtures of tests/golden: the oracle must still reproduce them on the CPU (no drift of the checker),
and the HIP kernels must match them on a GPU (bit-exact for the quantizer, attention tolerance otherwise)."""
import os

import numpy as np
import pytest

import oracle as O
from tests.cases import assert_attention_close, to_torch_bf16, upload

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
RULES = (("rocm_mla", O.RULE_ROCM_MLA), ("metal_gqa", O.RULE_METAL_GQA), ("cuda_gqa", O.RULE_CUDA_GQA))


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def test_oracle_reproduces_the_quantizer_fixture():
    g = load("q8g64_quantizer.npz")
    table = np.arange(8, dtype=np.uint32)
    for name, rule in RULES:
        codes = np.zeros_like(g[name + "_codes"])
        scales = np.zeros_like(g[name + "_scales"])
        O.q8g64_append_paged(rule, g["input"], codes, scales, table, 0, 16)
        assert np.array_equal(codes, g[name + "_codes"]), name
        assert np.array_equal(scales.view(np.uint8), g[name + "_scales"].view(np.uint8)), name


def test_oracle_reproduces_the_decode_fixture():
    g = load("gqa_decode_small.npz")
    case = dict(q=O.bf16_to_f32(g["q_bits"]), lens=g["lens"], tables=g["tables"], hq=8, hkv=2, d=128, block_tokens=16,
                scale_dtype=O.SCALE_F16, planes={n: g[n] for n in ("k_codes", "k_scales", "v_codes", "v_scales")})
    from tests.cases import oracle_gqa_decode

    assert np.array_equal(oracle_gqa_decode(case, float(g["score_scale"])), g["expected"])


@pytest.mark.gpu
def test_append_kernel_matches_the_quantizer_fixture_bit_for_bit():
    torch = pytest.importorskip("torch")
    from zllm_amd import ops

    g = load("q8g64_quantizer.npz")
    table = upload(np.arange(8, dtype=np.uint32))
    for name, rule in RULES:
        want_scales = g[name + "_scales"]
        codes = torch.zeros((128, 256), dtype=torch.int8, device="cuda")
        scales = torch.zeros(want_scales.shape, dtype=torch.float32 if want_scales.dtype == np.float32 else torch.int16, device="cuda")
        ops.q8g64_append(upload(g["input"]), codes, scales, table, 0, 16, rule)
        torch.cuda.synchronize()
        assert np.array_equal(codes.cpu().numpy(), g[name + "_codes"]), name
        assert np.array_equal(scales.cpu().numpy().view(np.uint8), want_scales.view(np.uint8)), name


@pytest.mark.gpu
def test_decode_kernel_matches_the_decode_fixture():
    torch = pytest.importorskip("torch")
    from zllm_amd import capi, ops

    g = load("gqa_decode_small.npz")
    out = ops.gqa_decode(to_torch_bf16(g["q_bits"], "cuda"), upload(g["k_codes"]), upload(g["k_scales"]), upload(g["v_codes"]),
                         upload(g["v_scales"]), upload(g["tables"]), upload(g["lens"]), 8, 2, 128, 16, float(g["score_scale"]),
                         int(g["lens"].max()), kv_format=capi.KV_Q8G64, scale_dtype=capi.SCALE_F16)
    torch.cuda.synchronize()
    assert_attention_close(out.cpu().numpy(), g["expected"], "decode fixture")


@pytest.mark.gpu
def test_mla_kernel_matches_the_mla_fixture():
    torch = pytest.importorskip("torch")
    from zllm_amd import ops

    g = load("mla_decode_small.npz")
    out = ops.mla_decode(to_torch_bf16(g["q_bits"], "cuda"), upload(g["kv_b_bits"]), upload(g["codes"]), upload(g["scales"]), upload(g["rope"]),
                         upload(g["tables"]), upload(g["lens"]), 4, 192, 256, 512, 64, 16, int(g["lens"].max()))
    torch.cuda.synchronize()
    assert_attention_close(out.cpu().numpy(), g["expected_f32"].reshape(out.shape), "MLA fixture")


@pytest.mark.gpu
def test_mla_kernel_matches_the_selected_token_fixture():
    torch = pytest.importorskip("torch")
    from zllm_amd import ops

    g = load("mla_decode_small.npz")
    out = ops.mla_decode(to_torch_bf16(g["q_bits"], "cuda"), upload(g["kv_b_bits"]), upload(g["codes"]), upload(g["scales"]), upload(g["rope"]),
                         upload(g["tables"]), upload(g["lens"]), 4, 192, 256, 512, 64, 16, int(g["lens"].max()), selection=upload(g["selection"]))
    torch.cuda.synchronize()
    assert_attention_close(out.cpu().numpy(), g["expected_selected_f32"].reshape(out.shape), "MLA selected-token fixture")


@pytest.mark.gpu
def test_prologue_kernel_matches_the_prologue_fixture_bit_for_bit():
    torch = pytest.importorskip("torch")
    from zllm_amd import ops

    g = load("gqa_prologue_small.npz")
    dev = {n: torch.zeros(g[n].shape, dtype=torch.int8 if "codes" in n else torch.int16, device="cuda")
           for n in ("k_codes", "k_scales", "v_codes", "v_scales")}
    q_out = ops.gqa_prologue(upload(g["q"]), upload(g["k"]), upload(g["v"]), upload(g["q_norm"]), upload(g["k_norm"]), upload(g["cos"]),
                             upload(g["sin"]), dev["k_codes"], dev["k_scales"], dev["v_codes"], dev["v_scales"], upload(g["table"]),
                             int(g["position"]), 4, 2, 128, int(g["rotary"]), 16, eps=float(g["eps"]), weight_offset=1.0)
    torch.cuda.synchronize()
    assert np.array_equal(q_out.cpu().numpy().view(np.uint32), g["expected_q"].view(np.uint32))
    for n in dev:
        assert np.array_equal(dev[n].cpu().numpy().view(g[n].dtype), g[n]), n


def test_oracle_reproduces_the_prologue_fixture():
    g = load("gqa_prologue_small.npz")
    rc, normed = O.rmsnorm_heads(g["q"], 4, 128, g["q_norm"], float(g["eps"]), 1.0)
    assert rc == 0
    rc, rotated = O.rope_apply(normed, 4, int(g["rotary"]), int(g["position"]), g["cos"], g["sin"], layout=0, placement=0)
    assert rc == 0
    assert np.array_equal(rotated.view(np.uint32), g["expected_q"].view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("window", [0, 64])
def test_prefill_kernel_matches_the_prefill_fixture(window):
    torch = pytest.importorskip("torch")
    from zllm_amd import capi, ops

    g = load("gqa_prefill_small.npz")
    out = ops.gqa_prefill_chunk(to_torch_bf16(g["q_bits"], "cuda"), upload(g["k_codes"]), upload(g["k_scales"]), upload(g["v_codes"]),
                                upload(g["v_scales"]), upload(g["table"]), int(g["prefix"]), 8, 2, 128, 16, float(g["score_scale"]),
                                window=window, scale_dtype=capi.SCALE_F16)
    torch.cuda.synchronize()
    assert_attention_close(out.cpu().numpy(), g[f"expected_window_{window}"], f"prefill fixture, window {window}")


def test_oracle_reproduces_the_block_attention_fixture():
    g = load("block_attention_small.npz")
    kd = O.gather_dequant_rows(O.FMT_Q8, g["k_codes"], g["k_scales"], O.SCALE_F16, g["table"], 16, 0, 100, 256)
    vd = O.gather_dequant_rows(O.FMT_Q8, g["v_codes"], g["v_scales"], O.SCALE_F16, g["table"], 16, 0, 100, 256)
    for name in ("varlen", "free"):
        rc, out = O.block_attention(O.bf16_to_f32(g["q_bits"]), kd, vd, 8, 2, 128, float(g["score_scale"]), g[f"visible_{name}"])
        assert rc == 0
        assert np.array_equal(out, g[f"expected_{name}"]), name


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["varlen", "free"])
def test_prefill_kernel_matches_the_block_attention_fixture(name):
    torch = pytest.importorskip("torch")
    from zllm_amd import ops

    g = load("block_attention_small.npz")
    visible = g[f"visible_{name}"]
    out = ops.gqa_prefill_chunk(to_torch_bf16(g["q_bits"], "cuda"), upload(g["k_codes"]), upload(g["k_scales"]), upload(g["v_codes"]),
                                upload(g["v_scales"]), upload(g["table"]), 100 - 40, 8, 2, 128, 16, float(g["score_scale"]),
                                visible_starts=upload(visible[:, 0].copy()), visible_ends=upload(visible[:, 1].copy()))
    torch.cuda.synchronize()
    assert_attention_close(out.cpu().numpy(), g[f"expected_{name}"], f"block attention fixture ({name})")


def test_oracle_reproduces_the_other_widths_mla_fixture():
    g = load("mla_other_widths_small.npz")
    spec = O.MlaSpec(128, 32, 3 * 96, 3 * 128, 3)
    for b, l in enumerate(g["lens"]):
        l = int(l)
        codes = O.gather_rows_bytes(g["codes"], g["tables"][b], 16, 0, l, 128)
        scales = O.gather_rows_bytes(g["scales"], g["tables"][b], 16, 0, l, 4).view(np.uint16)
        rope = O.gather_rows_bytes(g["rope"], g["tables"][b], 16, 0, l, 64).view(np.uint16)
        rc, _, out, _ = O.mla_absorbed_q8_history(spec, g["q_bits"][b:b + 1], 1, l - 1, codes, scales, 64, rope, l, g["kv_b_values"])
        assert rc == 0
        assert np.array_equal(out.reshape(-1), g["expected_f32"][b].reshape(-1))
    # the stored values are what the stored codes stand for: (code - 128) x bf16 scale of the row's 64-column group
    words, scale_bits = g["kv_b_words"], g["kv_b_scales"]
    codes = np.stack([(words >> np.uint32(8 * i)) & np.uint32(255) for i in range(4)], axis=2).reshape(words.shape[0], -1).astype(np.int32) - 128
    values = codes.astype(np.float32) * np.repeat(O.bf16_to_f32(scale_bits), 64, axis=1)
    assert np.array_equal(values, g["kv_b_values"])


@pytest.mark.gpu
def test_mla_kernels_match_the_other_widths_fixture():
    torch = pytest.importorskip("torch")
    from zllm_amd import capi, ops

    g = load("mla_other_widths_small.npz")
    out = ops.mla_decode(to_torch_bf16(g["q_bits"], "cuda"), upload(g["kv_b_words"]), upload(g["codes"]), upload(g["scales"]), upload(g["rope"]),
                         upload(g["tables"]), upload(g["lens"]), 3, 96, 128, 128, 32, 16, int(g["lens"].max()), kv_b_bits=8,
                         kv_b_scales=upload(g["kv_b_scales"]), kv_b_group=64, kv_b_scale_dtype=capi.SCALE_BF16)
    torch.cuda.synchronize()
    assert_attention_close(out.cpu().numpy(), g["expected_f32"].reshape(out.shape), "MLA fixture at latent 128 + rope 32 with W8 kv_b")

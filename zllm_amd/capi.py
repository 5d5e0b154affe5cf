"""ctypes view of include/zllm_attn.h.

Thin by design: the structures mirror the header field by field and every call goes
straight to the C ABI of ``libzllm_attn.so``.  There is no CPU fallback: if the HIP
library has not been built, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libzllm_attn.so")

SCALE_BF16, SCALE_F16, SCALE_F32 = 0, 1, 2
DTYPE_F32, DTYPE_BF16, DTYPE_F16 = 0, 1, 2
KV_Q8G64, KV_F16 = 0, 1
QUANT_ROCM_MLA, QUANT_METAL_GQA, QUANT_CUDA_GQA = 0, 1, 2
ROTARY_INTERLEAVED, ROTARY_SPLIT_HALF = 0, 1
STAGE_ALL, STAGE_PARTIAL, STAGE_MERGE = 0, 1, 2
MLA_ABSORB, MLA_PARTIAL, MLA_MERGE, MLA_PROJECT = 1, 2, 4, 8
MLA_WIDE_TILES = 16  # OR-ed into stage_mask: the split-KV partial on its second kernel where the call allows it

_u32, _u64, _f32, _int, _ptr = C.c_uint32, C.c_uint64, C.c_float, C.c_int, C.c_void_p


class Q8AppendArgs(C.Structure):
    _fields_ = [("src", _ptr), ("codes", _ptr), ("scales", _ptr), ("table", _ptr), ("positions", _ptr),
                ("position", _u32), ("rows", _u32), ("cols", _u32), ("block_tokens", _u32), ("ring_capacity", _u32),
                ("src_dtype", _int), ("rule", _int)]


class GqaPrologueArgs(C.Structure):
    _fields_ = [("q", _ptr), ("k", _ptr), ("v", _ptr), ("q_norm", _ptr), ("k_norm", _ptr), ("cosine", _ptr), ("sine", _ptr),
                ("q_out", _ptr), ("k_codes", _ptr), ("k_scales", _ptr), ("v_codes", _ptr), ("v_scales", _ptr), ("table", _ptr),
                ("positions", _ptr), ("rows", _u32), ("num_heads", _u32), ("num_kv_heads", _u32), ("head_dim", _u32),
                ("rotary_dim", _u32), ("rope_table_rows", _u32), ("position", _u32), ("block_tokens", _u32),
                ("ring_capacity", _u32), ("eps", C.c_float), ("weight_offset", C.c_float), ("src_dtype", _int),
                ("q_out_dtype", _int), ("rule", _int), ("split_half", _int)]


class HalfAppendArgs(C.Structure):
    _fields_ = [("src", _ptr), ("cache", _ptr), ("table", _ptr), ("position", _u32), ("rows", _u32), ("cols", _u32),
                ("block_tokens", _u32), ("ring_capacity", _u32), ("src_dtype", _int), ("dst_dtype", _int)]


class MlaAppendArgs(C.Structure):
    _fields_ = [("latent", _ptr), ("k_rope", _ptr), ("cosine", _ptr), ("sine", _ptr), ("latent_codes", _ptr),
                ("latent_scales", _ptr), ("rope_cache", _ptr), ("table", _ptr), ("positions", _ptr),
                ("position", _u32), ("rope_position", _u32), ("rows", _u32), ("latent_cols", _u32),
                ("rope_cols", _u32), ("rotary_dim", _u32), ("rotary_layout", _int), ("block_tokens", _u32)]


class GatherArgs(C.Structure):
    _fields_ = [("plane", _ptr), ("out", _ptr), ("table", _ptr), ("first", _u32), ("count", _u32),
                ("row_bytes", _u32), ("block_tokens", _u32), ("ring_capacity", _u32)]


class ScatterArgs(C.Structure):
    _fields_ = [("plane", _ptr), ("in_", _ptr), ("table", _ptr), ("first", _u32), ("count", _u32), ("row_bytes", _u32),
                ("block_tokens", _u32), ("ring_capacity", _u32)]


class MlaLayerRecord(C.Structure):
    _fields_ = [("rows", _u64), ("ownership", _u32), ("latent_cols", _u64), ("rope_cols", _u64), ("latent_group_size", _u64),
                ("latent", _ptr), ("latent_bytes", _u64), ("latent_scales", _ptr), ("latent_scales_bytes", _u64),
                ("rope", _ptr), ("rope_bytes", _u64)]


class GqaDecodeArgs(C.Structure):
    _fields_ = [("q", _ptr), ("k_plane", _ptr), ("k_scales", _ptr), ("v_plane", _ptr), ("v_scales", _ptr),
                ("tables", _ptr), ("kv_lens", _ptr), ("first_visible", _ptr), ("out", _ptr), ("workspace", _ptr),
                ("workspace_bytes", _u64), ("batch", _u32), ("num_heads", _u32), ("num_kv_heads", _u32),
                ("head_dim", _u32), ("table_stride", _u32), ("max_kv_len", _u32), ("total_kv_tokens", _u32),
                ("block_tokens", _u32), ("ring_capacity", _u32), ("score_scale", _f32), ("softcap", _f32), ("kv_format", _int),
                ("scale_dtype", _int), ("q_dtype", _int), ("stages", _u32), ("gate", _ptr), ("gate_cols", _u32), ("gate_dtype", _int)]


class GqaPrefillArgs(C.Structure):
    _fields_ = [("q", _ptr), ("k_plane", _ptr), ("k_scales", _ptr), ("v_plane", _ptr), ("v_scales", _ptr),
                ("table", _ptr), ("out", _ptr), ("workspace", _ptr), ("workspace_bytes", _u64), ("rows", _u32),
                ("position", _u32), ("window", _u32), ("num_heads", _u32), ("num_kv_heads", _u32), ("head_dim", _u32),
                ("block_tokens", _u32), ("score_scale", _f32), ("softcap", _f32), ("kv_format", _int),
                ("scale_dtype", _int), ("q_dtype", _int), ("out_dtype", _int), ("gate", _ptr), ("gate_cols", _u32),
                ("gate_dtype", _int), ("visible_ends", _ptr), ("table_stride", _u32), ("visible_starts", _ptr)]


class SplitRecordLayout(C.Structure):
    _fields_ = [("record_rows", _u64), ("partial_offset", _u64), ("stats_offset", _u64), ("first_rows_offset", _u64),
                ("chunk_tokens", _u32), ("max_chunks", _u32), ("dense", _u32)]


class MlaDecodeArgs(C.Structure):
    _fields_ = [("q", _ptr), ("kv_b", _ptr), ("latent_codes", _ptr), ("latent_scales", _ptr), ("rope_cache", _ptr),
                ("tables", _ptr), ("ctx_lens", _ptr), ("out", _ptr), ("workspace", _ptr), ("workspace_bytes", _u64),
                ("batch", _u32), ("heads", _u32), ("q_head_dim", _u32), ("kv_head_dim", _u32), ("latent_dim", _u32),
                ("rope_dim", _u32), ("table_stride", _u32), ("max_ctx_len", _u32), ("block_tokens", _u32),
                ("q_dtype", _int), ("out_dtype", _int), ("out_compact", _int), ("stage_mask", _u32),
                ("top_k", _u32), ("selection", _ptr), ("selection_counts", _ptr), ("query_rows", _u32),
                ("total_ctx_tokens", _u32), ("kv_b_scales", _ptr), ("kv_b_bits", _u32), ("kv_b_group", _u32),
                ("kv_b_scale_dtype", _int)]


# every symbol include/zllm_attn.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "zllm_attn_init": (_int, [_int, C.POINTER(_int)]),
    "zllm_attn_last_error": (C.c_char_p, []),
    "zllm_attn_key_range": (None, [_u64, _u64, _u64, C.POINTER(_u64), C.POINTER(_u64)]),
    "zllm_kv_bytes_per_token": (_u64, [_int, _u64, _u64, _u64]),
    "zllm_kv_layout_offsets": (_u64, [_int, _u64, _u64, _u64, _u64, _u64, _u64, C.POINTER(_u64)]),
    "zllm_kv_ring_write_plan": (_int, [_u64, _u64, _u64, _u64, C.POINTER(_u64)]),
    "zllm_attn_q8g64_append": (_int, [C.POINTER(Q8AppendArgs), _ptr]),
    "zllm_attn_half_append": (_int, [C.POINTER(HalfAppendArgs), _ptr]),
    "zllm_attn_gqa_prologue": (_int, [C.POINTER(GqaPrologueArgs), _ptr]),
    "zllm_attn_mla_append": (_int, [C.POINTER(MlaAppendArgs), _ptr]),
    "zllm_attn_gather_rows": (_int, [C.POINTER(GatherArgs), _ptr]),
    "zllm_attn_scatter_rows": (_int, [C.POINTER(ScatterArgs), _ptr]),
    "zllm_kv_mla_layer_wire_bytes": (_u64, [C.POINTER(MlaLayerRecord)]),
    "zllm_kv_mla_layer_write": (_int, [C.POINTER(MlaLayerRecord), _ptr, _u64, C.POINTER(_u64)]),
    "zllm_kv_mla_layer_read": (_int, [_ptr, _u64, C.POINTER(MlaLayerRecord), C.POINTER(_u64)]),
    "zllm_attn_gqa_decode_workspace_bytes": (_u64, [C.POINTER(GqaDecodeArgs)]),
    "zllm_attn_gqa_decode_split_plan": (_int, [C.POINTER(GqaDecodeArgs), C.POINTER(_u32), C.POINTER(_u32)]),
    "zllm_attn_gqa_decode_record_layout": (_int, [C.POINTER(GqaDecodeArgs), C.POINTER(SplitRecordLayout)]),
    "zllm_attn_gqa_decode": (_int, [C.POINTER(GqaDecodeArgs), _ptr]),
    "zllm_attn_static_scratch_bytes": (_u64, []),
    "zllm_attn_gqa_decode_static": (_int, [C.POINTER(GqaDecodeArgs), _ptr]),
    "zllm_attn_gqa_prefill_workspace_bytes": (_u64, [C.POINTER(GqaPrefillArgs)]),
    "zllm_attn_gqa_prefill_chunk": (_int, [C.POINTER(GqaPrefillArgs), _ptr]),
    "zllm_attn_mla_decode_workspace_bytes": (_u64, [C.POINTER(MlaDecodeArgs)]),
    "zllm_attn_mla_decode_record_layout": (_int, [C.POINTER(MlaDecodeArgs), C.POINTER(SplitRecordLayout)]),
    "zllm_attn_mla_decode": (_int, [C.POINTER(MlaDecodeArgs), _ptr]),
}

_lib = None


class ZllmAttnError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"zllm_attn error {code}: {message}")
        self.code = code


def load():
    """Load libzllm_attn.so and bind every declared symbol.  Raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `python -m zllm_amd.build` (hipcc, gfx950). "
                "There is no CPU fallback for the attention path.")
        lib = C.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def last_error() -> str:
    return load().zllm_attn_last_error().decode("utf-8", "replace")


def check(code: int) -> None:
    if code != 0:
        raise ZllmAttnError(code, last_error())

"""ctypes binding for the CPU oracle (oracle/zllm_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and
by the ``cpu_baseline`` leg of ``bench.py`` as the checker.  The product package
(``zllm_amd``) never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libzllm_oracle.so")

RULE_ROCM_MLA = 0   # bf16 scale, codes from the rounded scale
RULE_METAL_GQA = 1  # f16 scale, codes from the unrounded scale
RULE_CUDA_GQA = 2   # f32 scale
SCALE_BF16, SCALE_F16, SCALE_F32 = 0, 1, 2
FMT_Q8, FMT_F16, FMT_BF16 = 0, 1, 2


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a few seconds)."""
    src = os.path.join(_HERE, "zllm_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libzllm_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class MlaSpec(C.Structure):
    _fields_ = [
        ("kv_lora_rank", C.c_uint64),
        ("qk_rope_head_dim", C.c_uint64),
        ("q_projection_size", C.c_uint64),
        ("kv_projection_size", C.c_uint64),
        ("num_heads", C.c_uint64),
    ]

    @property
    def q_head_dim(self):
        return self.q_projection_size // self.num_heads

    @property
    def nope(self):
        return self.q_head_dim - self.qk_rope_head_dim

    @property
    def kv_head_dim(self):
        return self.kv_projection_size // self.num_heads

    @property
    def value_dim(self):
        return self.kv_head_dim - self.nope


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.zo_bf16_to_f32.restype = C.c_float
        _lib.zo_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.zo_f32_to_bf16.restype = C.c_uint16
        _lib.zo_f32_to_bf16.argtypes = [C.c_float]
        _lib.zo_f16_to_f32.restype = C.c_float
        _lib.zo_f16_to_f32.argtypes = [C.c_uint16]
        _lib.zo_f32_to_f16.restype = C.c_uint16
        _lib.zo_f32_to_f16.argtypes = [C.c_float]
        _lib.zo_paged_row.restype = C.c_uint64
        _lib.zo_paged_row.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32]
        _lib.zo_cache_capacity.restype = C.c_uint64
        _lib.zo_cache_capacity.argtypes = [C.c_uint64, C.c_uint64]
        _lib.zo_bytes_per_token.restype = C.c_uint64
        _lib.zo_bytes_per_token.argtypes = [C.c_int, C.c_uint64, C.c_uint64, C.c_uint64]
        _lib.zo_layout_offsets.restype = C.c_uint64
        _lib.zo_layout_offsets.argtypes = [C.c_int] + [C.c_uint64] * 6 + [C.c_void_p]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# --------------------------------------------------------------------------- conversions
def bf16_to_f32(bits):
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x):
    """zllm_f32_to_bf16 (hiprtc.rs:69-75), vectorised; identical to zo_f32_to_bf16."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounding = np.uint32(0x7FFF) + ((bits >> 16) & np.uint32(1))
    return ((bits + rounding) >> 16).astype(np.uint16)


def f16_to_f32(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)


# --------------------------------------------------------------------------- integer helpers
def key_range(window, query_position, key_end):
    s, e = C.c_uint64(), C.c_uint64()
    lib().zo_key_range(C.c_uint64(window), C.c_uint64(query_position), C.c_uint64(key_end), C.byref(s), C.byref(e))
    return s.value, e.value


def key_range_with_visible_end(window, query_position, key_end, visible_end):
    s, e = C.c_uint64(), C.c_uint64()
    lib().zo_key_range_with_visible_end(C.c_uint64(window), C.c_uint64(query_position), C.c_uint64(key_end),
                                        C.c_uint64(visible_end), C.byref(s), C.byref(e))
    return s.value, e.value


def paged_row(table, token, block_size):
    t = None if table is None else _c(table, np.uint32)
    return lib().zo_paged_row(_p(t), token, block_size)


def bytes_per_token(kind, a, b, group):
    return lib().zo_bytes_per_token(kind, a, b, group)


def layout_offsets(kind, a, b, group, layer_count, capacity, layer):
    out = np.zeros(5, dtype=np.uint64)
    total = lib().zo_layout_offsets(kind, a, b, group, layer_count, capacity, layer, _p(out))
    return total, out


def ring_write_plan(capacity, max_sequence_len, position, count):
    out = np.zeros(6, dtype=np.uint64)
    rc = lib().zo_ring_write_plan(C.c_uint64(capacity), C.c_uint64(max_sequence_len), C.c_uint64(position),
                                  C.c_uint64(count), _p(out))
    if rc != 0:
        return None
    return dict(zip(["end", "source_start", "token_count", "first_slot", "first_count", "second_count"],
                    [int(v) for v in out]))


# --------------------------------------------------------------------------- quantize / gather
def q8g64_append_paged(rule, x, codes, scales, table, position, block_size, group=64, ring_capacity=0):
    """Quantize rows of x [T, cols] into the planes in place."""
    x = _c(x, np.float32)
    rows, cols = x.shape
    t = None if table is None else _c(table, np.uint32)
    rc = lib().zo_q8g64_append_paged(C.c_int(rule), _p(x), _p(codes), _p(scales), _p(t), C.c_uint64(position),
                                     C.c_uint64(rows), C.c_uint64(cols), C.c_uint64(group), C.c_uint32(block_size),
                                     C.c_uint64(ring_capacity))
    assert rc == 0
    return rc


def half_append_paged(dtype, x, cache, table, position, block_size, ring_capacity=0):
    x = _c(x, np.float32)
    rows, cols = x.shape
    t = None if table is None else _c(table, np.uint32)
    rc = lib().zo_half_append_paged(C.c_int(dtype), _p(x), _p(cache), _p(t), C.c_uint64(position), C.c_uint64(rows),
                                    C.c_uint64(cols), C.c_uint32(block_size), C.c_uint64(ring_capacity))
    assert rc == 0


def gather_dequant_rows(fmt, plane, scales, scale_dtype, table, block_size, first, count, cols, group=64,
                        ring_capacity=0):
    out = np.empty((count, cols), dtype=np.float32)
    t = None if table is None else _c(table, np.uint32)
    rc = lib().zo_gather_dequant_rows(C.c_int(fmt), _p(plane), _p(scales), C.c_int(scale_dtype), _p(t),
                                      C.c_uint32(block_size), C.c_uint64(ring_capacity), C.c_uint64(first),
                                      C.c_uint64(count), C.c_uint64(cols), C.c_uint64(group), _p(out))
    assert rc == 0
    return out


def gather_rows_bytes(plane, table, block_size, first, count, row_bytes, ring_capacity=0):
    out = np.empty((count, row_bytes), dtype=np.uint8)
    t = None if table is None else _c(table, np.uint32)
    plane = plane.view(np.uint8)
    rc = lib().zo_gather_rows_bytes(_p(plane), _p(t), C.c_uint32(block_size), C.c_uint64(ring_capacity),
                                    C.c_uint64(first), C.c_uint64(count), C.c_uint64(row_bytes), _p(out))
    assert rc == 0
    return out


# --------------------------------------------------------------------------- GQA
def gqa_prefill_at_visible(query, key, value, kv_start, kv_end, position, num_heads, num_kv_heads, head_dim,
                           window=0, score_scale=1.0, softcap=0.0, visible_ends=None):
    """O3: query [T, Hq*d] f32; key/value dense f32 rows [kv_start, kv_end)."""
    query = _c(query, np.float32).reshape(-1, num_heads * head_dim)
    key = _c(key, np.float32)
    value = _c(value, np.float32)
    tokens = query.shape[0]
    out = np.empty_like(query)
    ve = None if visible_ends is None else _c(visible_ends, np.uint32)
    rc = lib().zo_gqa_prefill_at_visible_f32(_p(query), _p(key), _p(value), C.c_uint64(tokens), C.c_uint64(kv_start),
                                             C.c_uint64(kv_end), C.c_uint64(position), C.c_uint64(num_heads),
                                             C.c_uint64(num_kv_heads), C.c_uint64(head_dim), C.c_uint64(window),
                                             C.c_float(score_scale), C.c_float(softcap), _p(ve), _p(out))
    return rc, out


def gqa_decode_q8_direct(query, k_codes, k_scales, v_codes, v_scales, scale_dtype, first, length, num_heads, num_kv_heads, head_dim,
                         score_scale, softcap=0.0):
    """Decode attention of one sequence straight over dense Q8g64 rows (no f32 K/V): query [Hq*d] f32 -> [Hq*d] f32."""
    query = _c(query, np.float32).reshape(-1)
    k_codes = np.ascontiguousarray(k_codes).view(np.int8)
    v_codes = np.ascontiguousarray(v_codes).view(np.int8)
    k_scales = np.ascontiguousarray(k_scales)
    v_scales = np.ascontiguousarray(v_scales)
    out = np.empty(num_heads * head_dim, dtype=np.float32)
    rc = lib().zo_gqa_decode_q8_direct(_p(query), _p(k_codes), _p(k_scales), _p(v_codes), _p(v_scales), C.c_int(scale_dtype),
                                       C.c_uint64(first), C.c_uint64(length), C.c_uint64(num_heads), C.c_uint64(num_kv_heads),
                                       C.c_uint64(head_dim), C.c_float(score_scale), C.c_float(softcap), _p(out))
    return rc, out


def block_attention(query, key, value, num_heads, num_kv_heads, head_dim, score_scale, visible):
    query = _c(query, np.float32).reshape(-1, num_heads * head_dim)
    key = _c(key, np.float32).reshape(-1, num_kv_heads * head_dim)
    value = _c(value, np.float32).reshape(-1, num_kv_heads * head_dim)
    visible = _c(visible, np.uint32)
    out = np.empty_like(query)
    rc = lib().zo_block_attention_f32(_p(query), _p(key), _p(value), C.c_uint64(query.shape[0]),
                                      C.c_uint64(key.shape[0]), C.c_uint64(num_heads), C.c_uint64(num_kv_heads),
                                      C.c_uint64(head_dim), C.c_float(score_scale), _p(visible), _p(out))
    return rc, out


def rope_apply(data, head_count, rotary_dim, position, cos, sin, layout=0, placement=0):
    data = np.array(data, dtype=np.float32, copy=True)
    if data.ndim == 1:
        data = data[None, :]
    cos = _c(cos, np.float32)
    sin = _c(sin, np.float32)
    rc = lib().zo_rope_apply_f32(_p(data), C.c_uint64(data.shape[0]), C.c_uint64(data.shape[1]),
                                 C.c_uint64(head_count), C.c_uint64(rotary_dim), C.c_uint64(position), _p(cos),
                                 _p(sin), C.c_uint64(min(cos.size, sin.size)), C.c_int(layout), C.c_int(placement))
    return rc, data


def rmsnorm_heads(x, head_count, head_dim, weight, eps, weight_offset=0.0):
    """Per-head RMSNorm (weight_offset 1.0 = Gemma form).  x [rows, head_count * head_dim]."""
    x = _c(x, np.float32)
    rows = x.size // (head_count * head_dim)
    w = None if weight is None else _c(weight, np.float32)
    out = np.zeros_like(x)
    rc = lib().zo_rmsnorm_heads_f32(_p(x), C.c_uint64(rows), C.c_uint64(head_count), C.c_uint64(head_dim), _p(w),
                                    C.c_float(eps), C.c_float(weight_offset), _p(out))
    return rc, out


def sigmoid_gate(x, gate):
    x = _c(x, np.float32)
    gate = _c(gate, np.float32)
    rows = x.shape[0]
    out = np.zeros_like(x)
    rc = lib().zo_sigmoid_gate_f32(_p(x), _p(gate), C.c_uint64(rows), C.c_uint64(x.size // rows),
                                   C.c_uint64(gate.size // rows), _p(out))
    return rc, out


# --------------------------------------------------------------------------- MLA
def mla_reference_attention(query, projected_kv, rope_cache, rope_indices, spec: MlaSpec):
    query = _c(query, np.float32)
    projected_kv = _c(projected_kv, np.float32)
    rope_cache = _c(rope_cache, np.float32)
    idx = _c(rope_indices, np.uint64)
    rope_rows = rope_cache.size // max(1, spec.qk_rope_head_dim)
    out = np.zeros(spec.q_projection_size, dtype=np.float32)
    rc = lib().zo_mla_reference_attention(_p(query), _p(projected_kv), _p(rope_cache), C.c_uint64(rope_rows), _p(idx),
                                          C.c_uint64(idx.size), C.byref(spec), _p(out))
    return rc, out


def mla_selected_bf16_history(spec, query, query_rows, query_start, projected_kv, rope, history_rows, selection=None,
                              width=0):
    query = _c(query, np.uint16)
    projected_kv = _c(projected_kv, np.uint16)
    rope = _c(rope, np.uint16)
    sel = None if selection is None else _c(selection, np.uint32)
    out = np.zeros(query_rows * spec.num_heads * spec.value_dim, dtype=np.uint16)
    rc = lib().zo_mla_selected_bf16_history(C.byref(spec), _p(query), C.c_uint64(query_rows), C.c_uint64(query_start),
                                            _p(projected_kv), _p(rope), C.c_uint64(history_rows), _p(sel),
                                            C.c_uint64(width), _p(out))
    return rc, out


def mla_absorbed_q8_history(spec, query_bf16, query_rows, query_start, codes, scales_bf16, group, rope_bf16,
                            history_rows, kv_b, selection=None, width=0, want_weighted=False):
    """O7.  Returns (rc, out_bf16 bits, out_f32, weighted_f32 or None)."""
    query_bf16 = _c(query_bf16, np.uint16)
    codes = _c(codes, np.uint8) if codes.dtype != np.int8 else np.ascontiguousarray(codes).view(np.uint8)
    scales_bf16 = _c(scales_bf16, np.uint16)
    rope_bf16 = _c(rope_bf16, np.uint16)
    kv_b = _c(kv_b, np.float32)
    sel = None if selection is None else _c(selection, np.uint32)
    n = query_rows * spec.num_heads * spec.value_dim
    out_b = np.zeros(n, dtype=np.uint16)
    out_f = np.zeros(n, dtype=np.float32)
    weighted = np.zeros(query_rows * spec.num_heads * spec.kv_lora_rank, dtype=np.float32) if want_weighted else None
    rc = lib().zo_mla_absorbed_q8_history(C.byref(spec), _p(query_bf16), C.c_uint64(query_rows),
                                          C.c_uint64(query_start), _p(codes), _p(scales_bf16), C.c_uint64(group),
                                          _p(rope_bf16), C.c_uint64(history_rows), _p(kv_b), _p(sel),
                                          C.c_uint64(width), _p(out_b), _p(out_f), _p(weighted))
    return rc, out_b, out_f, weighted


def set_threads(n: int = 0) -> int:
    return lib().zo_set_threads(C.c_int(n))

"""Torch-tensor plumbing over the C ABI (device memory + the current HIP stream only).

Every function builds the argument block of include/zllm_attn.h from tensors and calls
the library; no arithmetic happens here.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import capi

_DTYPE = {torch.float32: capi.DTYPE_F32, torch.bfloat16: capi.DTYPE_BF16, torch.float16: capi.DTYPE_F16}


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, name):
    if t is not None and (not t.is_cuda or not t.is_contiguous()):
        raise ValueError(f"{name} must be a contiguous device tensor")
    return t


def init(device: int = 0) -> int:
    cu = C.c_int(0)
    capi.check(capi.load().zllm_attn_init(device, C.byref(cu)))
    return cu.value


def q8g64_append(src, codes, scales, table, position, block_tokens, rule, ring_capacity=0, positions=None):
    """Quantize rows of `src` [T, cols] into the paged planes (zllm_attn_q8g64_append)."""
    _dev(src, "src"), _dev(codes, "codes"), _dev(scales, "scales"), _dev(table, "table")
    args = capi.Q8AppendArgs(_ptr(src), _ptr(codes), _ptr(scales), _ptr(table), _ptr(positions), position,
                             src.shape[0], src.shape[1], block_tokens, ring_capacity, _DTYPE[src.dtype], rule)
    capi.check(capi.load().zllm_attn_q8g64_append(C.byref(args), _stream()))


def gqa_prologue(q, k, v, q_norm, k_norm, cos, sin, k_codes, k_scales, v_codes, v_scales, table, position, num_heads,
                 num_kv_heads, head_dim, rotary_dim, block_tokens, eps=1e-6, weight_offset=1.0, rule=capi.QUANT_METAL_GQA,
                 split_half=True, q_out_dtype=torch.float32, ring_capacity=0, positions=None):
    """Per-head RMSNorm + RoPE of Q and K, Q out as a tensor, K and V quantized into the pages (zllm_attn_gqa_prologue)."""
    rows = q.shape[0]
    q_out = torch.empty((rows, num_heads * head_dim), dtype=q_out_dtype, device=q.device)
    args = capi.GqaPrologueArgs()
    args.q, args.k, args.v = _ptr(q), _ptr(k), _ptr(v)
    args.q_norm, args.k_norm, args.cosine, args.sine = _ptr(q_norm), _ptr(k_norm), _ptr(cos), _ptr(sin)
    args.q_out, args.k_codes, args.k_scales = _ptr(q_out), _ptr(k_codes), _ptr(k_scales)
    args.v_codes, args.v_scales, args.table, args.positions = _ptr(v_codes), _ptr(v_scales), _ptr(table), _ptr(positions)
    args.rows, args.num_heads, args.num_kv_heads, args.head_dim = rows, num_heads, num_kv_heads, head_dim
    args.rotary_dim = rotary_dim
    args.rope_table_rows = 0 if cos is None else cos.shape[0]
    args.position, args.block_tokens, args.ring_capacity = position, block_tokens, ring_capacity
    args.eps, args.weight_offset = eps, weight_offset
    args.src_dtype, args.q_out_dtype, args.rule, args.split_half = _DTYPE[q.dtype], _DTYPE[q_out_dtype], rule, int(split_half)
    capi.check(capi.load().zllm_attn_gqa_prologue(C.byref(args), _stream()))
    return q_out


def half_append(src, cache, table, position, block_tokens, ring_capacity=0):
    _dev(src, "src"), _dev(cache, "cache"), _dev(table, "table")
    dst = capi.DTYPE_BF16 if cache.dtype == torch.bfloat16 else capi.DTYPE_F16
    args = capi.HalfAppendArgs(_ptr(src), _ptr(cache), _ptr(table), position, src.shape[0], src.shape[1],
                               block_tokens, ring_capacity, _DTYPE[src.dtype], dst)
    capi.check(capi.load().zllm_attn_half_append(C.byref(args), _stream()))


def mla_append(latent, k_rope, latent_codes, latent_scales, rope_cache, table, position, block_tokens, cos=None,
               sin=None, rotary_dim=0, rotary_layout=capi.ROTARY_SPLIT_HALF, rope_position=0, positions=None):
    for name, t in (("latent", latent), ("k_rope", k_rope), ("latent_codes", latent_codes),
                    ("latent_scales", latent_scales), ("rope_cache", rope_cache)):
        _dev(t, name)
    args = capi.MlaAppendArgs(_ptr(latent), _ptr(k_rope), _ptr(cos), _ptr(sin), _ptr(latent_codes),
                              _ptr(latent_scales), _ptr(rope_cache), _ptr(table), _ptr(positions), position,
                              rope_position, latent.shape[0], latent.shape[1], k_rope.shape[1], rotary_dim,
                              rotary_layout, block_tokens)
    capi.check(capi.load().zllm_attn_mla_append(C.byref(args), _stream()))


def gather_rows(plane, table, first, count, row_bytes, block_tokens, ring_capacity=0):
    out = torch.empty((count, row_bytes), dtype=torch.uint8, device=plane.device)
    args = capi.GatherArgs(_ptr(plane), _ptr(out), _ptr(table), first, count, row_bytes, block_tokens, ring_capacity)
    capi.check(capi.load().zllm_attn_gather_rows(C.byref(args), _stream()))
    return out


def scatter_rows(plane, rows, table, first, block_tokens, ring_capacity=0):
    """plane[paged_row(first + r)] = rows[r] (zllm_attn_scatter_rows); `rows` is a dense [count, row_bytes] uint8 tensor."""
    args = capi.ScatterArgs(_ptr(plane), _ptr(rows), _ptr(table), first, rows.shape[0], rows.shape[1], block_tokens, ring_capacity)
    capi.check(capi.load().zllm_attn_scatter_rows(C.byref(args), _stream()))


def gqa_decode_args(q, k_plane, k_scales, v_plane, v_scales, tables, kv_lens, num_heads, num_kv_heads, head_dim,
                    block_tokens, score_scale, max_kv_len, first_visible=None, softcap=0.0, ring_capacity=0,
                    kv_format=capi.KV_Q8G64, scale_dtype=capi.SCALE_F16, out=None, workspace=None, total_kv_tokens=0, gate=None):
    batch = q.shape[0]
    if out is None:
        out = torch.empty((batch, num_heads * head_dim), dtype=torch.float32, device=q.device)
    args = capi.GqaDecodeArgs()
    args.q, args.k_plane, args.k_scales = _ptr(q), _ptr(k_plane), _ptr(k_scales)
    args.v_plane, args.v_scales = _ptr(v_plane), _ptr(v_scales)
    args.tables, args.kv_lens, args.first_visible = _ptr(tables), _ptr(kv_lens), _ptr(first_visible)
    args.out = _ptr(out)
    args.batch, args.num_heads, args.num_kv_heads, args.head_dim = batch, num_heads, num_kv_heads, head_dim
    args.table_stride = 0 if tables is None else tables.shape[1]
    args.max_kv_len, args.block_tokens, args.ring_capacity = max_kv_len, block_tokens, ring_capacity
    args.total_kv_tokens = total_kv_tokens
    args.score_scale, args.softcap = score_scale, softcap
    args.kv_format, args.scale_dtype, args.q_dtype = kv_format, scale_dtype, _DTYPE[q.dtype]
    if gate is not None:
        args.gate, args.gate_cols, args.gate_dtype = _ptr(gate), gate.shape[1], _DTYPE[gate.dtype]
    need = capi.load().zllm_attn_gqa_decode_workspace_bytes(C.byref(args))
    if need == 0:
        raise capi.ZllmAttnError(-1, capi.last_error())
    if workspace is False:  # the static-scratch entry point ignores both fields
        return args, out, None
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    args.workspace, args.workspace_bytes = _ptr(workspace), workspace.numel()
    return args, out, workspace


def gqa_decode(*a, **kw):
    """Batched GQA decode over the paged cache (zllm_attn_gqa_decode).  Returns f32 [batch, Hq*d]."""
    args, out, workspace = gqa_decode_args(*a, **kw)
    capi.check(capi.load().zllm_attn_gqa_decode(C.byref(args), _stream()))
    return out


def gqa_decode_static(*a, **kw):
    """zllm_attn_gqa_decode_static: the same call over the library's static device array (no workspace of the caller's)."""
    args, out, _ = gqa_decode_args(*a, workspace=False, **kw)
    capi.check(capi.load().zllm_attn_gqa_decode_static(C.byref(args), _stream()))
    return out


def gqa_prefill_chunk_args(q, k_plane, k_scales, v_plane, v_scales, table, position, num_heads, num_kv_heads, head_dim,
                           block_tokens, score_scale, window=0, softcap=0.0, kv_format=capi.KV_Q8G64,
                           scale_dtype=capi.SCALE_F16, out_dtype=torch.float32, gate=None, visible_ends=None, workspace=True,
                           visible_starts=None):
    """The argument block of zllm_attn_gqa_prefill_chunk, the output tensor and the workspace tensor (None without one):
    for callers that launch the same call many times."""
    rows = q.shape[0]
    out = torch.empty((rows, num_heads * head_dim), dtype=out_dtype, device=q.device)
    args = capi.GqaPrefillArgs()
    args.q, args.k_plane, args.k_scales = _ptr(q), _ptr(k_plane), _ptr(k_scales)
    args.v_plane, args.v_scales, args.table, args.out = _ptr(v_plane), _ptr(v_scales), _ptr(table), _ptr(out)
    args.rows, args.position, args.window = rows, position, window
    args.num_heads, args.num_kv_heads, args.head_dim, args.block_tokens = num_heads, num_kv_heads, head_dim, block_tokens
    args.score_scale, args.softcap = score_scale, softcap
    args.kv_format, args.scale_dtype = kv_format, scale_dtype
    args.q_dtype, args.out_dtype = _DTYPE[q.dtype], _DTYPE[out_dtype]
    if gate is not None:
        args.gate, args.gate_cols, args.gate_dtype = _ptr(gate), gate.shape[1], _DTYPE[gate.dtype]
    args.visible_ends = _ptr(visible_ends)
    args.visible_starts = _ptr(visible_starts)
    args.table_stride = 0 if table is None else table.numel()
    scratch = None
    if workspace:
        need = capi.load().zllm_attn_gqa_prefill_workspace_bytes(C.byref(args))
        scratch = torch.empty(max(int(need), 256), dtype=torch.uint8, device=q.device)
        args.workspace, args.workspace_bytes = _ptr(scratch), scratch.numel()
    return args, out, scratch


def gqa_prefill_chunk(*a, **kw):
    """One chunk of causal GQA prefill over the paged cache (zllm_attn_gqa_prefill_chunk).  `workspace=False` passes none:
    a chunk that would be cut into KV splits then runs unsplit (geometries that need a workspace fail)."""
    args, out, _scratch = gqa_prefill_chunk_args(*a, **kw)
    capi.check(capi.load().zllm_attn_gqa_prefill_chunk(C.byref(args), _stream()))
    return out


def mla_decode_args(q, kv_b, latent_codes, latent_scales, rope_cache, tables, ctx_lens, heads, q_head_dim,
                    kv_head_dim, latent_dim, rope_dim, block_tokens, max_ctx_len, out_dtype=torch.float32,
                    out_compact=True, out=None, workspace=None, selection=None, selection_counts=None, query_rows=1,
                    total_ctx_tokens=0, wide_tiles=False, kv_b_bits=0, kv_b_scales=None, kv_b_group=0, kv_b_scale_dtype=capi.SCALE_BF16):
    """`q` holds every query row of the call, sequence-major: [batch * query_rows, heads * q_head_dim].
    `kv_b` is bf16 unless kv_b_bits says f32 (32) or packed 8- / 4-bit codes with `kv_b_scales` per `kv_b_group` columns."""
    rows = q.shape[0]
    batch = rows // query_rows
    value_dim = kv_head_dim - (q_head_dim - rope_dim)
    if out is None:
        cols = heads * value_dim if out_compact else heads * q_head_dim
        out = torch.zeros((rows, cols), dtype=out_dtype, device=q.device)
    args = capi.MlaDecodeArgs()
    args.q, args.kv_b, args.latent_codes = _ptr(q), _ptr(kv_b), _ptr(latent_codes)
    args.latent_scales, args.rope_cache = _ptr(latent_scales), _ptr(rope_cache)
    args.tables, args.ctx_lens, args.out = _ptr(tables), _ptr(ctx_lens), _ptr(out)
    args.batch, args.heads, args.q_head_dim, args.kv_head_dim = batch, heads, q_head_dim, kv_head_dim
    args.latent_dim, args.rope_dim = latent_dim, rope_dim
    args.table_stride = 0 if tables is None else tables.shape[1]
    args.max_ctx_len, args.block_tokens = max_ctx_len, block_tokens
    args.q_dtype, args.out_dtype, args.out_compact = _DTYPE[q.dtype], _DTYPE[out_dtype], int(out_compact)
    args.query_rows = query_rows
    args.total_ctx_tokens = total_ctx_tokens
    args.stage_mask = capi.MLA_WIDE_TILES if wide_tiles else 0
    args.kv_b_bits, args.kv_b_scales, args.kv_b_group, args.kv_b_scale_dtype = kv_b_bits, _ptr(kv_b_scales), kv_b_group, kv_b_scale_dtype
    if selection is not None:  # [batch, top_k] token positions (uint32 / int32)
        args.selection, args.top_k = _ptr(selection), selection.shape[1]
        args.selection_counts = _ptr(selection_counts)
    need = capi.load().zllm_attn_mla_decode_workspace_bytes(C.byref(args))
    if need == 0:
        raise capi.ZllmAttnError(-1, capi.last_error())
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    args.workspace, args.workspace_bytes = _ptr(workspace), workspace.numel()
    return args, out, workspace


def mla_decode(*a, **kw):
    args, out, workspace = mla_decode_args(*a, **kw)
    capi.check(capi.load().zllm_attn_mla_decode(C.byref(args), _stream()))
    return out

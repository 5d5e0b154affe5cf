/*
 * zllm_attn — C ABI of the MI355X (gfx950) attention hot path.
 *
 * GQA / MLA decode and chunked-prefill attention over a Q8g64 paged KV cache,
 * plus the quantizing page appends that feed it.  Every entry point stands in
 * for one launcher (`try_*`) of zllm-lab/zllm's ROCm kernel layer; the comment
 * above each names the reference interface it replaces (paths relative to the
 * zLLM tree).
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes only; device pointers are marked [dev].
 *   - the caller owns every allocation, including the workspace whose size the
 *     matching *_workspace_bytes function returns.  Nothing here allocates,
 *     frees or synchronises; launches are asynchronous on `stream`.
 *   - re-entrant: no mutable global state; the error text is thread-local.
 *   - return value: 0 = ok, negative = invalid argument (see
 *     zllm_attn_last_error), positive = a hipError_t from the launch.
 *   - shape errors are reported before anything is launched, as the reference
 *     launchers do (src/kernel/rocm/hip/tensor/attention.rs:1022-1030,
 *     src/kernel/rocm/hip/attention/paged_mla.rs:2940-2977).
 *
 * KV layout (kept from src/kv_cache/mod.rs:179-331 and
 * src/kernel/rocm/hip/attention/paged_mla/source.hip:46-54,191-201):
 *   planar per tensor; row = one token; physical row of logical token t is
 *   table[t / block_tokens] * block_tokens + t % block_tokens (a NULL table is
 *   the identity); codes plane int8 [rows][cols]; scales plane one 16-bit (or
 *   f32) value per 64 contiguous columns [rows][cols / 64].
 */
#ifndef ZLLM_ATTN_H
#define ZLLM_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hipStream_t, passed opaquely so that bindings need no HIP headers. */
typedef void* zllm_stream_t;

/* Exported from libzllm_attn.so (everything else in the library is hidden). */
#define ZLLM_API __attribute__((visibility("default")))

/* Scale storage of a Q8g64 plane; numbering of `zllm_scale`
 * (src/kernel/rocm/hip/hiprtc.rs:104-116). */
enum { ZLLM_SCALE_BF16 = 0, ZLLM_SCALE_F16 = 1, ZLLM_SCALE_F32 = 2 };

/* Element type of activations handed in / out. */
enum { ZLLM_DTYPE_F32 = 0, ZLLM_DTYPE_BF16 = 1, ZLLM_DTYPE_F16 = 2 };

/* KV storage format (src/config.rs:1108-1114 KvCacheFormat {F16, Q8g64}). */
enum { ZLLM_KV_Q8G64 = 0, ZLLM_KV_F16 = 1 };

/* Which reference quantizer the codes follow:
 *   ROCM_MLA : scale = absmax * (1/127) (1.0 if 0), stored bf16, codes =
 *              nearbyint(x / f32(stored))   (paged_mla/source.hip:183-201)
 *   METAL_GQA: scale = absmax / 127 (1.0 if 0), stored f16, codes =
 *              rint(x * (1 / scale))        (kernel/metal/attention/mod.rs:114-127)
 *   CUDA_GQA : as METAL_GQA, stored f32     (kernel/cuda/attention.rs:331-341) */
enum { ZLLM_QUANT_ROCM_MLA = 0, ZLLM_QUANT_METAL_GQA = 1, ZLLM_QUANT_CUDA_GQA = 2 };

/* RoPE pair layout (src/attention/rope.rs:106-110). */
enum { ZLLM_ROTARY_INTERLEAVED = 0, ZLLM_ROTARY_SPLIT_HALF = 1 };

/* Stage selection for the split-KV entry points. */
enum { ZLLM_STAGE_ALL = 0, ZLLM_STAGE_PARTIAL = 1, ZLLM_STAGE_MERGE = 2 };

enum { ZLLM_MLA_ABSORB = 1, ZLLM_MLA_PARTIAL = 2, ZLLM_MLA_MERGE = 4, ZLLM_MLA_PROJECT = 8 };
/* OR-ed into zllm_mla_decode_args::stage_mask beside the stage bits (alone = the whole chain): the split-KV partial runs on
 * its second kernel -- tiles of f16(code * scale) instead of integer codes beside a scale table, 32x32x16 matrix tiles on
 * the value side -- where the call allows it (dense, more than 32 heads, pages of a multiple of 32 tokens); other calls
 * run the default kernel.  Same records, same results within the attention tolerance. */
enum { ZLLM_MLA_WIDE_TILES = 16 };

#define ZLLM_GROUP_SIZE 64 /* src/kv_cache/mod.rs:29 DEFAULT_GROUP_SIZE */

/* Library / device bring-up.  Optional: every entry point works without it.
 * Returns 0 and fills `cu_count` (may be NULL) when a gfx950 device is current. */
ZLLM_API int zllm_attn_init(int device, int* cu_count);

/* Text of the last failure on the calling thread ("" if none). */
ZLLM_API const char* zllm_attn_last_error(void);

/* ------------------------------------------------------------------------- *
 * Host-side layout arithmetic (no GPU).                                      *
 * ------------------------------------------------------------------------- */

/* CausalWindow::key_range (src/attention/gqa.rs:54-62); window 0 = Full. */
ZLLM_API void zllm_attn_key_range(uint64_t window, uint64_t query_position, uint64_t key_end,
                         uint64_t* start, uint64_t* end);

/* KvCacheSpec::bytes_per_token (src/kv_cache/mod.rs:570-585).  kind 0 = MLA
 * (a = kv_lora_rank, b = qk_rope_head_dim), 1 = GQA (a = kv heads, b = head
 * dim).  0 on invalid input. */
ZLLM_API uint64_t zllm_kv_bytes_per_token(int kind, uint64_t a, uint64_t b, uint64_t group);

/* KvCacheLayout planar offsets (src/kv_cache/mod.rs:246-330), Int8 format.
 * MLA: offsets = {base, codes, scales, rope}; GQA: {base, K codes, K scales,
 * V codes, V scales}.  Returns total bytes, 0 on invalid input. */
ZLLM_API uint64_t zllm_kv_layout_offsets(int kind, uint64_t a, uint64_t b, uint64_t group, uint64_t layer_count,
                                uint64_t capacity, uint64_t layer, uint64_t offsets[5]);

/* HybridGqaCacheLayout::write_plan (src/kv_cache/mod.rs:440-455): ring append
 * plan for a sliding-window layer.  plan = {end, source_start, token_count,
 * first_slot, first_count, second_count}.  0 ok, -1 invalid. */
ZLLM_API int zllm_kv_ring_write_plan(uint64_t capacity, uint64_t max_sequence_len, uint64_t position, uint64_t count,
                            uint64_t plan[6]);

/* ------------------------------------------------------------------------- *
 * Page appends.                                                              *
 * ------------------------------------------------------------------------- */

/* Quantize `rows` rows of `cols` values to Q8g64 and scatter them through the
 * block table at logical tokens [position, position + rows).
 * Replaces try_paged_cache_append_f32_q8
 * (src/kernel/rocm/hip/attention/paged_mla.rs:347; kernel
 * paged_mla/source.hip:164-202) and, with rule METAL_GQA / CUDA_GQA, the GQA
 * quantizers (kernel/metal/attention/mod.rs:89-128,
 * kernel/cuda/attention.rs:314-343).  Codes and scale bits are bit-exact with
 * the rule named. */
typedef struct zllm_q8_append_args {
    const void* src;           /* [dev] [rows, cols], src_dtype */
    int8_t* codes;             /* [dev] codes plane */
    void* scales;              /* [dev] scales plane (16-bit or f32 per rule) */
    const uint32_t* table;     /* [dev] block table or NULL (identity) */
    const uint32_t* positions; /* [dev] optional: positions[0] overrides `position`
                                  (graph replay; source.hip:787-807) */
    uint32_t position;         /* first logical token written */
    uint32_t rows;
    uint32_t cols;             /* multiple of 64 */
    uint32_t block_tokens;     /* tokens per page (any value >= 1) */
    uint32_t ring_capacity;    /* 0, or token -> token % ring_capacity first
                                  (kernel/cuda/attention.rs:82-88) */
    int src_dtype;             /* ZLLM_DTYPE_* */
    int rule;                  /* ZLLM_QUANT_* */
} zllm_q8_append_args;
ZLLM_API int zllm_attn_q8g64_append(const zllm_q8_append_args* args, zllm_stream_t stream);

/* f32/bf16/f16 -> bf16 or f16 scatter through the table (unquantized KV).
 * Replaces try_paged_cache_append_f32_bf16 (paged_mla/source.hip:146-162) and
 * append_rows_f16 (kernel/cuda/attention.rs:82-88). */
typedef struct zllm_half_append_args {
    const void* src;       /* [dev] [rows, cols] */
    void* cache;           /* [dev] 16-bit plane */
    const uint32_t* table; /* [dev] or NULL */
    uint32_t position, rows, cols, block_tokens, ring_capacity;
    int src_dtype;         /* ZLLM_DTYPE_* */
    int dst_dtype;         /* ZLLM_DTYPE_BF16 or ZLLM_DTYPE_F16 */
} zllm_half_append_args;
ZLLM_API int zllm_attn_half_append(const zllm_half_append_args* args, zllm_stream_t stream);

/* MLA append: quantize the latent (rule ROCM_MLA), optionally rotate the last
 * `rotary_dim` rope columns, store rope as bf16; one launch.
 * Replaces try_paged_cache_append_mla_{,rope_}f32_q8_bf16
 * (src/kernel/rocm/hip/attention/paged_mla.rs:1038-1160; kernel
 * paged_mla/source.hip:672-785, `_indirect` :787-807). */
typedef struct zllm_mla_append_args {
    const float* latent;       /* [dev] [rows, latent_cols] */
    const float* k_rope;       /* [dev] [rows, rope_cols] */
    const float* cosine;       /* [dev] [*, rotary_dim / 2] or NULL when rotary_dim == 0 */
    const float* sine;         /* [dev] */
    int8_t* latent_codes;      /* [dev] */
    uint16_t* latent_scales;   /* [dev] bf16 bits */
    uint16_t* rope_cache;      /* [dev] bf16 bits */
    const uint32_t* table;     /* [dev] or NULL */
    const uint32_t* positions; /* [dev] optional {position, rope_position} */
    uint32_t position;
    uint32_t rope_position;    /* row of the cos/sin tables for the first token */
    uint32_t rows, latent_cols, rope_cols, rotary_dim;
    int rotary_layout;         /* ZLLM_ROTARY_* */
    uint32_t block_tokens;
} zllm_mla_append_args;
ZLLM_API int zllm_attn_mla_append(const zllm_mla_append_args* args, zllm_stream_t stream);

/* Bit-exact gather of plane rows: out[r] = plane[paged_row(first + r)].
 * Serves KV snapshot download (src/backend/rocm/kv_cache.rs:3344) and is the
 * page/index gathering check. */
typedef struct zllm_gather_args {
    const void* plane;     /* [dev] */
    void* out;             /* [dev] [count, row_bytes] dense */
    const uint32_t* table; /* [dev] or NULL */
    uint32_t first, count, row_bytes, block_tokens, ring_capacity;
} zllm_gather_args;
ZLLM_API int zllm_attn_gather_rows(const zllm_gather_args* args, zllm_stream_t stream);

/* Inverse of zllm_attn_gather_rows: plane[paged_row(first + r)] = in[r].  Serves KV snapshot upload
 * (the restore half of src/backend/rocm/kv_cache.rs:3344-3598: a downloaded layer goes back into
 * whatever pages the restored sequence owns). */
typedef struct zllm_scatter_args {
    void* plane;           /* [dev] */
    const void* in;        /* [dev] [count, row_bytes] dense */
    const uint32_t* table; /* [dev] or NULL */
    uint32_t first, count, row_bytes, block_tokens, ring_capacity;
} zllm_scatter_args;
ZLLM_API int zllm_attn_scatter_rows(const zllm_scatter_args* args, zllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * KV snapshot wire format of one MLA layer (host side, no device access).     *
 * ------------------------------------------------------------------------- */

/* MlaLayerSerde (src/backend/rocm/kv_cache.rs:2067-2083) as write_mla_layer / read_mla_layer
 * put it on the wire (src/runtime/glm52/rocm_swap.rs:1090-1138; integers are u64 little-endian,
 * rocm_swap.rs:1145-1153):
 *   rows, ownership byte (0 Full, 1 BlockParity(0), 2 BlockParity(1), 3 InterleavedPair),
 *   latent_cols, rope_cols, latent_group_size, len + latent bytes,
 *   flag byte (+ len + scale bytes when 1), len + rope bytes.
 * latent_group_size 0 = bf16 latent without scales; otherwise Q8 codes + bf16 scales. */
typedef struct zllm_mla_layer_record {
    uint64_t rows;
    uint32_t ownership;           /* ZLLM_KV_OWNERSHIP_* */
    uint64_t latent_cols, rope_cols, latent_group_size;
    const uint8_t* latent;        /* [host] rows * latent_cols (Q8) or * 2 (bf16) bytes */
    uint64_t latent_bytes;
    const uint8_t* latent_scales; /* [host] rows * (latent_cols / group) * 2 bytes, or NULL */
    uint64_t latent_scales_bytes;
    const uint8_t* rope;          /* [host] rows * rope_cols * 2 bytes */
    uint64_t rope_bytes;
} zllm_mla_layer_record;
enum { ZLLM_KV_OWNERSHIP_FULL = 0, ZLLM_KV_OWNERSHIP_PARITY0 = 1, ZLLM_KV_OWNERSHIP_PARITY1 = 2, ZLLM_KV_OWNERSHIP_INTERLEAVED = 3 };
/* Bytes write would produce; 0 when the record's lengths do not match its shape. */
ZLLM_API uint64_t zllm_kv_mla_layer_wire_bytes(const zllm_mla_layer_record* record);
/* Serialise into out[0 .. capacity); *written = bytes produced.  0 ok, -1 invalid / too small. */
ZLLM_API int zllm_kv_mla_layer_write(const zllm_mla_layer_record* record, uint8_t* out, uint64_t capacity, uint64_t* written);
/* Parse one record from in[0 .. len): pointers in *record point into `in`; *consumed = bytes read.
 * 0 ok, -1 truncated or malformed (same conditions as read_mla_layer's errors), -2 shape and
 * blob lengths disagree. */
ZLLM_API int zllm_kv_mla_layer_read(const uint8_t* in, uint64_t len, zllm_mla_layer_record* record, uint64_t* consumed);

/* ------------------------------------------------------------------------- *
 * GQA decode: one query row per sequence, split-KV flash decoding.           *
 * ------------------------------------------------------------------------- */

/* Replaces try_gqa_decode_cached_f32
 * (src/kernel/rocm/hip/tensor/attention.rs:1021-1074; kernels
 * tensor/attention/source.hip:1272-1362), extended to a batch of sequences
 * over a paged Q8g64 (or f16) cache.  Sequence b attends logical tokens
 * [first_visible[b], kv_lens[b]) (CausalWindow::key_range of its last row,
 * src/attention/gqa.rs:54-62).  An empty range yields zeros, never NaN
 * (gqa.rs:201-204, source.hip:1361). */
typedef struct zllm_gqa_decode_args {
    const void* q;                 /* [dev] [batch, num_heads * head_dim], q_dtype */
    const void* k_plane;           /* [dev] K codes (Q8) or f16 K rows */
    const void* k_scales;          /* [dev] K scales (Q8 only) */
    const void* v_plane;           /* [dev] */
    const void* v_scales;          /* [dev] */
    const uint32_t* tables;        /* [dev] [batch, table_stride] block tables */
    const uint32_t* kv_lens;       /* [dev] [batch] */
    const uint32_t* first_visible; /* [dev] [batch] or NULL (= 0) */
    float* out;                    /* [dev] [batch, num_heads * head_dim] f32 */
    void* workspace;               /* [dev] zllm_attn_gqa_decode_workspace_bytes */
    uint64_t workspace_bytes;
    uint32_t batch;
    uint32_t num_heads, num_kv_heads, head_dim; /* head_dim in {64, 128, 192, 256}; f16 caches 128 / 256 */
    uint32_t table_stride;         /* entries per sequence in `tables` */
    uint32_t max_kv_len;           /* host upper bound of kv_lens, below 2^31: sizes the grid and the split plan.  A call
                                      recorded into a HIP graph stays valid only while every kv_lens[b] on the
                                      device is <= max_kv_len; tokens past the planned splits are not read */
    uint32_t total_kv_tokens;      /* host bound: sum of the visible lengths (0 = unknown, batch * max_kv_len is
                                      assumed).  Pass it for batches of unequal lengths and for sliding windows:
                                      planned as if every sequence were max_kv_len long, a long sequence among short
                                      ones (or a short window) gets few workgroups.  With it the splits are sized for
                                      the tokens there are and the split records for the splits there are (see
                                      zllm_attn_gqa_decode_record_layout), so it must not be below the real sum --
                                      like max_kv_len it has to hold for every replay of a recorded call.  Splits
                                      beyond the records it sized are dropped (wrong output, nothing out of bounds) */
    uint32_t block_tokens;
    uint32_t ring_capacity;        /* 0 or sliding-window ring rows (token % capacity) */
    float score_scale;             /* > 0 */
    float softcap;                 /* 0 = off; else s <- softcap * tanh(s / softcap) */
    int kv_format;                 /* ZLLM_KV_* */
    int scale_dtype;               /* ZLLM_SCALE_* (Q8 only) */
    int q_dtype;                   /* ZLLM_DTYPE_* */
    uint32_t stages;               /* 0 = partial + merge; ZLLM_STAGE_PARTIAL leaves the
                                      un-merged (partial, max, sum) records in the workspace
                                      for a caller that combines shards itself
                                      (cf. try_paged_mla_attention_ct_shard,
                                      paged_mla.rs:3642); ZLLM_STAGE_MERGE combines records
                                      already in the workspace */
    /* Output gate, the sigmoid_gate step that follows attention in HybridAttention::full
     * (src/attention/hybrid.rs:79; src/backend/cpu/context.rs:419-432): out *= 1 / (1 + exp(-gate)).
     * NULL = no gate. */
    const void* gate;              /* [dev] [rows, gate_cols], gate_dtype */
    uint32_t gate_cols;            /* num_heads * head_dim, or 1 (one gate per row) */
    int gate_dtype;                /* ZLLM_DTYPE_F32 or ZLLM_DTYPE_BF16 */
} zllm_gqa_decode_args;
ZLLM_API uint64_t zllm_attn_gqa_decode_workspace_bytes(const zllm_gqa_decode_args* args);
/* The split plan the call would run with: every sequence's visible range is cut into at most *max_chunks splits of at
 * most *chunk_tokens tokens (a multiple of 32), so max_chunks * chunk_tokens >= max_kv_len.  It is fixed by the host
 * arguments alone (the tile / split geometry of try_gqa_decode_cached_f32,
 * src/kernel/rocm/hip/tensor/attention.rs:1031-1046): a sequence whose kv_lens[b] on the device has grown past
 * max_kv_len -- a recorded graph replayed too long -- is read up to max_chunks * chunk_tokens tokens only.
 * 0 ok, negative = invalid arguments. */
ZLLM_API int zllm_attn_gqa_decode_split_plan(const zllm_gqa_decode_args* args, uint32_t* chunk_tokens, uint32_t* max_chunks);
/* Where a call's split records lie in its workspace, for a caller that combines ZLLM_STAGE_PARTIAL records itself
 * (the reference sizes its records per launch the same way, src/kernel/rocm/hip/attention/paged_mla.rs:2987-2994,
 * 3248-3257): partial f32 [record_rows][heads][width] at partial_offset (width = head_dim for GQA, latent_dim for MLA),
 * (max, sum) f32 pairs [record_rows][heads][2] at stats_offset.  Split c of record group g (a sequence; for MLA calls
 * with query_rows > 1, a query row) is row g * max_chunks + c when dense == 0 -- a plan for equal lengths -- and row
 * first_rows[g] + c when dense == 1: a ragged plan numbers its records over the live splits only, in group order, so the
 * workspace grows with the tokens there are and not with batch x longest sequence; first_rows is u32 [groups] at
 * first_rows_offset, written by the partial stage (entries of groups without splits are not written).  A group has
 * min(max_chunks, ceil(n / chunk_tokens)) splits, n = its visible tokens (GQA: counted from first_visible rounded down to
 * a multiple of 32).  A record is un-normalised: partial = sum of p x value with p = 2^(score - max), max the largest
 * scaled score of the split in base-2 units (score x score_scale x log2 e), sum = sum of p; an empty split has
 * (max, sum) = (-inf, 0).  Combined: out = sum_c partial_c 2^(max_c - M) / sum_c sum_c 2^(max_c - M), M = max_c max_c. */
typedef struct zllm_split_record_layout {
    uint64_t record_rows;
    uint64_t partial_offset;
    uint64_t stats_offset;
    uint64_t first_rows_offset; /* 0 when dense == 0 */
    uint32_t chunk_tokens, max_chunks;
    uint32_t dense;
} zllm_split_record_layout;
ZLLM_API int zllm_attn_gqa_decode_record_layout(const zllm_gqa_decode_args* args, zllm_split_record_layout* layout);
ZLLM_API int zllm_attn_gqa_decode(const zllm_gqa_decode_args* args, zllm_stream_t stream);

/* zllm_attn_gqa_decode for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose launcher takes its
 * split records from a pool (src/kernel/rocm/hip/tensor/attention.rs:1031-1046).  Same arguments, same kernels
 * and the same output bits as zllm_attn_gqa_decode, except that `workspace` / `workspace_bytes` are ignored: the
 * split records go to an array that is part of the library's device code (zllm_attn_static_scratch_bytes() bytes
 * on every GPU the library is loaded on, held until the process ends).  A call whose
 * zllm_attn_gqa_decode_workspace_bytes exceeds that size is rejected (negative return, nothing launched).
 * Nothing in the array has to survive between calls and nothing in it has to be cleared.  All calls on one GPU
 * share the one array: calls that overlap on a GPU (two streams, two threads) race and must be serialised by the
 * caller.  zllm_attn_init(device, ...) looks the array's address up for that device; without it the first call
 * on a device does (make that call, or the init call, before a capture begins). */
ZLLM_API uint64_t zllm_attn_static_scratch_bytes(void);
ZLLM_API int zllm_attn_gqa_decode_static(const zllm_gqa_decode_args* args, zllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * GQA chunked prefill: T query rows appended at `position`.                  *
 * ------------------------------------------------------------------------- */

/* Replaces try_block_attention_resident_f32 driven with causal ranges
 * (src/kernel/rocm/hip/tensor/attention.rs:727-798,
 * src/backend/rocm/attention.rs:2232-2242).  Row r attends logical tokens
 * key_range(position + r, position + rows) of one sequence whose K/V
 * (including the chunk's own rows) are already in the paged cache.
 * Q8g64 caches (head_dim 64 / 128 / 256, scales of any type) and f16 caches
 * (head_dim 128 / 256) run matrix-core chunk kernels.  A chunk with too few row tiles
 * for the device -- a short chunk over a long prefix -- is cut into KV splits
 * (parts of a tile's visible range, combined like a decode call's splits) when the
 * caller passes zllm_attn_gqa_prefill_workspace_bytes of 16-byte aligned workspace
 * for their records, and runs unsplit (same results, one workgroup walking the whole
 * prefix per tile) when it passes none or less.  A chunk of a few rows (one to three
 * over a long prefix, up to sixteen over a short one) is a decode step in all but name
 * -- the reference decodes through this path with one row
 * (src/backend/rocm/attention.rs:2202-2231) -- and, given that workspace, runs every
 * row as one item of the split-KV decode kernels.  So does what is
 * left -- f32 queries other than over Q8g64 with 16-bit scales at head_dim 128; more
 * than 128 query heads per KV head at head_dim 256; head_dim 192 -- whatever the number of rows
 * (bound by cache bandwidth, not by the matrix cores); that cannot run without the
 * workspace. */
typedef struct zllm_gqa_prefill_args {
    const void* q;         /* [dev] [rows, num_heads * head_dim], q_dtype */
    const void* k_plane;   /* [dev] */
    const void* k_scales;  /* [dev] */
    const void* v_plane;   /* [dev] */
    const void* v_scales;  /* [dev] */
    const uint32_t* table; /* [dev] block table of the sequence */
    void* out;             /* [dev] [rows, num_heads * head_dim], out_dtype */
    void* workspace;       /* [dev] */
    uint64_t workspace_bytes;
    uint32_t rows;         /* chunk length T */
    uint32_t position;     /* tokens already cached before the chunk; position + rows stays below 2^31 */
    uint32_t window;       /* 0 = full causal, else sliding window size */
    uint32_t num_heads, num_kv_heads, head_dim;
    uint32_t block_tokens;
    float score_scale;
    float softcap;
    int kv_format, scale_dtype, q_dtype, out_dtype;
    /* Output gate, the sigmoid_gate step that follows attention in HybridAttention::full
     * (src/attention/hybrid.rs:79; src/backend/cpu/context.rs:419-432): out *= 1 / (1 + exp(-gate)).
     * NULL = no gate. */
    const void* gate;              /* [dev] [rows, gate_cols], gate_dtype */
    uint32_t gate_cols;            /* num_heads * head_dim, or 1 (one gate per row) */
    int gate_dtype;                /* ZLLM_DTYPE_F32 or ZLLM_DTYPE_BF16 */
    /* Explicit visible ends, the multimodal case in which the rows of a visual block read to the end of their
     * block (CausalWindow::key_range_with_visible_end, src/attention/gqa.rs:65-68;
     * gqa_prefill_attention_cached_visible, src/backend/rocm/attention.rs:2256-2316; per-row ranges of
     * BlockAttentionBackend::block_attention, src/backend/mod.rs:1583-1616): row r attends
     * [start of key_range(position + r), min(max(position + r + 1, visible_ends[r]), position + rows)).
     * Absolute token positions.  NULL = causal. */
    const uint32_t* visible_ends;  /* [dev] [rows] or NULL */
    uint32_t table_stride;         /* entries in `table` (0 = not stated: the table must cover position + rows) */
    /* Explicit row ranges, BlockAttentionSpec::visible (src/attention/block.rs:10-16; the varlen and segment forms of
     * BlockAttentionBackend::block_attention, src/backend/mod.rs:1582-1617, are ranges too): with visible_starts given,
     * row r attends exactly the cache rows [visible_starts[r], min(visible_ends[r], position + rows)) -- no causal
     * rule, no window (window must be 0, visible_ends must be given); an empty range gives a zero row.  `position +
     * rows` is then only the number of cache rows the call may read. */
    const uint32_t* visible_starts; /* [dev] [rows] or NULL */
} zllm_gqa_prefill_args;
ZLLM_API uint64_t zllm_attn_gqa_prefill_workspace_bytes(const zllm_gqa_prefill_args* args);
ZLLM_API int zllm_attn_gqa_prefill_chunk(const zllm_gqa_prefill_args* args, zllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * Pre-attention prologue of a GQA layer.                                     *
 * ------------------------------------------------------------------------- */

/* One launch for what HybridAttention::full does between the projections and the
 * attention call (src/attention/hybrid.rs:66-78): per-head RMSNorm of Q and K
 * (gemma_rmsnorm_heads / rmsnorm_heads, src/kernel/cpu/vae.rs:297-334), RoPE of
 * both at the row's position (rope_prefix, src/attention/rope.rs:120-164), and
 * the quantizing page append of K and V (as zllm_attn_q8g64_append).  The
 * normalise-and-rotate half is what the trait hook
 * fused_rmsnorm_qkv_head_norm_rope (src/backend/mod.rs:1515-1538) asks of a
 * backend; the Q/K/V projections stay with the caller's GEMM.
 * Q comes out as a tensor for zllm_attn_gqa_decode / _prefill_chunk; K and V go
 * straight into the pages.  Arithmetic is f32 with separately rounded steps
 * in the reference's order, so Q (f32) and the K/V codes and scales are
 * bit-exact with the CPU chain norm -> rope -> quantize. */
typedef struct zllm_gqa_prologue_args {
    const void* q;             /* [dev] [rows, num_heads * head_dim], src_dtype */
    const void* k;             /* [dev] [rows, num_kv_heads * head_dim], src_dtype */
    const void* v;             /* [dev] [rows, num_kv_heads * head_dim], src_dtype */
    const float* q_norm;       /* [dev] [head_dim] or NULL (no Q norm) */
    const float* k_norm;       /* [dev] [head_dim] or NULL (no K norm) */
    const float* cosine;       /* [dev] [rope_table_rows, rotary_dim / 2]; unused when rotary_dim == 0 */
    const float* sine;
    void* q_out;               /* [dev] [rows, num_heads * head_dim], q_out_dtype */
    int8_t* k_codes;           /* [dev] paged planes, as in zllm_q8_append_args */
    void* k_scales;
    int8_t* v_codes;
    void* v_scales;
    const uint32_t* table;     /* [dev] block table or NULL (identity) */
    const uint32_t* positions; /* [dev] optional: positions[0] overrides `position` (graph replay) */
    uint32_t rows, num_heads, num_kv_heads;
    uint32_t head_dim;         /* multiple of 64, at most 256 */
    uint32_t rotary_dim;       /* even, <= head_dim; the first rotary_dim columns of a head rotate */
    uint32_t rope_table_rows;  /* rows of cosine / sine: position + rows must not exceed it */
    uint32_t position;         /* first row's token position: RoPE angle and page slot */
    uint32_t block_tokens, ring_capacity;
    float eps;                 /* RMSNorm epsilon (> 0 when a norm weight is given) */
    float weight_offset;       /* 1 = Gemma form (1 + weight), 0 = plain */
    int src_dtype;             /* ZLLM_DTYPE_* of q, k, v */
    int q_out_dtype;           /* ZLLM_DTYPE_F32 or ZLLM_DTYPE_BF16 */
    int rule;                  /* ZLLM_QUANT_* of the K/V pages */
    int split_half;            /* 1 = pairs (i, i + rotary_dim / 2), 0 = interleaved (2 i, 2 i + 1) */
} zllm_gqa_prologue_args;
ZLLM_API int zllm_attn_gqa_prologue(const zllm_gqa_prologue_args* args, zllm_stream_t stream);

/* ------------------------------------------------------------------------- *
 * MLA absorbed decode over the Q8g64 latent cache.                           *
 * ------------------------------------------------------------------------- */

/* Replaces try_paged_mla_attention_ct_into
 * (src/kernel/rocm/hip/attention/paged_mla.rs:2870-2914, inner :2917-3634), one query row per sequence or a
 * prefill chunk of `query_rows` rows (the dense prefill arm, kernel mla_paged_dense_latent_f32,
 * paged_mla/source.hip:3739):
 * absorb (q_nope . W_kv_b[h, 0:nope, :] -> bf16) -> split-KV partial -> LSE
 * merge -> project value (weighted . W_kv_b[h, nope:, :]^T).  Output rows have
 * stride q_head_dim with only the first value_dim entries of each head slot
 * written (src/attention/mla.rs:134) when out_compact == 0, or are compact
 * [batch, heads * value_dim] (src/kernel/cpu/mla.rs:1064-1075) otherwise. */
typedef struct zllm_mla_decode_args {
    const void* q;                /* [dev] [batch * rows, heads * q_head_dim], q_dtype */
    const uint16_t* kv_b;         /* [dev] bf16 bits [heads * kv_head_dim, latent_dim]; another form with kv_b_bits */
    const int8_t* latent_codes;   /* [dev] [rows, latent_dim] */
    const uint16_t* latent_scales;/* [dev] bf16 bits [rows, latent_dim / 64] */
    const uint16_t* rope_cache;   /* [dev] bf16 bits [rows, rope_dim] */
    const uint32_t* tables;       /* [dev] [batch, table_stride] */
    const uint32_t* ctx_lens;     /* [dev] [batch] tokens visible to the (last) query row of each sequence */
    void* out;                    /* [dev] out_dtype */
    void* workspace;              /* [dev] */
    uint64_t workspace_bytes;
    uint32_t batch, heads;
    uint32_t q_head_dim;          /* nope + rope */
    uint32_t kv_head_dim;         /* nope + value */
    uint32_t latent_dim;          /* a multiple of 64 up to 1024; 512 runs the matrix-core kernels */
    uint32_t rope_dim;            /* even, up to 256; 64 runs the matrix-core kernels */
    uint32_t table_stride;
    uint32_t max_ctx_len;         /* host upper bound of ctx_lens, below 2^31 (split plan); a recorded graph stays valid
                                     only while every ctx_lens[b] <= max_ctx_len */
    uint32_t block_tokens;
    int q_dtype;                  /* ZLLM_DTYPE_F32 or ZLLM_DTYPE_BF16 */
    int out_dtype;                /* ZLLM_DTYPE_F32 or ZLLM_DTYPE_BF16 */
    int out_compact;
    uint32_t stage_mask;          /* 0 = whole chain; else OR of ZLLM_MLA_ABSORB / _PARTIAL / _MERGE /
                                     _PROJECT (and optionally ZLLM_MLA_WIDE_TILES): run only those stages on
                                     the records already in the
                                     workspace (shard exchange, per-stage timing;
                                     cf. paged_mla.rs:3068-3081 per-stage profile) */
    /* Selected-token (sparse) decode, the `selection` arm of the same launch
     * (paged_mla.rs:3092-3105,3192-3195; kernel side source.hip:4738-4764): a sequence whose
     * context is longer than top_k attends only to the tokens selection[b, 0 .. count_b), count_b =
     * selection_counts[b] when given, else top_k; a sequence with ctx_len <= top_k stays dense.
     * Entries are token positions (< ctx_len), used in the order given.  NULL = dense. */
    uint32_t top_k;
    const uint32_t* selection;        /* [dev] [batch * rows, top_k] or NULL */
    const uint32_t* selection_counts; /* [dev] [batch * rows] or NULL */
    /* Query rows per sequence.  0 or 1: a decode step.  T > 1: a prefill chunk -- the last T tokens of every
     * sequence are its query rows (already appended to the cache), causal inside the chunk: row r sees
     * ctx_lens[b] - (T - 1 - r) tokens, i.e. position + r + 1 with position = ctx_lens[b] - T
     * (MlaPrefillBackend::mla_prefill_attention{,_rope}, src/backend/mod.rs:1134-1152; the query_rows > 1 arm of
     * try_paged_mla_attention_ct_into, src/kernel/rocm/hip/attention/paged_mla.rs:3397-3549; causal rule as in
     * src/kernel/cpu/mla.rs:958-1018).  q is [batch * T, heads * q_head_dim] and out [batch * T, ...], sequence-major;
     * a selection holds one list per query row.  The reference returns bf16 for T > 1
     * (src/backend/rocm/attention.rs:17-19): pass out_dtype = ZLLM_DTYPE_BF16 for that.  batch * T <= 65535. */
    uint32_t query_rows;
    /* Host bound for batches of unequal lengths: the sum of ctx_lens over the sequences (0 = unknown, every sequence is
     * planned as max_ctx_len long, and a long sequence among short ones gets few workgroups).  With it the splits are
     * sized for the tokens there are and the split records for the splits there are (zllm_attn_mla_decode_record_layout),
     * so it must not be below the real sum -- like max_ctx_len it has to hold for every replay of a recorded call;
     * splits beyond the records it sized are dropped (wrong output, nothing out of bounds). */
    uint32_t total_ctx_tokens;
    /* kv_b in the other forms the reference's weight loader reads (paged_weight,
     * src/kernel/rocm/hip/attention/paged_mla/source.hip:2-26; W8A16 / W4A16 of ct_mla_weight,
     * src/backend/rocm/attention.rs:181-192).  kv_b_bits 0 or 16: bf16 at kv_b.  32: f32 at kv_b.  8 / 4: codes at kv_b,
     * packed low bits first into 32-bit words, ceil(latent_dim / (32 / bits)) words a row; element = (code - 128) or
     * (code - 8) times kv_b_scales[row * (latent_dim / kv_b_group) + column / kv_b_group], scales of kv_b_scale_dtype
     * (ZLLM_SCALE_*).  Only the absorb and projection stages read kv_b: with any form but bf16 those two run on the
     * vector ALUs, f32 throughout. */
    const void* kv_b_scales;      /* [dev] or NULL */
    uint32_t kv_b_bits;
    uint32_t kv_b_group;          /* columns per scale; divides latent_dim */
    int kv_b_scale_dtype;
} zllm_mla_decode_args;
ZLLM_API uint64_t zllm_attn_mla_decode_workspace_bytes(const zllm_mla_decode_args* args);
/* The record layout of a call, as zllm_attn_gqa_decode_record_layout gives it for GQA; record groups are query rows. */
ZLLM_API int zllm_attn_mla_decode_record_layout(const zllm_mla_decode_args* args, zllm_split_record_layout* layout);
ZLLM_API int zllm_attn_mla_decode(const zllm_mla_decode_args* args, zllm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* ZLLM_ATTN_H */

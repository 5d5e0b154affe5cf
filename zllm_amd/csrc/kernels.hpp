// Kernel parameter blocks and launch functions (internal; the public surface is include/zllm_attn.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace zllm {

struct Q8AppendParams {
    const void* src;
    signed char* codes;
    void* scales;
    const unsigned int* table;
    const unsigned int* positions;
    unsigned int position, rows, cols, block_tokens, ring_capacity;
    int src_dtype, rule;
};

struct GqaPrologueParams {
    const void* q;
    const void* k;
    const void* v;
    const float* q_norm;
    const float* k_norm;
    const float* cosine;
    const float* sine;
    void* q_out;
    signed char* k_codes;
    void* k_scales;
    signed char* v_codes;
    void* v_scales;
    const unsigned int* table;
    const unsigned int* positions;
    unsigned int rows, num_heads, num_kv_heads, head_dim, rotary_dim, position, block_tokens, ring_capacity;
    float eps, weight_offset;
    int src_dtype, q_out_dtype, rule, split_half;
};

struct HalfAppendParams {
    const void* src;
    unsigned short* cache;
    const unsigned int* table;
    unsigned int position, rows, cols, block_tokens, ring_capacity;
    int src_dtype, dst_dtype;
};

struct MlaAppendParams {
    const float* latent;
    const float* k_rope;
    const float* cosine;
    const float* sine;
    signed char* latent_codes;
    unsigned short* latent_scales;
    unsigned short* rope_cache;
    const unsigned int* table;
    const unsigned int* positions;
    unsigned int position, rope_position, rows, latent_cols, rope_cols, rotary_dim, split_half, block_tokens;
};

struct GatherParams {
    const void* plane;
    void* out;
    const unsigned int* table;
    unsigned int first, count, row_bytes, block_tokens, ring_capacity;
};

struct ScatterParams {
    void* plane;
    const void* in;
    const unsigned int* table;
    unsigned int first, count, row_bytes, block_tokens, ring_capacity;
};

// Split-KV geometry shared by the partial and merge kernels.
struct SplitPlan {
    unsigned int chunk_tokens; // tokens per split (multiple of 32)
    unsigned int max_chunks;   // grid extent over splits
};

struct GqaDecodeParams {
    const void* q;
    const unsigned char* k_plane;
    const unsigned char* k_scales;
    const unsigned char* v_plane;
    const unsigned char* v_scales;
    const unsigned int* tables;
    const unsigned int* kv_lens;
    const unsigned int* first_visible;
    float* out;
    float* partial; // [record row][num_heads][head_dim]
    float* stats;   // [record row][num_heads][2] = (max, sum)
    // Record rows.  record_rows == 0: row = sequence * max_chunks + split.  Otherwise the records are numbered like the
    // work items, densely over the live splits: row = first_rows[sequence] + split, `record_rows` rows in all; the
    // partial kernel writes first_rows, the merge reads it.
    unsigned int* first_rows;
    unsigned int record_rows;
    unsigned int batch, num_heads, num_kv_heads, head_dim, group;
    unsigned int table_stride, block_tokens, block_shift, ring_capacity;
    unsigned int chunk_tokens, max_chunks;
    float score_scale, softcap;
    int q_dtype;
    const void* gate; // optional sigmoid output gate [batch][gate_cols]
    unsigned int gate_cols;
    int gate_dtype;
    // split merge only: query rows per sequence (0 = 1).  Record row v belongs to sequence v / query_rows and sees
    // kv_lens[sequence] - (query_rows - 1 - v % query_rows) tokens; `batch` then counts record rows.
    unsigned int query_rows;
    unsigned int table_shared; // 1: every item reads the one table at `tables` (rows of a prefill chunk); table_stride still bounds it
    int out_dtype;             // split merge: element type of `out` (0 f32, 1 bf16, 2 f16)
    // partial kernels: (sequence, split) items a workgroup runs side by side, each with one wave per KV head of its block
    // (0 = 1).  More than one when the KV heads alone would leave the workgroup's waves unused.
    unsigned int items_per_group;
    // split merge only: every record row has this many splits (0: the count follows from kv_lens and first_visible)
    unsigned int fixed_chunks;
};

struct GqaPrefillParams {
    const void* q;
    const unsigned char* k_plane;
    const unsigned char* k_scales;
    const unsigned char* v_plane;
    const unsigned char* v_scales;
    const unsigned int* table;
    void* out;
    unsigned int rows, position, window;
    unsigned int num_heads, num_kv_heads, head_dim, group;
    unsigned int block_tokens, block_shift;
    float score_scale, softcap;
    int q_dtype, out_dtype;
    const void* gate; // optional sigmoid output gate [rows][gate_cols]
    unsigned int gate_cols;
    int gate_dtype;
    const unsigned int* visible_ends; // optional [rows]: row r reads up to max(position + r + 1, visible_ends[r])
    const unsigned int* visible_starts; // optional [rows], with visible_ends: row r reads exactly [visible_starts[r], visible_ends[r])
    // KV splits of a chunk that has too few row tiles for the CUs: workgroup z of a row tile attends part z of the tile's
    // visible range (equal 32-aligned parts of at most chunk_tokens) and leaves un-normalised records for the split merge:
    // partial [rows][max_chunks][num_heads][head_dim], stats [rows][max_chunks][num_heads][2] = (max, sum).  max_chunks <= 1:
    // no splits, the kernel writes `out` itself.
    float* partial;
    float* stats;
    unsigned int chunk_tokens, max_chunks;
};

struct MlaDecodeParams {
    const void* q;
    const unsigned short* kv_b;
    const signed char* latent_codes;
    const unsigned short* latent_scales;
    const unsigned short* rope_cache;
    const unsigned int* tables;
    const unsigned int* ctx_lens;
    void* out;
    unsigned short* absorbed; // bf16 [batch][heads][latent_dim + rope_dim] (absorbed nope | q_rope)
    float* partial;           // [record row][heads][latent_dim]
    float* stats;             // [record row][heads][2]
    // Record rows.  record_rows == 0: row = query row * max_chunks + split, and the partial grid is (split, head block,
    // query row).  Otherwise records and work items are numbered densely over the live splits (grid = (item, head block)):
    // row = first_rows[query row] + split; the partial kernel writes first_rows, the merges read it.
    unsigned int* first_rows;
    unsigned int record_rows;
    float* weighted;          // [batch][heads][latent_dim]
    unsigned int batch, heads, q_head_dim, kv_head_dim, latent_dim, rope_dim, nope_dim, value_dim;
    unsigned int column_split; // mla_absorb_mfma: waves that share a block of sixteen rows (set by the launcher)
    unsigned int table_stride, block_tokens, block_shift;
    unsigned int chunk_tokens, max_chunks;
    float score_scale;
    int q_dtype, out_dtype, out_compact;
    const unsigned int* selection;        // [batch][top_k] token positions, or nullptr (dense)
    const unsigned int* selection_counts; // [batch] or nullptr
    unsigned int top_k;
    // kv_b [heads * kv_head_dim, latent_dim] in another form than bf16 (mla_generic.hip): bits 32 = f32, 8 / 4 = codes in
    // 32-bit words with a scale per row and `kv_b_group` columns; 16 = bf16 at `kv_b`
    const void* kv_b_scales;
    unsigned int kv_b_bits, kv_b_group;
    int kv_b_scale_dtype;
    // Query rows per sequence (>= 1).  With more than one, the last query_rows tokens of a sequence are its query rows
    // (a prefill chunk, causal inside the chunk): `batch` counts query rows over all sequences, row v belongs to
    // sequence v / query_rows and sees ctx_lens[sequence] - (query_rows - 1 - v % query_rows) tokens.
    unsigned int query_rows;
};

// Chunked prefill over Q8g64 with 16-bit scales at head_dim 128: whether the chunk runs row tiles of 128 (row, head) pairs
// instead of 256.  True for a chunk whose pairs all fit the smaller tile, and for one that is much longer than what lies before it (its row tiles' ranges grow from almost
// nothing to the whole chunk) when the full-size tiles would be at most one workgroup per compute unit: twice as many
// workgroups, handed out longest first, even the launch out.  The split planner and the launcher both ask.
bool gqa_prefill_half_tiles(unsigned int rows, unsigned int position, unsigned int window, unsigned int num_heads, unsigned int num_kv_heads,
                            unsigned int head_dim, int kv_format, int scale_dtype, int q_dtype);

// KV heads (= waves) per GQA decode workgroup for a head dimension.
unsigned int gqa_decode_max_waves(unsigned int head_dim);
unsigned int gqa_decode_items_per_group(unsigned int head_dim, unsigned int num_kv_heads);

hipError_t launch_q8g64_append(const Q8AppendParams& p, hipStream_t stream);
hipError_t launch_scatter_rows(const ScatterParams& p, hipStream_t stream);
hipError_t launch_gqa_prologue(const GqaPrologueParams& p, hipStream_t stream);
hipError_t launch_half_append(const HalfAppendParams& p, hipStream_t stream);
hipError_t launch_mla_append(const MlaAppendParams& p, hipStream_t stream);
hipError_t launch_gather_rows(const GatherParams& p, hipStream_t stream);

// kv_format: 0 = Q8g64, 1 = f16; scale_dtype: 0 = bf16, 1 = f16 (Q8 only).
hipError_t launch_gqa_decode(const GqaDecodeParams& p, int kv_format, int scale_dtype, unsigned int stages, hipStream_t stream);
hipError_t launch_gqa_prefill(const GqaPrefillParams& p, int kv_format, int scale_dtype, hipStream_t stream);
hipError_t launch_mla_decode(const MlaDecodeParams& p, unsigned int stage_mask, hipStream_t stream);
// The vector-ALU kernels for latent / rope widths other than 512 / 64 and for kv_b in other forms than bf16 (mla_generic.hip).
hipError_t launch_mla_absorb_any(const MlaDecodeParams& p, hipStream_t stream);
hipError_t launch_mla_partial_any(const MlaDecodeParams& p, hipStream_t stream);
hipError_t launch_mla_project_any(const MlaDecodeParams& p, hipStream_t stream);
// The split-KV partial on 32x32x16 matrix tiles (mla_partial_x32.hip): which calls it takes, and its launch.
bool mla_partial_x32_takes(const MlaDecodeParams& p);
hipError_t launch_mla_partial_x32(const MlaDecodeParams& p, hipStream_t stream);
// LSE combine of split records: uses kv_lens, first_visible, partial, stats, out, batch, num_heads,
// head_dim, chunk_tokens, max_chunks of the parameter block.
hipError_t launch_split_merge(const GqaDecodeParams& p, hipStream_t stream);
// lens[r], first[r] = visible range of row r of a prefill chunk (window 0 = full causal; visible_ends optional; with
// visible_starts the range is [visible_starts[r], visible_ends[r]) as given)
hipError_t launch_prefill_row_ranges(unsigned int* lens, unsigned int* first, const unsigned int* visible_ends, const unsigned int* visible_starts, unsigned int rows,
                                     unsigned int position, unsigned int window, hipStream_t stream);

} // namespace zllm

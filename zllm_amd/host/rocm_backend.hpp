// Host side of the attention path above the C ABI (include/zllm_attn.h), in C++ because the reference's
// host side is compiled code (Rust) and no Rust toolchain exists here.  Names, argument meaning and error
// behaviour follow the reference's backend traits for this path:
//   GqaPrefillBackend::gqa_prefill_attention_cached   src/backend/mod.rs:1484-1494, ROCm body
//                                                     src/backend/rocm/attention.rs:2202-2254
//   GqaPrefillBackend::gqa_prefill_attention_cached_{visible,from}   src/backend/mod.rs:1495-1513
//   MlaPrefillBackend::mla_prefill_attention{,_rope}  src/backend/mod.rs:1134-1152, attention.rs:1732-1764
//   DecodeBackend::{append_mla, append_mla_rope,
//                   mla_decode_attention}             src/backend/mod.rs:1162-1180, attention.rs:1805-1832
//   CausalWindow::{key_range, cache_capacity}         src/attention/gqa.rs:54-75
//   GqaSpec / MlaSpec                                 src/attention/gqa.rs:144-168, src/attention/mla.rs:5-70
//   BackendError                                      src/backend/mod.rs:38-46
// A cache here belongs to one sequence, as the reference's RocmKvCache does (src/backend/rocm/kv_cache.rs);
// the batched entry points of the C ABI are the extension a serving loop would use directly.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <memory>
#include <optional>
#include <string>
#include <utility>
#include <vector>

namespace zllm_amd {

struct BackendError {
    enum class Kind { UnsupportedLayer, ExpertLoad, Compute };
    Kind kind = Kind::Compute;
    size_t layer = 0;
    std::string msg;
    std::string to_string() const;
};

// Rust's Result<T, BackendError>: either a value or an error, never both.
template <class T> class Result {
  public:
    Result(T value) : value_(std::move(value)) {}
    Result(BackendError error) : error_(std::move(error)) {}
    bool is_ok() const { return value_.has_value(); }
    bool is_err() const { return !value_.has_value(); }
    T& unwrap() { return *value_; }
    const T& unwrap() const { return *value_; }
    const BackendError& unwrap_err() const { return error_; }

  private:
    std::optional<T> value_;
    BackendError error_;
};
struct Unit {};

struct CausalWindow {
    bool sliding = false;
    size_t size = 0;
    static CausalWindow Full() { return CausalWindow{}; }
    static CausalWindow Sliding(size_t size) { return CausalWindow{true, size}; }
    // [start, end) of the keys a query at `query_position` sees among `key_end` cached keys
    std::pair<size_t, size_t> key_range(size_t query_position, size_t key_end) const;
    size_t cache_capacity(size_t max_sequence_len) const;
};

struct GqaSpec {
    size_t num_heads = 0, num_kv_heads = 0, head_dim = 0, rope_dim = 0;
    float rope_theta = 10000.0f;
    bool use_qk_norm = false;
    CausalWindow window;
    float score_scale = 0.0f;
    bool output_gate = false;
    size_t group_size() const { return num_heads / num_kv_heads; }
};

// Head geometry and explicit per-row visible ranges of the model-independent block attention
// (GqaGeometry, src/attention/gqa.rs:11-37; BlockAttentionSpec, src/attention/block.rs:10-63).
struct GqaGeometry {
    size_t num_heads = 0, num_kv_heads = 0, head_dim = 0;
    std::optional<std::string> validate() const;
};

struct BlockAttentionSpec {
    GqaGeometry geometry;
    float score_scale = 0.0f;
    std::vector<std::pair<size_t, size_t>> visible; // [start, end) of the KV rows each query row sees
    std::optional<std::string> validate(size_t query_rows, size_t kv_rows) const;
    static BlockAttentionSpec full(GqaGeometry geometry, size_t query_rows, size_t kv_rows, float score_scale);
    // two prefix sums cut the rows into isolated sequences: the rows of query segment i see the KV rows of segment i
    static Result<BlockAttentionSpec> varlen(GqaGeometry geometry, size_t query_rows, size_t kv_rows, const std::vector<size_t>& query_offsets,
                                             const std::vector<size_t>& kv_offsets, float score_scale);
};

enum class RotaryLayout { SplitHalf, Interleaved };

struct MlaSpec {
    size_t q_lora_rank = 0, kv_lora_rank = 0, qk_rope_head_dim = 0, q_projection_size = 0, kv_projection_size = 0, num_heads = 0;
    float rope_theta = 10000.0f;
    RotaryLayout rotary_layout = RotaryLayout::SplitHalf;
    std::optional<std::string> validate() const; // message when the dimensions are inconsistent
    size_t q_head_dim() const { return q_projection_size / num_heads; }
    size_t qk_nope_dim() const { return q_head_dim() - qk_rope_head_dim; }
    size_t kv_head_dim() const { return kv_projection_size / num_heads; }
    size_t value_dim() const { return kv_head_dim() - qk_nope_dim(); }
    size_t kv_a_out() const { return kv_lora_rank + qk_rope_head_dim; }
};

// Sparse-attention (DSA) parameters the selected-token decode needs (src/attention/dsa.rs): the list length.
struct DsaSpec {
    size_t top_k = 0;
};

enum class DType { F32 = 0, BF16 = 1, F16 = 2 };
size_t dtype_bytes(DType dtype);

// Device buffer with shared ownership.  allocate() is hipMalloc / hipFree; a buffer a RocmContext hands out (outputs,
// staged uploads, scratch planes) comes from that context's pool and goes back to it when the last owner lets go.
class DeviceBuffer {
  public:
    static Result<DeviceBuffer> allocate(size_t bytes);
    static DeviceBuffer adopt(std::shared_ptr<void> block, size_t bytes);
    void* data() const { return ptr_.get(); }
    size_t bytes() const { return bytes_; }

  private:
    std::shared_ptr<void> ptr_;
    size_t bytes_ = 0;
};

// Row-major device tensor (the reference's RocmTensor with a resident device buffer).
struct RocmTensor {
    DeviceBuffer device;
    size_t rows = 0, cols = 0;
    DType dtype = DType::F32;
};

// kv_b resident on the device (the reference's RocmWeight): bf16, or the W8A16 / W4A16 form of RocmQuantizedWeight
// (src/backend/rocm/attention.rs:181-192) -- codes packed low bits first into 32-bit words, a scale per row and
// `group_size` columns.
struct RocmWeight {
    DeviceBuffer device;
    size_t rows = 0, cols = 0;
    unsigned bits = 16;       // 16 bf16, 32 f32, 8 / 4 codes
    DeviceBuffer scales;      // 8 / 4 bits only
    size_t group_size = 0;
    DType scale_dtype = DType::BF16;
};

// What the reference's DsaState hands to the selected-token decode: the token positions the indexer chose for the
// current query row, `top_k` per row, resident on the device.  The indexer itself (scores, radix top-k) is outside
// this path; a state is built from a list here.
struct RocmDsaState {
    DeviceBuffer selection; // u32 [top_k]
    size_t top_k = 0;
};

enum class KvCacheFormat { F16, Q8g64 };

// How a cache hands out pages.  Identity is the reference's policy (block i -> physical block i, one table built at
// full capacity, src/backend/rocm/mod.rs:335-379): planes then start small and grow by doubling.  Scrambled places
// the pages in a fixed pseudo-random order over the whole pool, which commits the pool up front; it exists to drive
// the kernels through a table that is not the identity.
enum class TablePolicy { Identity, Scrambled };

// Rows a cache plane holds after an append that needs `required` of at most `limit` rows: unchanged when it already
// holds them, else the larger of `required`, twice `current` and 64, rounded up to 64 rows and capped at `limit`
// (committed_cache_rows, src/backend/rocm/mod.rs:303-313).
Result<size_t> committed_cache_rows(size_t current, size_t required, size_t limit);

enum class RocmKvOwnership { Full = 0, BlockParity0 = 1, BlockParity1 = 2, InterleavedPair = 3 };

// Host form of one MLA layer for session snapshots (the reference's MlaLayerSerde, src/backend/rocm/kv_cache.rs:2067-2083):
// plain bytes + shape, no device handles.
struct MlaLayerSerde {
    size_t rows = 0;
    RocmKvOwnership ownership = RocmKvOwnership::Full;
    size_t latent_cols = 0, rope_cols = 0;
    size_t latent_group_size = 0;                     // 0 = bf16 latent without scales, else the Q8 group size
    std::vector<uint8_t> latent;                      // Q8: rows x latent_cols
    std::optional<std::vector<uint8_t>> latent_scales; // Q8: rows x (latent_cols / group) x 2
    std::vector<uint8_t> rope;                        // rows x rope_cols x 2 (bf16)
};
// write_mla_layer / read_mla_layer (src/runtime/glm52/rocm_swap.rs:1090-1138): `write` appends to `out`; `read` parses one
// record at `offset` and advances it.
Result<Unit> write_mla_layer(std::vector<uint8_t>& out, const MlaLayerSerde& layer);
Result<MlaLayerSerde> read_mla_layer(const std::vector<uint8_t>& in, size_t& offset);

// Paged KV cache of one sequence: planar code / scale planes per layer plus one block table.
class RocmKvCache {
  public:
    // Q8g64 GQA cache: K codes, K scales (f16), V codes, V scales per layer
    static Result<RocmKvCache> new_gqa(size_t layers, size_t num_kv_heads, size_t head_dim, size_t block_tokens, size_t max_tokens,
                                       TablePolicy policy = TablePolicy::Identity);
    // MLA cache: Q8g64 latent (bf16 scales) + bf16 rope per layer
    static Result<RocmKvCache> new_mla(size_t layers, size_t latent_dim, size_t rope_dim, size_t block_tokens, size_t max_tokens,
                                       TablePolicy policy = TablePolicy::Identity);
    size_t len(size_t layer) const { return layer < lens_.size() ? lens_[layer] : 0; }
    // rows the layer's planes hold right now (grows with the appends under TablePolicy::Identity)
    size_t committed_rows(size_t layer) const { return layer < layers_.size() ? layers_[layer].committed_rows : 0; }
    // 0, or the number of rows a sliding-window layer keeps as a ring (token t in slot t % capacity)
    size_t ring_capacity(size_t layer) const { return layer < layers_.size() ? layers_[layer].ring_capacity : 0; }
    // Rollback: only the logical length moves, pages and the kept prefix stay where they are and the next append
    // overwrites the tail (truncate_rows / truncate_layer_rows, src/backend/rocm/kv_cache.rs:509-586).
    Result<Unit> truncate_rows(size_t rows);
    Result<Unit> truncate_layer_rows(size_t layer, size_t rows);
    size_t layers() const { return lens_.size(); }
    size_t block_tokens() const { return block_tokens_; }
    size_t max_tokens() const { return max_tokens_; }
    const std::vector<uint32_t>& block_table() const { return table_host_; }

  private:
    friend class RocmContext;
    struct Layer {
        DeviceBuffer a_codes, a_scales, b_codes, b_scales; // GQA: K, V; MLA: latent codes / scales, rope in b_codes
        size_t committed_rows = 0;
        size_t ring_capacity = 0;
    };
    static Result<RocmKvCache> create(bool mla, size_t layers, size_t cols, size_t rope_cols, size_t block_tokens, size_t max_tokens,
                                      TablePolicy policy);
    // bytes of one row in each of the layer's planes (0 = plane unused)
    void plane_row_bytes(size_t (&bytes)[4]) const;
    // make the layer's planes hold `required` rows (grow_cache_buffer, src/backend/rocm/mod.rs:315-322: a larger
    // buffer, the used prefix copied device to device on `stream`)
    Result<Unit> reserve_rows(size_t layer, size_t required, hipStream_t stream);
    bool mla_ = false;
    TablePolicy policy_ = TablePolicy::Identity;
    size_t cols_ = 0, rope_cols_ = 0, block_tokens_ = 0, max_tokens_ = 0, pool_rows_ = 0;
    std::vector<Layer> layers_;
    std::vector<size_t> lens_;
    std::vector<uint32_t> table_host_;
    DeviceBuffer table_;
};

// What a context did on the host side so far; a serving loop in steady state moves none of the first three.
struct HostCounters {
    size_t device_allocations = 0;  // hipMalloc calls made for pooled buffers, the workspace and resident tables
    size_t rope_table_uploads = 0;  // uploads of a cos/sin prefix
    size_t stream_waits = 0;        // hipStreamSynchronize calls made inside attention and append methods
    size_t staged_uploads = 0;      // small host arrays (visible ends, selections) sent through the pinned ring
};

// One context drives one HIP stream and keeps that stream's scratch.  A context and its copies (they share the scratch)
// belong to one thread at a time; a thread that wants a stream of its own creates a context of its own, which is the
// reference's model as well -- its active device and stream are thread-local (src/kernel/rocm/hip/mod.rs:15-50).
// Tensors and buffers a context handed out may be dropped on any thread.
class RocmContext {
  public:
    static Result<RocmContext> create(int device_id);
    HostCounters counters() const;
    int device_id() const { return device_id_; }
    hipStream_t stream() const { return stream_; }
    Result<Unit> synchronize() const;

    Result<RocmTensor> tensor_from_f32(const std::vector<float>& host, size_t rows, size_t cols, DType dtype = DType::F32) const;
    Result<std::vector<float>> tensor_to_f32(const RocmTensor& tensor) const;
    // DecodeBackend::prepare_mla_kv_b: kv_b [heads * kv_head_dim, latent] -> bf16 on the device
    Result<RocmWeight> prepare_mla_kv_b(const std::vector<float>& weight, size_t rows, size_t cols) const;
    // The same weight quantized on the way in: 8- or 4-bit codes with one bf16 scale per row and `group_size` columns
    // (scale = largest magnitude of the group / 127 or / 7, rounded to bf16; code = round(value / scale) + 128 or + 8).
    Result<RocmWeight> prepare_mla_kv_b_quantized(const std::vector<float>& weight, size_t rows, size_t cols, unsigned bits,
                                                  size_t group_size) const;
    // What a quantized weight's codes stand for, as f32 [rows, cols] (for callers that check against a CPU reference).
    Result<std::vector<float>> dequantized_kv_b(const RocmWeight& weight) const;

    // Backend::gqa_prefill_attention (src/backend/mod.rs:1477; ROCm body src/backend/rocm/attention.rs:2151-2170): causal
    // attention of a chunk over its own K/V, nothing cached.  K and V go to dense f16 scratch planes on the way in.
    Result<RocmTensor> gqa_prefill_attention(const RocmTensor& query, const RocmTensor& key, const RocmTensor& value, const GqaSpec& spec) const;
    // The same with a visible end per row (right-padded text encoders; src/backend/mod.rs:1479-1482).
    Result<RocmTensor> gqa_prefill_attention_visible(const RocmTensor& query, const RocmTensor& key, const RocmTensor& value, const GqaSpec& spec,
                                                     const std::vector<uint32_t>& visible_ends) const;
    // BlockAttentionBackend::block_attention (src/backend/mod.rs:1582-1584; ROCm body src/backend/rocm/attention.rs:118-144):
    // query and KV lengths differ, every query row sees exactly its range.  Returns f32 [query.rows, num_heads * head_dim].
    Result<RocmTensor> block_attention(const RocmTensor& query, const RocmTensor& key, const RocmTensor& value, const BlockAttentionSpec& spec) const;
    // block_attention_segments (src/backend/mod.rs:1586-1598): the KV rows arrive as several tensors in order; each is
    // written behind the one before it into the scratch planes, no concatenated copy is made on the way.
    Result<RocmTensor> block_attention_segments(const RocmTensor& query, const std::vector<const RocmTensor*>& keys,
                                                const std::vector<const RocmTensor*>& values, const BlockAttentionSpec& spec) const;
    // block_attention_prefix_suffix (src/backend/mod.rs:1601-1616): the KV rows are a resident prefix followed by this
    // step's short suffix; the two are written one behind the other into the scratch planes, never concatenated on the host.
    Result<RocmTensor> block_attention_prefix_suffix(const RocmTensor& query, const RocmTensor& prefix_key, const RocmTensor& prefix_value,
                                                     const RocmTensor& suffix_key, const RocmTensor& suffix_value,
                                                     const BlockAttentionSpec& spec) const;
    // Appends the chunk's K/V rows at `position` (must equal the layer's cached length), then attends:
    // one row -> split-KV decode, more rows -> chunked prefill (causal, optional sliding window).
    // Returns f32 [rows, num_heads * head_dim].  A sliding-window layer appended with retain_full_cache == false keeps
    // only CausalWindow::cache_capacity rows, as a ring (HybridGqaCacheLayout, src/kv_cache/mod.rs:397-456); such a layer
    // takes a multi-row chunk at position 0 only, as the reference's CPU backend does (src/backend/cpu/attention.rs:401-409).
    // The cache length moves only after every launch of the call was accepted.
    Result<RocmTensor> gqa_prefill_attention_cached(RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& query,
                                                    const RocmTensor& key, const RocmTensor& value, const GqaSpec& spec,
                                                    bool retain_full_cache) const;
    // The same with explicit visible ends per chunk row (multimodal blocks; src/backend/mod.rs:1495-1511).
    Result<RocmTensor> gqa_prefill_attention_cached_visible(RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& query,
                                                            const RocmTensor& key, const RocmTensor& value, const GqaSpec& spec,
                                                            const std::vector<uint32_t>& visible_ends, bool retain_full_cache) const;
    // Attention of a layer that shares another layer's K/V (src/backend/mod.rs:1513): nothing is appended, the source
    // layer must already hold position + rows rows.
    Result<RocmTensor> gqa_prefill_attention_cached_from(const RocmKvCache& cache, size_t source_layer, size_t position, const RocmTensor& query,
                                                         const GqaSpec& spec) const;
    // The shared-KV form with visible ends (visual blocks on a shared layer; src/backend/mod.rs:1575-1578).
    Result<RocmTensor> gqa_prefill_attention_cached_from_visible(const RocmKvCache& cache, size_t source_layer, size_t position,
                                                                 const RocmTensor& query, const GqaSpec& spec,
                                                                 const std::vector<uint32_t>& visible_ends) const;
    // MlaPrefillBackend: append the chunk, then attend with one query row per chunk row (causal inside the chunk).
    // Returns bf16 [rows, heads * value_dim] for more than one row, f32 for one (src/backend/rocm/attention.rs:17-19).
    Result<RocmTensor> mla_prefill_attention(const RocmTensor& query, const RocmTensor& latent, const RocmTensor& k_rope, const RocmWeight& kv_b,
                                             RocmKvCache* cache, size_t layer, const MlaSpec& spec) const;
    Result<RocmTensor> mla_prefill_attention_rope(const RocmTensor& query, const RocmTensor& latent, const RocmTensor& k_rope, const RocmWeight& kv_b,
                                                  RocmKvCache* cache, size_t layer, size_t position, const std::vector<float>& cos,
                                                  const std::vector<float>& sin, const MlaSpec& spec) const;
    Result<Unit> append_mla(RocmKvCache& cache, size_t layer, const RocmTensor& latent, const RocmTensor& rope) const;
    Result<Unit> append_mla_rope(RocmKvCache& cache, size_t layer, const RocmTensor& latent, const RocmTensor& rope, size_t rotary_dim,
                                 RotaryLayout layout, size_t position, const std::vector<float>& cos, const std::vector<float>& sin) const;
    // Session snapshot of an MLA cache (download_layers, src/backend/rocm/kv_cache.rs:3344-3388): every layer's rows
    // [0, len) gathered through the block table into host bytes; and its inverse, into whatever pages `cache` owns.
    Result<std::vector<std::optional<MlaLayerSerde>>> download_layers(const RocmKvCache& cache) const;
    Result<Unit> upload_layers(RocmKvCache& cache, const std::vector<std::optional<MlaLayerSerde>>& layers) const;
    // query [1, heads * q_head_dim]; returns f32 [1, heads * value_dim]
    Result<RocmTensor> mla_decode_attention(const RocmTensor& query, const RocmKvCache& cache, const RocmWeight& kv_b, size_t layer,
                                            size_t position, const MlaSpec& spec) const;
    // DecodeBackend::mla_decode_attention_selected (src/backend/mod.rs:1227, ROCm body src/backend/rocm/attention.rs:1927-1940):
    // a context longer than dsa.top_k attends to the positions in `state` only, a shorter one stays dense.
    Result<RocmTensor> mla_decode_attention_selected(const RocmTensor& query, const RocmKvCache& cache, const RocmWeight& kv_b, size_t layer,
                                                     size_t position, const MlaSpec& mla, const DsaSpec& dsa, const RocmDsaState& state) const;
    Result<RocmDsaState> dsa_state_from_selection(const std::vector<uint32_t>& selection) const;

  private:
    // Device scratch of the context's stream, kept between calls: the split-KV workspace (grown when a call needs
    // more), a ring of small metadata records (lengths, window starts) and a ring for small arrays (visible ends,
    // selections) that travel host -> device from pinned memory, a pool that output tensors and scratch planes are
    // taken from and returned to, an identity block table and the cos/sin tables already on the device -- so that a
    // call in steady state neither allocates nor waits for the stream.  Blocks are reused in stream order: everything
    // the context launches runs on its one stream, so a block that went back to the pool is next written by work
    // queued behind its last reader.
    struct Scratch;
    Result<void*> workspace(size_t bytes) const;
    Result<const uint32_t*> upload_meta(const uint32_t (&values)[4]) const;
    Result<DeviceBuffer> pooled(size_t bytes) const;
    Result<DeviceBuffer> upload_words(const uint32_t* words, size_t count) const;
    Result<const uint32_t*> identity_table(size_t pages) const;
    // cos/sin of a model live on the device once per host table (keyed like the reference's table cache,
    // src/backend/rocm/compressed_sparse.rs:20-36,323-348): the committed prefix doubles as positions arrive
    Result<std::pair<const float*, const float*>> resident_rope_tables(const std::vector<float>& cos, const std::vector<float>& sin,
                                                                       size_t required) const;
    Result<Unit> wait_for_stream() const;
    // dense rows -> f16 scratch planes [pages * 64, cols] behind the identity table; `parts` are written one behind the other
    struct DensePlanes;
    Result<DensePlanes> dense_f16_planes(const std::vector<const RocmTensor*>& keys, const std::vector<const RocmTensor*>& values, size_t cols,
                                         size_t cache_rows) const;
    Result<RocmTensor> attend_dense(const RocmTensor& query, const DensePlanes& planes, size_t position, const GqaGeometry& geometry,
                                    float score_scale, size_t window, const uint32_t* starts_dev, const uint32_t* ends_dev) const;
    Result<Unit> append_gqa_rows(RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& key, const RocmTensor& value) const;
    Result<RocmTensor> gqa_attend(const RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& query, const GqaSpec& spec,
                                  const uint32_t* visible_ends_dev) const;
    Result<RocmTensor> gqa_cached_impl(RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& query, const RocmTensor& key,
                                       const RocmTensor& value, const GqaSpec& spec, const std::vector<uint32_t>* visible_ends,
                                       bool retain_full_cache) const;
    Result<RocmTensor> mla_decode_impl(const RocmTensor& query, const RocmKvCache& cache, const RocmWeight& kv_b, size_t layer, size_t position,
                                       const MlaSpec& spec, const RocmDsaState* state) const;
    std::shared_ptr<Scratch> scratch_;
    Result<Unit> append_mla_impl(RocmKvCache& cache, size_t layer, const RocmTensor& latent, const RocmTensor& rope, size_t rotary_dim,
                                 RotaryLayout layout, size_t position, const float* cos_dev, const float* sin_dev) const;
    int device_id_ = 0;
    hipStream_t stream_ = nullptr;
};

} // namespace zllm_amd

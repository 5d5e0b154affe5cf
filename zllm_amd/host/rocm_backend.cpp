// Implementation of the host-side backend mirror over the C ABI.  Device memory comes from hipMalloc here
// (the C ABI itself never allocates); every attention call runs on the context's stream.
#include "rocm_backend.hpp"

#include <math.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <numeric>

#include "../../include/zllm_attn.h"

namespace zllm_amd {

namespace {

BackendError compute_error(std::string msg)
{
    BackendError e;
    e.kind = BackendError::Kind::Compute;
    e.msg = std::move(msg);
    return e;
}

BackendError hip_error(const char* what, hipError_t err)
{
    return compute_error(std::string(what) + ": " + hipGetErrorString(err));
}

BackendError abi_error(const char* what, int code)
{
    return compute_error(std::string(what) + ": " + zllm_attn_last_error() + " (code " + std::to_string(code) + ")");
}

uint16_t f32_to_bf16_bits(float value)
{
    uint32_t bits;
    memcpy(&bits, &value, 4);
    const uint32_t rounding = 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)((bits + rounding) >> 16);
}

float bf16_bits_to_f32(uint16_t v)
{
    const uint32_t bits = (uint32_t)v << 16;
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

// IEEE binary16 <-> binary32 (round to nearest even), for host-side tensor conversion only
uint16_t f32_to_f16_bits(float value)
{
    const _Float16 h = (_Float16)value;
    uint16_t out;
    memcpy(&out, &h, 2);
    return out;
}

float f16_bits_to_f32(uint16_t v)
{
    _Float16 h;
    memcpy(&h, &v, 2);
    return (float)h;
}

int abi_dtype(DType dtype)
{
    return dtype == DType::F32 ? ZLLM_DTYPE_F32 : dtype == DType::BF16 ? ZLLM_DTYPE_BF16 : ZLLM_DTYPE_F16;
}

} // namespace

std::string BackendError::to_string() const
{
    switch (kind) {
    case Kind::UnsupportedLayer: return "unsupported model layer L" + std::to_string(layer);
    case Kind::ExpertLoad: return "expert load failed: " + msg;
    default: return "backend compute failed: " + msg;
    }
}

std::pair<size_t, size_t> CausalWindow::key_range(size_t query_position, size_t key_end) const
{
    const size_t end = std::min(query_position + 1, key_end);
    size_t start = 0;
    if (sliding) {
        start = query_position + 1 > size ? query_position + 1 - size : 0;
    }
    return {std::min(start, end), end};
}

size_t CausalWindow::cache_capacity(size_t max_sequence_len) const
{
    return sliding ? std::min(size, max_sequence_len) : max_sequence_len;
}

std::optional<std::string> MlaSpec::validate() const
{
    if (num_heads == 0 || q_projection_size % num_heads != 0 || kv_projection_size % num_heads != 0) {
        return "MLA head dimensions invalid: q_proj=" + std::to_string(q_projection_size) + " kv_proj=" + std::to_string(kv_projection_size) +
               " heads=" + std::to_string(num_heads);
    }
    if (qk_rope_head_dim > 0 && (qk_rope_head_dim % 2 != 0 || !isfinite(rope_theta) || rope_theta <= 0.0f)) {
        return "MLA RoPE parameters invalid: rope_dim=" + std::to_string(qk_rope_head_dim);
    }
    if (qk_rope_head_dim > q_head_dim()) {
        return "MLA rope dim " + std::to_string(qk_rope_head_dim) + " exceeds query head dim " + std::to_string(q_head_dim());
    }
    if (qk_nope_dim() > kv_head_dim()) {
        return "MLA nope dim " + std::to_string(qk_nope_dim()) + " exceeds KV head dim " + std::to_string(kv_head_dim());
    }
    return std::nullopt;
}

size_t dtype_bytes(DType dtype)
{
    return dtype == DType::F32 ? 4 : 2;
}

Result<DeviceBuffer> DeviceBuffer::allocate(size_t bytes)
{
    void* raw = nullptr;
    const hipError_t err = hipMalloc(&raw, std::max<size_t>(bytes, 256));
    if (err != hipSuccess) {
        return hip_error("hipMalloc", err);
    }
    DeviceBuffer out;
    out.ptr_ = std::shared_ptr<void>(raw, [](void* p) { (void)hipFree(p); });
    out.bytes_ = bytes;
    return out;
}

DeviceBuffer DeviceBuffer::adopt(std::shared_ptr<void> block, size_t bytes)
{
    DeviceBuffer out;
    out.ptr_ = std::move(block);
    out.bytes_ = bytes;
    return out;
}

// ------------------------------------------------------------------------------------------------ cache
namespace {

// Pages are handed out in a fixed scrambled order so that the block table is never the identity.
std::vector<uint32_t> scrambled_pages(size_t pages)
{
    std::vector<uint32_t> ids(pages);
    std::iota(ids.begin(), ids.end(), 0u);
    uint64_t state = 0x9e3779b97f4a7c15ull;
    for (size_t i = pages; i > 1; --i) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        std::swap(ids[i - 1], ids[(size_t)((state >> 33) % i)]);
    }
    return ids;
}

} // namespace

Result<size_t> committed_cache_rows(size_t current, size_t required, size_t limit)
{
    constexpr size_t kBlock = 64; // ROCM_KV_BLOCK_SIZE (src/backend/rocm/mod.rs:301)
    if (required == 0 || required > limit) {
        return compute_error("ROCm cache required=" + std::to_string(required) + " exceeds the logical limit " + std::to_string(limit));
    }
    if (current >= required) {
        return current;
    }
    const size_t target = std::max(std::max(required, current * 2), kBlock);
    const size_t aligned = (target + kBlock - 1) / kBlock * kBlock;
    return std::max(std::min(aligned, limit), required);
}

void RocmKvCache::plane_row_bytes(size_t (&bytes)[4]) const
{
    if (mla_) {
        bytes[0] = cols_;
        bytes[1] = cols_ / 64 * 2;
        bytes[2] = rope_cols_ * 2;
        bytes[3] = 0;
    } else {
        bytes[0] = cols_;
        bytes[1] = cols_ / 64 * 2;
        bytes[2] = cols_;
        bytes[3] = cols_ / 64 * 2;
    }
}

Result<RocmKvCache> RocmKvCache::create(bool mla, size_t layers, size_t cols, size_t rope_cols, size_t block_tokens, size_t max_tokens,
                                        TablePolicy policy)
{
    RocmKvCache cache;
    cache.mla_ = mla;
    cache.policy_ = policy;
    cache.cols_ = cols;
    cache.rope_cols_ = rope_cols;
    cache.block_tokens_ = block_tokens;
    cache.max_tokens_ = max_tokens;
    const size_t pages = (max_tokens + block_tokens - 1) / block_tokens;
    if (pages > UINT32_MAX) {
        return compute_error("ROCm KV block ID exceeds u32");
    }
    cache.pool_rows_ = pages * block_tokens;
    // the table is built once, at full capacity: rebuilding it as the cache grows would put an upload and a stream
    // synchronisation on every page boundary of a decode loop (src/backend/rocm/mod.rs:353-356)
    if (policy == TablePolicy::Identity) {
        cache.table_host_.resize(pages);
        std::iota(cache.table_host_.begin(), cache.table_host_.end(), 0u);
    } else {
        cache.table_host_ = scrambled_pages(pages);
    }
    auto table = DeviceBuffer::allocate(pages * 4);
    if (table.is_err()) {
        return table.unwrap_err();
    }
    cache.table_ = table.unwrap();
    const hipError_t err = hipMemcpy(cache.table_.data(), cache.table_host_.data(), pages * 4, hipMemcpyHostToDevice);
    if (err != hipSuccess) {
        return hip_error("block table upload", err);
    }
    cache.layers_.resize(layers);
    cache.lens_.assign(layers, 0);
    if (policy == TablePolicy::Scrambled) { // any page may be named from the first append on: commit the pool
        for (size_t l = 0; l < layers; ++l) {
            auto done = cache.reserve_rows(l, cache.pool_rows_, nullptr);
            if (done.is_err()) {
                return done.unwrap_err();
            }
        }
    }
    return cache;
}

Result<Unit> RocmKvCache::reserve_rows(size_t layer, size_t required, hipStream_t stream)
{
    Layer& planes = layers_[layer];
    if (planes.committed_rows >= required) {
        return Unit{};
    }
    auto rows_r = committed_cache_rows(planes.committed_rows, required, pool_rows_);
    if (rows_r.is_err()) {
        return rows_r.unwrap_err();
    }
    // whole pages: a page's rows are addressed through its table entry
    const size_t rows = std::min((rows_r.unwrap() + block_tokens_ - 1) / block_tokens_ * block_tokens_, pool_rows_);
    size_t row_bytes[4];
    plane_row_bytes(row_bytes);
    DeviceBuffer* buffers[4] = {&planes.a_codes, &planes.a_scales, &planes.b_codes, &planes.b_scales};
    for (int i = 0; i < 4; ++i) {
        if (row_bytes[i] == 0) {
            continue;
        }
        auto grown = DeviceBuffer::allocate(rows * row_bytes[i]);
        if (grown.is_err()) {
            return grown.unwrap_err();
        }
        if (planes.committed_rows != 0) {
            // under the identity table the used rows are a prefix of the plane
            hipError_t err = hipMemcpyAsync(grown.unwrap().data(), buffers[i]->data(), planes.committed_rows * row_bytes[i], hipMemcpyDeviceToDevice, stream);
            if (err == hipSuccess) {
                err = hipStreamSynchronize(stream); // the old plane is released below
            }
            if (err != hipSuccess) {
                return hip_error("cache growth copy", err);
            }
        }
        *buffers[i] = grown.unwrap();
    }
    planes.committed_rows = rows;
    return Unit{};
}

Result<RocmKvCache> RocmKvCache::new_gqa(size_t layers, size_t num_kv_heads, size_t head_dim, size_t block_tokens, size_t max_tokens,
                                         TablePolicy policy)
{
    const size_t cols = num_kv_heads * head_dim;
    if (layers == 0 || cols == 0 || cols % 64 != 0 || block_tokens == 0 || max_tokens == 0) {
        return compute_error("Rocm GQA cache: invalid geometry");
    }
    return create(false, layers, cols, 0, block_tokens, max_tokens, policy);
}

Result<RocmKvCache> RocmKvCache::new_mla(size_t layers, size_t latent_dim, size_t rope_dim, size_t block_tokens, size_t max_tokens,
                                         TablePolicy policy)
{
    if (layers == 0 || latent_dim == 0 || latent_dim % 64 != 0 || rope_dim == 0 || block_tokens == 0 || max_tokens == 0) {
        return compute_error("Rocm MLA cache: invalid geometry");
    }
    return create(true, layers, latent_dim, rope_dim, block_tokens, max_tokens, policy);
}

Result<Unit> RocmKvCache::truncate_rows(size_t rows)
{
    if (rows > max_tokens_) {
        return compute_error("ROCm KV truncate rows=" + std::to_string(rows) + " exceeds the logical limit " + std::to_string(max_tokens_));
    }
    for (size_t layer = 0; layer < lens_.size(); ++layer) {
        if (rows > lens_[layer]) {
            return compute_error("L" + std::to_string(layer) + " ROCm KV truncate rows=" + std::to_string(rows) + " exceeds the current length " +
                                 std::to_string(lens_[layer]));
        }
    }
    for (size_t& len : lens_) {
        len = rows;
    }
    return Unit{};
}

Result<Unit> RocmKvCache::truncate_layer_rows(size_t layer, size_t rows)
{
    if (rows > max_tokens_) {
        return compute_error("L" + std::to_string(layer) + " ROCm KV truncate rows=" + std::to_string(rows) + " exceeds the logical limit " +
                             std::to_string(max_tokens_));
    }
    if (layer >= lens_.size()) {
        return BackendError{BackendError::Kind::UnsupportedLayer, layer, ""};
    }
    if (rows > lens_[layer]) {
        return compute_error("L" + std::to_string(layer) + " ROCm KV truncate rows=" + std::to_string(rows) + " exceeds the current length " +
                             std::to_string(lens_[layer]));
    }
    lens_[layer] = rows;
    return Unit{};
}

// ---------------------------------------------------------------------------------------------- snapshot wire format
Result<Unit> write_mla_layer(std::vector<uint8_t>& out, const MlaLayerSerde& layer)
{
    zllm_mla_layer_record rec;
    memset(&rec, 0, sizeof(rec));
    rec.rows = layer.rows;
    rec.ownership = (uint32_t)layer.ownership;
    rec.latent_cols = layer.latent_cols;
    rec.rope_cols = layer.rope_cols;
    rec.latent_group_size = layer.latent_group_size;
    static const uint8_t empty = 0;
    rec.latent = layer.latent.empty() ? &empty : layer.latent.data();
    rec.latent_bytes = layer.latent.size();
    if (layer.latent_scales.has_value()) {
        rec.latent_scales = layer.latent_scales->empty() ? &empty : layer.latent_scales->data();
        rec.latent_scales_bytes = layer.latent_scales->size();
    }
    rec.rope = layer.rope.empty() ? &empty : layer.rope.data();
    rec.rope_bytes = layer.rope.size();
    const uint64_t need = zllm_kv_mla_layer_wire_bytes(&rec);
    if (need == 0) {
        return compute_error("GLM cache MLA layer: blob lengths do not match the shape");
    }
    const size_t at = out.size();
    out.resize(at + need);
    uint64_t written = 0;
    const int code = zllm_kv_mla_layer_write(&rec, out.data() + at, need, &written);
    if (code != 0) {
        out.resize(at);
        return abi_error("zllm_kv_mla_layer_write", code);
    }
    return Unit{};
}

Result<MlaLayerSerde> read_mla_layer(const std::vector<uint8_t>& in, size_t& offset)
{
    if (offset > in.size()) {
        return compute_error("GLM cache MLA layer: offset past the end");
    }
    zllm_mla_layer_record rec;
    uint64_t used = 0;
    const int code = zllm_kv_mla_layer_read(in.data() + offset, in.size() - offset, &rec, &used);
    if (code != 0) {
        return abi_error("zllm_kv_mla_layer_read", code);
    }
    MlaLayerSerde layer;
    layer.rows = rec.rows;
    layer.ownership = (RocmKvOwnership)rec.ownership;
    layer.latent_cols = rec.latent_cols;
    layer.rope_cols = rec.rope_cols;
    layer.latent_group_size = rec.latent_group_size;
    layer.latent.assign(rec.latent, rec.latent + rec.latent_bytes);
    if (rec.latent_scales != nullptr) {
        layer.latent_scales = std::vector<uint8_t>(rec.latent_scales, rec.latent_scales + rec.latent_scales_bytes);
    }
    layer.rope.assign(rec.rope, rec.rope + rec.rope_bytes);
    offset += used;
    return layer;
}

// ---------------------------------------------------------------------------------------------- context
struct RocmContext::Scratch {
    static constexpr size_t kSlots = 256;
    static constexpr size_t kStageBytes = 1 << 20;       // pinned ring for small arrays
    static constexpr size_t kPoolKeepBytes = 2ull << 30; // idle blocks kept beyond this are released
    hipStream_t stream = nullptr;
    DeviceBuffer workspace;
    uint32_t* meta_host = nullptr; // pinned, kSlots records of four u32
    DeviceBuffer meta_dev;
    size_t next = 0;
    uint8_t* stage_host = nullptr; // pinned, kStageBytes
    size_t stage_next = 0;
    // idle blocks by capacity; a block is reused for a request of at least half its size.  Tensors may be dropped on any
    // thread, so the map has a lock of its own; everything else here belongs to the thread that drives the context.
    std::mutex pool_lock;
    std::multimap<size_t, void*> idle;
    size_t idle_bytes = 0;
    DeviceBuffer identity;         // u32 [identity_pages]: 0, 1, 2, ...
    size_t identity_pages = 0;
    struct RopeTables {
        const float *cos_host, *sin_host; // identity of the host tables, as the reference keys them
        size_t host_elements, elements;   // length of the host tables, committed prefix
        float first, last;                // cos[0] and cos[elements - 1] when committed: a reused address is told apart
        DeviceBuffer cos, sin;
    };
    std::vector<RopeTables> rope;
    HostCounters counters;
    ~Scratch()
    {
        if (meta_host != nullptr) {
            (void)hipHostFree(meta_host);
        }
        if (stage_host != nullptr) {
            (void)hipHostFree(stage_host);
        }
        for (auto& block : idle) {
            (void)hipFree(block.second);
        }
    }
    static size_t size_class(size_t bytes)
    {
        // powers of two up to 1 MiB, then multiples of 1 MiB: a decode loop's outputs all land in one class
        size_t cls = 256;
        while (cls < bytes && cls < (1u << 20)) {
            cls *= 2;
        }
        return cls >= bytes ? cls : (bytes + (1u << 20) - 1) >> 20 << 20;
    }
    void give_back(void* block, size_t capacity)
    {
        {
            std::lock_guard<std::mutex> hold(pool_lock);
            if (idle_bytes + capacity <= kPoolKeepBytes) {
                idle.emplace(capacity, block);
                idle_bytes += capacity;
                return;
            }
        }
        (void)hipFree(block);
    }
};

Result<RocmContext> RocmContext::create(int device_id)
{
    int cus = 0;
    const int rc = zllm_attn_init(device_id, &cus);
    if (rc != 0) {
        return abi_error("zllm_attn_init", rc);
    }
    RocmContext ctx;
    ctx.device_id_ = device_id;
    hipError_t err = hipSetDevice(device_id);
    if (err == hipSuccess) {
        err = hipStreamCreate(&ctx.stream_); // default priority
    }
    if (err != hipSuccess) {
        return hip_error("stream", err);
    }
    auto scratch = std::make_shared<Scratch>();
    scratch->stream = ctx.stream_;
    err = hipHostMalloc((void**)&scratch->meta_host, Scratch::kSlots * 16, hipHostMallocDefault);
    if (err != hipSuccess) {
        return hip_error("pinned metadata ring", err);
    }
    auto meta = DeviceBuffer::allocate(Scratch::kSlots * 16);
    if (meta.is_err()) {
        return meta.unwrap_err();
    }
    scratch->meta_dev = meta.unwrap();
    err = hipHostMalloc((void**)&scratch->stage_host, Scratch::kStageBytes, hipHostMallocDefault);
    if (err != hipSuccess) {
        return hip_error("pinned staging ring", err);
    }
    scratch->counters.device_allocations = 1;
    ctx.scratch_ = scratch;
    return ctx;
}

HostCounters RocmContext::counters() const
{
    return scratch_->counters;
}

Result<Unit> RocmContext::wait_for_stream() const
{
    ++scratch_->counters.stream_waits;
    const hipError_t err = hipStreamSynchronize(stream_);
    if (err != hipSuccess) {
        return hip_error("hipStreamSynchronize", err);
    }
    return Unit{};
}

Result<DeviceBuffer> RocmContext::pooled(size_t bytes) const
{
    Scratch& s = *scratch_;
    size_t real = Scratch::size_class(std::max<size_t>(bytes, 1));
    void* block = nullptr;
    {
        std::lock_guard<std::mutex> hold(s.pool_lock);
        auto found = s.idle.lower_bound(real);
        if (found != s.idle.end() && found->first <= real * 2) {
            block = found->second;
            real = found->first;
            s.idle_bytes -= real;
            s.idle.erase(found);
        }
    }
    if (block == nullptr) {
        const hipError_t err = hipMalloc(&block, real);
        if (err != hipSuccess) {
            return hip_error("hipMalloc", err);
        }
        ++s.counters.device_allocations;
    }
    // the block returns to the pool of the context that made it; if that is gone, it is released
    std::weak_ptr<Scratch> home = scratch_;
    return DeviceBuffer::adopt(std::shared_ptr<void>(block,
                                                     [home, real](void* p) {
                                                         if (auto pool = home.lock()) {
                                                             pool->give_back(p, real);
                                                         } else {
                                                             (void)hipFree(p);
                                                         }
                                                     }),
                               bytes);
}

Result<DeviceBuffer> RocmContext::upload_words(const uint32_t* words, size_t count) const
{
    Scratch& s = *scratch_;
    const size_t bytes = count * 4;
    auto buffer = pooled(bytes);
    if (buffer.is_err()) {
        return buffer;
    }
    if (bytes > Scratch::kStageBytes) {
        // larger than the ring: an ordinary copy, which waits for the stream's earlier work and for itself
        const hipError_t err = hipMemcpy(buffer.unwrap().data(), words, bytes, hipMemcpyHostToDevice);
        if (err != hipSuccess) {
            return hip_error("upload", err);
        }
        return buffer;
    }
    const size_t aligned = (bytes + 63) / 64 * 64;
    if (s.stage_next + aligned > Scratch::kStageBytes) {
        // the ring wrapped: copies still in flight may read its start
        auto waited = wait_for_stream();
        if (waited.is_err()) {
            return waited.unwrap_err();
        }
        s.stage_next = 0;
    }
    uint8_t* host = s.stage_host + s.stage_next;
    memcpy(host, words, bytes);
    const hipError_t err = hipMemcpyAsync(buffer.unwrap().data(), host, bytes, hipMemcpyHostToDevice, stream_);
    if (err != hipSuccess) {
        return hip_error("staged upload", err);
    }
    s.stage_next += aligned;
    ++s.counters.staged_uploads;
    return buffer;
}

Result<const uint32_t*> RocmContext::identity_table(size_t pages) const
{
    Scratch& s = *scratch_;
    if (pages > s.identity_pages) {
        const size_t grown = std::max<size_t>(std::max(pages, s.identity_pages * 2), 1024);
        std::vector<uint32_t> ids(grown);
        std::iota(ids.begin(), ids.end(), 0u);
        auto table = pooled(grown * 4);
        if (table.is_err()) {
            return table.unwrap_err();
        }
        // an ordinary copy: it waits for the stream, so launches that still read the old table are done before it goes
        const hipError_t err = hipMemcpy(table.unwrap().data(), ids.data(), grown * 4, hipMemcpyHostToDevice);
        if (err != hipSuccess) {
            return hip_error("identity table upload", err);
        }
        s.identity = table.unwrap();
        s.identity_pages = grown;
    }
    return (const uint32_t*)s.identity.data();
}

Result<std::pair<const float*, const float*>> RocmContext::resident_rope_tables(const std::vector<float>& cos, const std::vector<float>& sin,
                                                                                size_t required) const
{
    Scratch& s = *scratch_;
    if (cos.size() != sin.size()) {
        return compute_error("ROCm RoPE cos=" + std::to_string(cos.size()) + " sin=" + std::to_string(sin.size()) + " differ");
    }
    required = std::max<size_t>(required, 1);
    if (required > cos.size()) {
        return compute_error("ROCm RoPE needs " + std::to_string(required) + " elements, the tables hold " + std::to_string(cos.size()));
    }
    Scratch::RopeTables* entry = nullptr;
    for (auto& held : s.rope) {
        if (held.cos_host == cos.data() && held.sin_host == sin.data() && held.host_elements == cos.size()) {
            entry = &held;
            break;
        }
    }
    if (entry != nullptr && entry->elements >= required && entry->first == cos[0] && entry->last == cos[entry->elements - 1]) {
        return std::make_pair((const float*)entry->cos.data(), (const float*)entry->sin.data());
    }
    // commit a prefix: at least what is needed, at least twice what was there and 64 KiB, a power of two, never past the table
    size_t elements = std::max(std::max<size_t>(required, 16384), entry != nullptr ? entry->elements * 2 : 0);
    size_t pow2 = 1;
    while (pow2 < elements) {
        pow2 *= 2;
    }
    elements = std::max(std::min(pow2, cos.size()), required);
    auto cos_dev = pooled(elements * 4);
    auto sin_dev = pooled(elements * 4);
    if (cos_dev.is_err() || sin_dev.is_err()) {
        return cos_dev.is_err() ? cos_dev.unwrap_err() : sin_dev.unwrap_err();
    }
    hipError_t err = hipMemcpy(cos_dev.unwrap().data(), cos.data(), elements * 4, hipMemcpyHostToDevice);
    if (err == hipSuccess) {
        err = hipMemcpy(sin_dev.unwrap().data(), sin.data(), elements * 4, hipMemcpyHostToDevice);
    }
    if (err != hipSuccess) {
        return hip_error("rotary table upload", err);
    }
    ++s.counters.rope_table_uploads;
    if (entry == nullptr) {
        if (s.rope.size() == 16) {
            s.rope.erase(s.rope.begin()); // a model has a handful of tables; the oldest goes first
        }
        s.rope.emplace_back();
        entry = &s.rope.back();
    }
    *entry = Scratch::RopeTables{cos.data(), sin.data(), cos.size(), elements, cos[0], cos[elements - 1], cos_dev.unwrap(), sin_dev.unwrap()};
    return std::make_pair((const float*)entry->cos.data(), (const float*)entry->sin.data());
}

Result<void*> RocmContext::workspace(size_t bytes) const
{
    Scratch& s = *scratch_;
    if (bytes > s.workspace.bytes()) {
        // kernels in flight may still use the old buffer: wait for them before it is released
        auto waited = wait_for_stream();
        if (waited.is_err()) {
            return waited.unwrap_err();
        }
        auto grown = DeviceBuffer::allocate(std::max(bytes, s.workspace.bytes() * 2));
        if (grown.is_err()) {
            return grown.unwrap_err();
        }
        ++s.counters.device_allocations;
        s.workspace = grown.unwrap();
    }
    return s.workspace.data();
}

Result<const uint32_t*> RocmContext::upload_meta(const uint32_t (&values)[4]) const
{
    Scratch& s = *scratch_;
    if (s.next == Scratch::kSlots) {
        // the ring wrapped: the oldest records may still be read by launches in flight
        auto waited = wait_for_stream();
        if (waited.is_err()) {
            return waited.unwrap_err();
        }
        s.next = 0;
    }
    uint32_t* host = s.meta_host + 4 * s.next;
    uint32_t* dev = (uint32_t*)s.meta_dev.data() + 4 * s.next;
    memcpy(host, values, 16);
    const hipError_t err = hipMemcpyAsync(dev, host, 16, hipMemcpyHostToDevice, stream_);
    if (err != hipSuccess) {
        return hip_error("metadata upload", err);
    }
    ++s.next;
    return (const uint32_t*)dev;
}

Result<Unit> RocmContext::synchronize() const
{
    const hipError_t err = hipStreamSynchronize(stream_);
    if (err != hipSuccess) {
        return hip_error("hipStreamSynchronize", err);
    }
    return Unit{};
}

Result<RocmTensor> RocmContext::tensor_from_f32(const std::vector<float>& host, size_t rows, size_t cols, DType dtype) const
{
    if (host.size() != rows * cols) {
        return compute_error("tensor_from_f32: data length does not match rows x cols");
    }
    auto buf = DeviceBuffer::allocate(rows * cols * dtype_bytes(dtype));
    if (buf.is_err()) {
        return buf.unwrap_err();
    }
    RocmTensor t;
    t.device = buf.unwrap();
    t.rows = rows;
    t.cols = cols;
    t.dtype = dtype;
    hipError_t err;
    if (dtype == DType::F32) {
        err = hipMemcpy(t.device.data(), host.data(), host.size() * 4, hipMemcpyHostToDevice);
    } else {
        std::vector<uint16_t> half(host.size());
        for (size_t i = 0; i < host.size(); ++i) {
            half[i] = dtype == DType::BF16 ? f32_to_bf16_bits(host[i]) : f32_to_f16_bits(host[i]);
        }
        err = hipMemcpy(t.device.data(), half.data(), half.size() * 2, hipMemcpyHostToDevice);
    }
    if (err != hipSuccess) {
        return hip_error("tensor upload", err);
    }
    return t;
}

Result<std::vector<float>> RocmContext::tensor_to_f32(const RocmTensor& tensor) const
{
    hipError_t err = hipStreamSynchronize(stream_);
    if (err != hipSuccess) {
        return hip_error("hipStreamSynchronize", err);
    }
    const size_t n = tensor.rows * tensor.cols;
    std::vector<float> out(n);
    if (tensor.dtype == DType::F32) {
        err = hipMemcpy(out.data(), tensor.device.data(), n * 4, hipMemcpyDeviceToHost);
    } else {
        std::vector<uint16_t> half(n);
        err = hipMemcpy(half.data(), tensor.device.data(), n * 2, hipMemcpyDeviceToHost);
        for (size_t i = 0; i < n; ++i) {
            out[i] = tensor.dtype == DType::BF16 ? bf16_bits_to_f32(half[i]) : f16_bits_to_f32(half[i]);
        }
    }
    if (err != hipSuccess) {
        return hip_error("tensor download", err);
    }
    return out;
}

Result<RocmWeight> RocmContext::prepare_mla_kv_b(const std::vector<float>& weight, size_t rows, size_t cols) const
{
    auto t = tensor_from_f32(weight, rows, cols, DType::BF16);
    if (t.is_err()) {
        return t.unwrap_err();
    }
    RocmWeight w;
    w.device = t.unwrap().device;
    w.rows = rows;
    w.cols = cols;
    return w;
}

Result<RocmWeight> RocmContext::prepare_mla_kv_b_quantized(const std::vector<float>& weight, size_t rows, size_t cols, unsigned bits,
                                                           size_t group_size) const
{
    if ((bits != 8 && bits != 4) || group_size == 0 || cols % group_size != 0 || weight.size() != rows * cols || cols % (32 / bits) != 0) {
        return compute_error("prepare_mla_kv_b_quantized: bits=" + std::to_string(bits) + " group=" + std::to_string(group_size) + " for [" +
                             std::to_string(rows) + "," + std::to_string(cols) + "]");
    }
    const int top = bits == 8 ? 127 : 7, offset = bits == 8 ? 128 : 8;
    const size_t per_word = 32 / bits, words_per_row = cols / per_word, groups = cols / group_size;
    std::vector<uint32_t> words(rows * words_per_row, 0u);
    std::vector<uint16_t> scale_bits(rows * groups);
    for (size_t r = 0; r < rows; ++r) {
        for (size_t g = 0; g < groups; ++g) {
            float largest = 0.0f;
            for (size_t c = g * group_size; c < (g + 1) * group_size; ++c) {
                largest = std::max(largest, fabsf(weight[r * cols + c]));
            }
            const uint16_t stored = f32_to_bf16_bits(largest > 0.0f ? largest / (float)top : 1.0f);
            const float scale = bf16_bits_to_f32(stored);
            scale_bits[r * groups + g] = stored;
            for (size_t c = g * group_size; c < (g + 1) * group_size; ++c) {
                const int code = std::max(-top - 1, std::min(top, (int)lrintf(weight[r * cols + c] / scale))) + offset;
                words[r * words_per_row + c / per_word] |= (uint32_t)code << ((c % per_word) * bits);
            }
        }
    }
    RocmWeight w;
    w.rows = rows;
    w.cols = cols;
    w.bits = bits;
    w.group_size = group_size;
    w.scale_dtype = DType::BF16;
    auto codes = DeviceBuffer::allocate(words.size() * 4);
    auto scales = DeviceBuffer::allocate(scale_bits.size() * 2);
    if (codes.is_err() || scales.is_err()) {
        return codes.is_err() ? codes.unwrap_err() : scales.unwrap_err();
    }
    hipError_t err = hipMemcpy(codes.unwrap().data(), words.data(), words.size() * 4, hipMemcpyHostToDevice);
    if (err == hipSuccess) {
        err = hipMemcpy(scales.unwrap().data(), scale_bits.data(), scale_bits.size() * 2, hipMemcpyHostToDevice);
    }
    if (err != hipSuccess) {
        return hip_error("weight upload", err);
    }
    w.device = codes.unwrap();
    w.scales = scales.unwrap();
    return w;
}

Result<std::vector<float>> RocmContext::dequantized_kv_b(const RocmWeight& weight) const
{
    if (weight.bits != 8 && weight.bits != 4) {
        return compute_error("dequantized_kv_b: the weight holds no codes");
    }
    const size_t per_word = 32 / weight.bits, words_per_row = weight.cols / per_word, groups = weight.cols / weight.group_size;
    std::vector<uint32_t> words(weight.rows * words_per_row);
    std::vector<uint16_t> scale_bits(weight.rows * groups);
    hipError_t err = hipMemcpy(words.data(), weight.device.data(), words.size() * 4, hipMemcpyDeviceToHost);
    if (err == hipSuccess) {
        err = hipMemcpy(scale_bits.data(), weight.scales.data(), scale_bits.size() * 2, hipMemcpyDeviceToHost);
    }
    if (err != hipSuccess) {
        return hip_error("weight download", err);
    }
    const int offset = weight.bits == 8 ? 128 : 8;
    std::vector<float> out(weight.rows * weight.cols);
    for (size_t r = 0; r < weight.rows; ++r) {
        for (size_t c = 0; c < weight.cols; ++c) {
            const uint32_t code = (words[r * words_per_row + c / per_word] >> ((c % per_word) * weight.bits)) & ((1u << weight.bits) - 1u);
            out[r * weight.cols + c] = (float)((int)code - offset) * bf16_bits_to_f32(scale_bits[r * groups + c / weight.group_size]);
        }
    }
    return out;
}

namespace {

// HybridGqaCacheLayout::write_plan (src/kv_cache/mod.rs:440-455) for a layer that keeps `capacity` rows
struct RingPlan {
    size_t source_start, token_count;
};

RingPlan ring_write_plan(size_t capacity, size_t position, size_t count)
{
    const size_t end = position + count;
    const size_t write_start = std::max(position, end > capacity ? end - capacity : 0);
    return RingPlan{write_start - position, end - write_start};
}

BackendError unsupported_layer(size_t layer)
{
    BackendError e;
    e.kind = BackendError::Kind::UnsupportedLayer;
    e.layer = layer;
    return e;
}

} // namespace

Result<Unit> RocmContext::append_gqa_rows(RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& key, const RocmTensor& value) const
{
    RocmKvCache::Layer& planes = cache.layers_[layer];
    const size_t ring = planes.ring_capacity;
    const size_t total = position + key.rows;
    auto reserved = cache.reserve_rows(layer, ring != 0 ? std::min(total, ring) : total, stream_);
    if (reserved.is_err()) {
        return reserved.unwrap_err();
    }
    // a ring keeps the chunk's last `capacity` rows only
    const RingPlan plan = ring != 0 ? ring_write_plan(ring, position, key.rows) : RingPlan{0, key.rows};
    const RocmTensor* sources[2] = {&key, &value};
    void* codes[2] = {planes.a_codes.data(), planes.b_codes.data()};
    void* scales[2] = {planes.a_scales.data(), planes.b_scales.data()};
    for (int i = 0; i < 2; ++i) {
        zllm_q8_append_args a;
        memset(&a, 0, sizeof(a));
        a.src = (const char*)sources[i]->device.data() + plan.source_start * sources[i]->cols * dtype_bytes(sources[i]->dtype);
        a.codes = (int8_t*)codes[i];
        a.scales = scales[i];
        a.table = (const uint32_t*)cache.table_.data();
        a.position = (uint32_t)(position + plan.source_start);
        a.rows = (uint32_t)plan.token_count;
        a.cols = (uint32_t)cache.cols_;
        a.block_tokens = (uint32_t)cache.block_tokens_;
        a.ring_capacity = (uint32_t)ring;
        a.src_dtype = abi_dtype(sources[i]->dtype);
        a.rule = ZLLM_QUANT_METAL_GQA;
        const int rc = zllm_attn_q8g64_append(&a, stream_);
        if (rc != 0) {
            return abi_error("zllm_attn_q8g64_append", rc);
        }
    }
    return Unit{};
}

// Attention of `query.rows` rows at `position` over the layer's rows [.., position + query.rows), which are in the cache.
Result<RocmTensor> RocmContext::gqa_attend(const RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& query, const GqaSpec& spec,
                                           const uint32_t* visible_ends_dev) const
{
    const RocmKvCache::Layer& planes = cache.layers_[layer];
    const size_t query_cols = spec.num_heads * spec.head_dim;
    const size_t total = position + query.rows;
    auto out_buf = pooled(query.rows * query_cols * 4);
    if (out_buf.is_err()) {
        return out_buf.unwrap_err();
    }
    RocmTensor out;
    out.device = out_buf.unwrap();
    out.rows = query.rows;
    out.cols = query_cols;
    out.dtype = DType::F32;
    const size_t table_stride = cache.table_host_.size();

    if (query.rows == 1 && visible_ends_dev == nullptr) {
        const auto range = spec.window.key_range(position, total);
        const uint32_t host_meta[4] = {(uint32_t)total, (uint32_t)range.first, 0u, 0u};
        auto meta = upload_meta(host_meta);
        if (meta.is_err()) {
            return meta.unwrap_err();
        }
        zllm_gqa_decode_args a;
        memset(&a, 0, sizeof(a));
        a.q = query.device.data();
        a.k_plane = planes.a_codes.data();
        a.k_scales = planes.a_scales.data();
        a.v_plane = planes.b_codes.data();
        a.v_scales = planes.b_scales.data();
        a.tables = (const uint32_t*)cache.table_.data();
        a.kv_lens = meta.unwrap();
        a.first_visible = spec.window.sliding ? meta.unwrap() + 1 : nullptr;
        a.out = (float*)out.device.data();
        a.batch = 1;
        a.num_heads = (uint32_t)spec.num_heads;
        a.num_kv_heads = (uint32_t)spec.num_kv_heads;
        a.head_dim = (uint32_t)spec.head_dim;
        a.table_stride = (uint32_t)table_stride;
        a.max_kv_len = (uint32_t)total;
        a.block_tokens = (uint32_t)cache.block_tokens_;
        a.ring_capacity = (uint32_t)planes.ring_capacity;
        a.score_scale = spec.score_scale;
        a.kv_format = ZLLM_KV_Q8G64;
        a.scale_dtype = ZLLM_SCALE_F16;
        a.q_dtype = abi_dtype(query.dtype);
        const uint64_t need = zllm_attn_gqa_decode_workspace_bytes(&a);
        if (need == 0) {
            return abi_error("zllm_attn_gqa_decode_workspace_bytes", -1);
        }
        auto ws = workspace(need);
        if (ws.is_err()) {
            return ws.unwrap_err();
        }
        a.workspace = ws.unwrap();
        a.workspace_bytes = need;
        const int rc = zllm_attn_gqa_decode(&a, stream_);
        if (rc != 0) {
            return abi_error("zllm_attn_gqa_decode", rc);
        }
        return out;
    }
    if (planes.ring_capacity != 0 && total > planes.ring_capacity) {
        return compute_error("sliding-window GQA cannot attend a multi-token chunk over a ring that has wrapped");
    }
    zllm_gqa_prefill_args a;
    memset(&a, 0, sizeof(a));
    a.q = query.device.data();
    a.k_plane = planes.a_codes.data();
    a.k_scales = planes.a_scales.data();
    a.v_plane = planes.b_codes.data();
    a.v_scales = planes.b_scales.data();
    a.table = (const uint32_t*)cache.table_.data();
    a.table_stride = (uint32_t)table_stride;
    a.out = out.device.data();
    a.rows = (uint32_t)query.rows;
    a.position = (uint32_t)position;
    a.window = spec.window.sliding ? (uint32_t)spec.window.size : 0u;
    a.num_heads = (uint32_t)spec.num_heads;
    a.num_kv_heads = (uint32_t)spec.num_kv_heads;
    a.head_dim = (uint32_t)spec.head_dim;
    a.block_tokens = (uint32_t)cache.block_tokens_;
    a.score_scale = spec.score_scale;
    a.kv_format = ZLLM_KV_Q8G64;
    a.scale_dtype = ZLLM_SCALE_F16;
    a.q_dtype = abi_dtype(query.dtype);
    a.out_dtype = ZLLM_DTYPE_F32;
    a.visible_ends = visible_ends_dev;
    const uint64_t need = zllm_attn_gqa_prefill_workspace_bytes(&a);
    if (need != 0) {
        auto ws = workspace(need);
        if (ws.is_err()) {
            return ws.unwrap_err();
        }
        a.workspace = ws.unwrap();
        a.workspace_bytes = need;
    }
    const int rc = zllm_attn_gqa_prefill_chunk(&a, stream_);
    if (rc != 0) {
        return abi_error("zllm_attn_gqa_prefill_chunk", rc);
    }
    return out;
}

Result<RocmTensor> RocmContext::gqa_cached_impl(RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& query, const RocmTensor& key,
                                                const RocmTensor& value, const GqaSpec& spec, const std::vector<uint32_t>* visible_ends,
                                                bool retain_full_cache) const
{
    if (spec.num_heads == 0 || spec.num_kv_heads == 0 || spec.head_dim == 0 || spec.num_heads % spec.num_kv_heads != 0) {
        return compute_error("Rocm GQA spec invalid");
    }
    const size_t query_cols = spec.num_heads * spec.head_dim;
    const size_t kv_cols = spec.num_kv_heads * spec.head_dim;
    if (query.rows != key.rows || query.rows != value.rows || query.cols != query_cols || key.cols != kv_cols || value.cols != kv_cols) {
        return compute_error("Rocm GQA cached prefill shape mismatch: Q=[" + std::to_string(query.rows) + "," + std::to_string(query.cols) + "] K=[" +
                             std::to_string(key.rows) + "," + std::to_string(key.cols) + "] V=[" + std::to_string(value.rows) + "," +
                             std::to_string(value.cols) + "]");
    }
    if (cache.mla_ || layer >= cache.layers_.size() || cache.cols_ != kv_cols) {
        return unsupported_layer(layer);
    }
    if (query.rows == 0) {
        return compute_error("Rocm GQA cached prefill: empty chunk");
    }
    if (visible_ends != nullptr && visible_ends->size() != query.rows) {
        return compute_error("GQA visible_ends=" + std::to_string(visible_ends->size()) + ", expected " + std::to_string(query.rows));
    }
    // position must be the current cache length (src/backend/rocm/attention.rs:2226-2229)
    if (cache.lens_[layer] != position) {
        return compute_error("Rocm GQA L" + std::to_string(layer) + " device cache incomplete: rows=" + std::to_string(cache.lens_[layer]) + "/" +
                             std::to_string(position));
    }
    const size_t total = position + query.rows;
    if (total > cache.max_tokens_ || total > UINT32_MAX) {
        return compute_error("Rocm GQA cache position overflow");
    }
    // a sliding-window layer that need not keep everything keeps a ring of cache_capacity rows
    const size_t ring = spec.window.sliding && !retain_full_cache ? spec.window.cache_capacity(cache.max_tokens_) : 0;
    RocmKvCache::Layer& planes = cache.layers_[layer];
    if (position == 0) {
        planes.ring_capacity = ring;
    } else if (planes.ring_capacity != ring) {
        return compute_error("Rocm GQA L" + std::to_string(layer) + ": the layer was filled with another retention (ring of " +
                             std::to_string(planes.ring_capacity) + " rows)");
    }
    // the ends travel through the pinned ring into a pooled block, which goes back to the pool when this call
    // returns and is next written by work queued behind the launches that read it
    const uint32_t* ends_dev = nullptr;
    DeviceBuffer ends_buf;
    if (visible_ends != nullptr) {
        auto buf = upload_words(visible_ends->data(), visible_ends->size());
        if (buf.is_err()) {
            return buf.unwrap_err();
        }
        ends_buf = buf.unwrap();
        ends_dev = (const uint32_t*)ends_buf.data();
    }
    if (ring != 0 && query.rows > 1) {
        // the reference's CPU backend (src/backend/cpu/attention.rs:401-409): a multi-token chunk on a draining sliding layer
        // attends to itself at position 0 and is rejected elsewhere
        if (position != 0) {
            return compute_error("sliding-window GQA does not take a multi-token prefill at a non-zero position");
        }
        if (total > ring) {
            // the ring cannot hold the whole chunk: attend over a cache of the chunk's own, then keep the tail
            auto own = RocmKvCache::new_gqa(1, spec.num_kv_heads, spec.head_dim, cache.block_tokens_, total);
            if (own.is_err()) {
                return own.unwrap_err();
            }
            RocmKvCache chunk_cache = own.unwrap();
            auto appended = append_gqa_rows(chunk_cache, 0, 0, key, value);
            if (appended.is_err()) {
                return appended.unwrap_err();
            }
            auto out = gqa_attend(chunk_cache, 0, 0, query, spec, ends_dev);
            if (out.is_err()) {
                return out;
            }
            auto kept = append_gqa_rows(cache, layer, 0, key, value);
            if (kept.is_err()) {
                return kept.unwrap_err();
            }
            auto waited = wait_for_stream(); // the chunk's own cache dies with this scope
            if (waited.is_err()) {
                return waited.unwrap_err();
            }
            cache.lens_[layer] = total;
            return out;
        }
    }
    auto appended = append_gqa_rows(cache, layer, position, key, value);
    if (appended.is_err()) {
        return appended.unwrap_err();
    }
    auto out = gqa_attend(cache, layer, position, query, spec, ends_dev);
    if (out.is_err()) {
        return out; // the cache length is left alone: the rows written past it are overwritten by the next append
    }
    cache.lens_[layer] = total;
    return out;
}

Result<RocmTensor> RocmContext::gqa_prefill_attention_cached(RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& query,
                                                             const RocmTensor& key, const RocmTensor& value, const GqaSpec& spec,
                                                             bool retain_full_cache) const
{
    return gqa_cached_impl(cache, layer, position, query, key, value, spec, nullptr, retain_full_cache);
}

Result<RocmTensor> RocmContext::gqa_prefill_attention_cached_visible(RocmKvCache& cache, size_t layer, size_t position, const RocmTensor& query,
                                                                     const RocmTensor& key, const RocmTensor& value, const GqaSpec& spec,
                                                                     const std::vector<uint32_t>& visible_ends, bool retain_full_cache) const
{
    return gqa_cached_impl(cache, layer, position, query, key, value, spec, &visible_ends, retain_full_cache);
}

Result<RocmTensor> RocmContext::gqa_prefill_attention_cached_from(const RocmKvCache& cache, size_t source_layer, size_t position,
                                                                  const RocmTensor& query, const GqaSpec& spec) const
{
    if (spec.num_heads == 0 || spec.num_kv_heads == 0 || spec.head_dim == 0 || spec.num_heads % spec.num_kv_heads != 0) {
        return compute_error("Rocm GQA spec invalid");
    }
    if (cache.mla_ || source_layer >= cache.layers_.size()) {
        return unsupported_layer(source_layer);
    }
    const size_t required = position + query.rows;
    // shape rule of the shared-KV path (src/backend/cpu/attention.rs:439-446); a ring or a longer source cannot serve it:
    // the rows after the chunk would be visible to the kernels' causal ranges only by position, which they respect
    if (query.rows == 0 || query.cols != spec.num_heads * spec.head_dim || cache.cols_ != spec.num_kv_heads * spec.head_dim ||
        cache.lens_[source_layer] < required) {
        return compute_error("GQA shared cache L" + std::to_string(source_layer) + " incomplete: Q=[" + std::to_string(query.rows) + "," +
                             std::to_string(query.cols) + "], cache rows=" + std::to_string(cache.lens_[source_layer]) +
                             ", required_rows=" + std::to_string(required));
    }
    return gqa_attend(cache, source_layer, position, query, spec, nullptr);
}

Result<RocmTensor> RocmContext::gqa_prefill_attention_cached_from_visible(const RocmKvCache& cache, size_t source_layer, size_t position,
                                                                           const RocmTensor& query, const GqaSpec& spec,
                                                                           const std::vector<uint32_t>& visible_ends) const
{
    if (spec.num_heads == 0 || spec.num_kv_heads == 0 || spec.head_dim == 0 || spec.num_heads % spec.num_kv_heads != 0) {
        return compute_error("Rocm GQA spec invalid");
    }
    if (cache.mla_ || source_layer >= cache.layers_.size()) {
        return unsupported_layer(source_layer);
    }
    if (visible_ends.size() != query.rows) {
        return compute_error("GQA visible_ends=" + std::to_string(visible_ends.size()) + ", expected " + std::to_string(query.rows));
    }
    const size_t required = position + query.rows;
    if (query.rows == 0 || query.cols != spec.num_heads * spec.head_dim || cache.cols_ != spec.num_kv_heads * spec.head_dim ||
        cache.lens_[source_layer] < required) {
        return compute_error("GQA shared cache L" + std::to_string(source_layer) + " incomplete: Q=[" + std::to_string(query.rows) + "," +
                             std::to_string(query.cols) + "], cache rows=" + std::to_string(cache.lens_[source_layer]) +
                             ", required_rows=" + std::to_string(required));
    }
    auto ends = upload_words(visible_ends.data(), visible_ends.size());
    if (ends.is_err()) {
        return ends.unwrap_err();
    }
    return gqa_attend(cache, source_layer, position, query, spec, (const uint32_t*)ends.unwrap().data());
}

// ---------------------------------------------------------------------------------------- dense K/V
std::optional<std::string> GqaGeometry::validate() const
{
    if (num_heads == 0 || num_kv_heads == 0 || head_dim == 0 || num_heads % num_kv_heads != 0) {
        return "GQA geometry invalid: query_heads=" + std::to_string(num_heads) + " kv_heads=" + std::to_string(num_kv_heads) +
               " head_dim=" + std::to_string(head_dim);
    }
    return std::nullopt;
}

std::optional<std::string> BlockAttentionSpec::validate(size_t query_rows, size_t kv_rows) const
{
    if (auto bad = geometry.validate()) {
        return bad;
    }
    if (!isfinite(score_scale) || score_scale <= 0.0f) {
        return "block attention score_scale=" + std::to_string(score_scale) + " invalid";
    }
    if (visible.size() != query_rows) {
        return "block attention visible=" + std::to_string(visible.size()) + ", expected query_rows=" + std::to_string(query_rows);
    }
    for (size_t r = 0; r < visible.size(); ++r) {
        if (visible[r].first >= visible[r].second || visible[r].second > kv_rows) {
            return "block attention query=" + std::to_string(r) + " visible range " + std::to_string(visible[r].first) + ".." +
                   std::to_string(visible[r].second) + " outside KV rows=" + std::to_string(kv_rows);
        }
    }
    return std::nullopt;
}

BlockAttentionSpec BlockAttentionSpec::full(GqaGeometry geometry, size_t query_rows, size_t kv_rows, float score_scale)
{
    BlockAttentionSpec spec;
    spec.geometry = geometry;
    spec.score_scale = score_scale;
    spec.visible.assign(query_rows, std::make_pair((size_t)0, kv_rows));
    return spec;
}

Result<BlockAttentionSpec> BlockAttentionSpec::varlen(GqaGeometry geometry, size_t query_rows, size_t kv_rows,
                                                      const std::vector<size_t>& query_offsets, const std::vector<size_t>& kv_offsets,
                                                      float score_scale)
{
    auto rising = [](const std::vector<size_t>& offsets) {
        for (size_t i = 1; i < offsets.size(); ++i) {
            if (offsets[i - 1] >= offsets[i]) {
                return false;
            }
        }
        return true;
    };
    if (query_offsets.size() < 2 || query_offsets.size() != kv_offsets.size() || query_offsets.front() != 0 || kv_offsets.front() != 0 ||
        query_offsets.back() != query_rows || kv_offsets.back() != kv_rows || !rising(query_offsets) || !rising(kv_offsets)) {
        return compute_error("varlen attention offsets invalid: Q=" + std::to_string(query_rows) + " KV=" + std::to_string(kv_rows));
    }
    BlockAttentionSpec spec;
    spec.geometry = geometry;
    spec.score_scale = score_scale;
    spec.visible.reserve(query_rows);
    for (size_t i = 1; i < query_offsets.size(); ++i) {
        spec.visible.insert(spec.visible.end(), query_offsets[i] - query_offsets[i - 1], std::make_pair(kv_offsets[i - 1], kv_offsets[i]));
    }
    if (auto bad = spec.validate(query_rows, kv_rows)) {
        return compute_error(*bad);
    }
    return spec;
}

struct RocmContext::DensePlanes {
    DeviceBuffer key, value; // f16 [pages * kBlock, cols]
    const uint32_t* table = nullptr;
    size_t pages = 0, cols = 0;
    static constexpr size_t kBlock = 64;
};

Result<RocmContext::DensePlanes> RocmContext::dense_f16_planes(const std::vector<const RocmTensor*>& keys, const std::vector<const RocmTensor*>& values,
                                                               size_t cols, size_t cache_rows) const
{
    DensePlanes planes;
    planes.cols = cols;
    planes.pages = (cache_rows + DensePlanes::kBlock - 1) / DensePlanes::kBlock;
    if (planes.pages == 0 || planes.pages * DensePlanes::kBlock > UINT32_MAX) {
        return compute_error("ROCm dense attention: " + std::to_string(cache_rows) + " cache rows");
    }
    auto table = identity_table(planes.pages);
    if (table.is_err()) {
        return table.unwrap_err();
    }
    planes.table = table.unwrap();
    auto key = pooled(planes.pages * DensePlanes::kBlock * cols * 2);
    auto value = pooled(planes.pages * DensePlanes::kBlock * cols * 2);
    if (key.is_err() || value.is_err()) {
        return key.is_err() ? key.unwrap_err() : value.unwrap_err();
    }
    planes.key = key.unwrap();
    planes.value = value.unwrap();
    const std::vector<const RocmTensor*>* sources[2] = {&keys, &values};
    void* targets[2] = {planes.key.data(), planes.value.data()};
    for (int i = 0; i < 2; ++i) {
        size_t at = 0;
        for (const RocmTensor* part : *sources[i]) {
            if (part->rows == 0) {
                continue;
            }
            zllm_half_append_args a;
            memset(&a, 0, sizeof(a));
            a.src = part->device.data();
            a.cache = targets[i];
            a.table = planes.table;
            a.position = (uint32_t)at;
            a.rows = (uint32_t)part->rows;
            a.cols = (uint32_t)cols;
            a.block_tokens = (uint32_t)DensePlanes::kBlock;
            a.src_dtype = abi_dtype(part->dtype);
            a.dst_dtype = ZLLM_DTYPE_F16;
            const int rc = zllm_attn_half_append(&a, stream_);
            if (rc != 0) {
                return abi_error("zllm_attn_half_append", rc);
            }
            at += part->rows;
        }
    }
    return planes;
}

// `query.rows` rows at `position` over the planes' rows [0, position + query.rows): causal (with `window`, with visible ends)
// when `starts_dev` is null, the exact ranges [starts, ends) otherwise.
Result<RocmTensor> RocmContext::attend_dense(const RocmTensor& query, const DensePlanes& planes, size_t position, const GqaGeometry& geometry,
                                             float score_scale, size_t window, const uint32_t* starts_dev, const uint32_t* ends_dev) const
{
    const size_t query_cols = geometry.num_heads * geometry.head_dim;
    auto out_buf = pooled(query.rows * query_cols * 4);
    if (out_buf.is_err()) {
        return out_buf.unwrap_err();
    }
    zllm_gqa_prefill_args a;
    memset(&a, 0, sizeof(a));
    a.q = query.device.data();
    a.k_plane = planes.key.data();
    a.v_plane = planes.value.data();
    a.table = planes.table;
    a.table_stride = (uint32_t)planes.pages;
    a.out = out_buf.unwrap().data();
    a.rows = (uint32_t)query.rows;
    a.position = (uint32_t)position;
    a.window = (uint32_t)window;
    a.num_heads = (uint32_t)geometry.num_heads;
    a.num_kv_heads = (uint32_t)geometry.num_kv_heads;
    a.head_dim = (uint32_t)geometry.head_dim;
    a.block_tokens = (uint32_t)DensePlanes::kBlock;
    a.score_scale = score_scale;
    a.kv_format = ZLLM_KV_F16;
    a.scale_dtype = ZLLM_SCALE_F16;
    a.q_dtype = abi_dtype(query.dtype);
    a.out_dtype = ZLLM_DTYPE_F32;
    a.visible_starts = starts_dev;
    a.visible_ends = ends_dev;
    const uint64_t need = zllm_attn_gqa_prefill_workspace_bytes(&a);
    if (need != 0) {
        auto ws = workspace(need);
        if (ws.is_err()) {
            return ws.unwrap_err();
        }
        a.workspace = ws.unwrap();
        a.workspace_bytes = need;
    }
    const int rc = zllm_attn_gqa_prefill_chunk(&a, stream_);
    if (rc != 0) {
        return abi_error("zllm_attn_gqa_prefill_chunk", rc);
    }
    RocmTensor out;
    out.device = out_buf.unwrap();
    out.rows = query.rows;
    out.cols = query_cols;
    out.dtype = DType::F32;
    return out;
}

Result<RocmTensor> RocmContext::gqa_prefill_attention(const RocmTensor& query, const RocmTensor& key, const RocmTensor& value, const GqaSpec& spec) const
{
    const GqaGeometry geometry{spec.num_heads, spec.num_kv_heads, spec.head_dim};
    if (auto bad = geometry.validate()) {
        return compute_error(*bad);
    }
    const size_t query_cols = spec.num_heads * spec.head_dim, kv_cols = spec.num_kv_heads * spec.head_dim;
    if (query.rows == 0 || query.rows != key.rows || query.rows != value.rows || query.cols != query_cols || key.cols != kv_cols ||
        value.cols != kv_cols) {
        return compute_error("Rocm GQA prefill shape mismatch: Q=[" + std::to_string(query.rows) + "," + std::to_string(query.cols) + "] K=[" +
                             std::to_string(key.rows) + "," + std::to_string(key.cols) + "] V=[" + std::to_string(value.rows) + "," +
                             std::to_string(value.cols) + "]");
    }
    auto planes = dense_f16_planes({&key}, {&value}, kv_cols, key.rows);
    if (planes.is_err()) {
        return planes.unwrap_err();
    }
    return attend_dense(query, planes.unwrap(), 0, geometry, spec.score_scale, spec.window.sliding ? spec.window.size : 0, nullptr, nullptr);
}

Result<RocmTensor> RocmContext::gqa_prefill_attention_visible(const RocmTensor& query, const RocmTensor& key, const RocmTensor& value,
                                                              const GqaSpec& spec, const std::vector<uint32_t>& visible_ends) const
{
    const GqaGeometry geometry{spec.num_heads, spec.num_kv_heads, spec.head_dim};
    if (auto bad = geometry.validate()) {
        return compute_error(*bad);
    }
    const size_t query_cols = spec.num_heads * spec.head_dim, kv_cols = spec.num_kv_heads * spec.head_dim;
    if (query.rows == 0 || query.rows != key.rows || query.rows != value.rows || query.cols != query_cols || key.cols != kv_cols ||
        value.cols != kv_cols || visible_ends.size() != query.rows) {
        return compute_error("Rocm GQA visible prefill shape mismatch: Q=[" + std::to_string(query.rows) + "," + std::to_string(query.cols) + "] K=[" +
                             std::to_string(key.rows) + "," + std::to_string(key.cols) + "] V=[" + std::to_string(value.rows) + "," +
                             std::to_string(value.cols) + "] visible=" + std::to_string(visible_ends.size()));
    }
    auto planes = dense_f16_planes({&key}, {&value}, kv_cols, key.rows);
    if (planes.is_err()) {
        return planes.unwrap_err();
    }
    auto ends = upload_words(visible_ends.data(), visible_ends.size());
    if (ends.is_err()) {
        return ends.unwrap_err();
    }
    return attend_dense(query, planes.unwrap(), 0, geometry, spec.score_scale, spec.window.sliding ? spec.window.size : 0, nullptr,
                        (const uint32_t*)ends.unwrap().data());
}

Result<RocmTensor> RocmContext::block_attention_segments(const RocmTensor& query, const std::vector<const RocmTensor*>& keys,
                                                         const std::vector<const RocmTensor*>& values, const BlockAttentionSpec& spec) const
{
    if (keys.size() != values.size() || keys.empty()) {
        return compute_error("block attention segments K/V count=" + std::to_string(keys.size()) + "/" + std::to_string(values.size()));
    }
    const size_t query_cols = spec.geometry.num_heads * spec.geometry.head_dim, kv_cols = spec.geometry.num_kv_heads * spec.geometry.head_dim;
    size_t kv_rows = 0;
    for (size_t i = 0; i < keys.size(); ++i) {
        if (keys[i] == nullptr || values[i] == nullptr || keys[i]->cols != kv_cols || values[i]->cols != kv_cols || keys[i]->rows != values[i]->rows) {
            return compute_error("ROCm block attention shape mismatch in K/V segment " + std::to_string(i));
        }
        kv_rows += keys[i]->rows;
    }
    if (auto bad = spec.validate(query.rows, kv_rows)) {
        return compute_error(*bad);
    }
    if (query.cols != query_cols) {
        return compute_error("ROCm block attention shape mismatch: Q=[" + std::to_string(query.rows) + "," + std::to_string(query.cols) + "]");
    }
    if (kv_rows > UINT32_MAX || query.rows > UINT32_MAX) {
        return compute_error("ROCm block attention visible range beyond u32");
    }
    // the entry point reads no cache row at or past position + rows: put the query rows at the end of whichever is longer
    const size_t cache_rows = std::max(kv_rows, query.rows);
    auto planes = dense_f16_planes(keys, values, kv_cols, cache_rows);
    if (planes.is_err()) {
        return planes.unwrap_err();
    }
    std::vector<uint32_t> ranges(2 * query.rows);
    for (size_t r = 0; r < query.rows; ++r) {
        ranges[r] = (uint32_t)spec.visible[r].first;
        ranges[query.rows + r] = (uint32_t)spec.visible[r].second;
    }
    auto ranges_dev = upload_words(ranges.data(), ranges.size());
    if (ranges_dev.is_err()) {
        return ranges_dev.unwrap_err();
    }
    const uint32_t* starts = (const uint32_t*)ranges_dev.unwrap().data();
    return attend_dense(query, planes.unwrap(), cache_rows - query.rows, spec.geometry, spec.score_scale, 0, starts, starts + query.rows);
}

Result<RocmTensor> RocmContext::block_attention_prefix_suffix(const RocmTensor& query, const RocmTensor& prefix_key, const RocmTensor& prefix_value,
                                                              const RocmTensor& suffix_key, const RocmTensor& suffix_value,
                                                              const BlockAttentionSpec& spec) const
{
    return block_attention_segments(query, {&prefix_key, &suffix_key}, {&prefix_value, &suffix_value}, spec);
}

Result<RocmTensor> RocmContext::block_attention(const RocmTensor& query, const RocmTensor& key, const RocmTensor& value,
                                                const BlockAttentionSpec& spec) const
{
    return block_attention_segments(query, {&key}, {&value}, spec);
}

Result<Unit> RocmContext::append_mla_impl(RocmKvCache& cache, size_t layer, const RocmTensor& latent, const RocmTensor& rope, size_t rotary_dim,
                                          RotaryLayout layout, size_t position, const float* cos_dev, const float* sin_dev) const
{
    if (!cache.mla_ || layer >= cache.layers_.size()) {
        return unsupported_layer(layer);
    }
    if (latent.rows != rope.rows || latent.cols != cache.cols_ || rope.cols != cache.rope_cols_ || latent.dtype != DType::F32 ||
        rope.dtype != DType::F32) {
        return compute_error("Rocm MLA append shape mismatch: latent=[" + std::to_string(latent.rows) + "," + std::to_string(latent.cols) + "] rope=[" +
                             std::to_string(rope.rows) + "," + std::to_string(rope.cols) + "]");
    }
    const size_t at = cache.lens_[layer];
    if (at + latent.rows > cache.max_tokens_) {
        return compute_error("Rocm MLA cache is full");
    }
    auto reserved = cache.reserve_rows(layer, at + latent.rows, stream_);
    if (reserved.is_err()) {
        return reserved.unwrap_err();
    }
    RocmKvCache::Layer& planes = cache.layers_[layer];
    zllm_mla_append_args a;
    memset(&a, 0, sizeof(a));
    a.latent = (const float*)latent.device.data();
    a.k_rope = (const float*)rope.device.data();
    a.cosine = cos_dev;
    a.sine = sin_dev;
    a.latent_codes = (int8_t*)planes.a_codes.data();
    a.latent_scales = (uint16_t*)planes.a_scales.data();
    a.rope_cache = (uint16_t*)planes.b_codes.data();
    a.table = (const uint32_t*)cache.table_.data();
    a.position = (uint32_t)at;
    a.rope_position = (uint32_t)position;
    a.rows = (uint32_t)latent.rows;
    a.latent_cols = (uint32_t)cache.cols_;
    a.rope_cols = (uint32_t)cache.rope_cols_;
    a.rotary_dim = (uint32_t)rotary_dim;
    a.rotary_layout = layout == RotaryLayout::SplitHalf ? ZLLM_ROTARY_SPLIT_HALF : ZLLM_ROTARY_INTERLEAVED;
    a.block_tokens = (uint32_t)cache.block_tokens_;
    const int rc = zllm_attn_mla_append(&a, stream_);
    if (rc != 0) {
        return abi_error("zllm_attn_mla_append", rc);
    }
    cache.lens_[layer] = at + latent.rows;
    return Unit{};
}

Result<Unit> RocmContext::append_mla(RocmKvCache& cache, size_t layer, const RocmTensor& latent, const RocmTensor& rope) const
{
    return append_mla_impl(cache, layer, latent, rope, 0, RotaryLayout::SplitHalf, 0, nullptr, nullptr);
}

Result<Unit> RocmContext::append_mla_rope(RocmKvCache& cache, size_t layer, const RocmTensor& latent, const RocmTensor& rope, size_t rotary_dim,
                                          RotaryLayout layout, size_t position, const std::vector<float>& cos, const std::vector<float>& sin) const
{
    const size_t half = rotary_dim / 2;
    if (rotary_dim == 0 || rotary_dim % 2 != 0 || rotary_dim > rope.cols || cos.size() != sin.size() ||
        cos.size() < (position + rope.rows) * half) {
        return compute_error("Rocm MLA append: rotary tables do not cover position " + std::to_string(position));
    }
    auto tables = resident_rope_tables(cos, sin, (position + rope.rows) * half);
    if (tables.is_err()) {
        return tables.unwrap_err();
    }
    return append_mla_impl(cache, layer, latent, rope, rotary_dim, layout, position, tables.unwrap().first, tables.unwrap().second);
}

Result<RocmTensor> RocmContext::mla_decode_attention(const RocmTensor& query, const RocmKvCache& cache, const RocmWeight& kv_b, size_t layer,
                                                     size_t position, const MlaSpec& spec) const
{
    return mla_decode_impl(query, cache, kv_b, layer, position, spec, nullptr);
}

Result<RocmTensor> RocmContext::mla_decode_attention_selected(const RocmTensor& query, const RocmKvCache& cache, const RocmWeight& kv_b,
                                                              size_t layer, size_t position, const MlaSpec& mla, const DsaSpec& dsa,
                                                              const RocmDsaState& state) const
{
    if (dsa.top_k == 0 || state.top_k != dsa.top_k || state.selection.data() == nullptr) {
        return compute_error("Rocm MLA selected decode: the DSA state holds " + std::to_string(state.top_k) + " positions, top_k is " +
                             std::to_string(dsa.top_k));
    }
    return mla_decode_impl(query, cache, kv_b, layer, position, mla, &state);
}

Result<RocmDsaState> RocmContext::dsa_state_from_selection(const std::vector<uint32_t>& selection) const
{
    if (selection.empty()) {
        return compute_error("Rocm DSA state: empty selection");
    }
    auto buffer = upload_words(selection.data(), selection.size());
    if (buffer.is_err()) {
        return buffer.unwrap_err();
    }
    RocmDsaState state;
    state.selection = buffer.unwrap();
    state.top_k = selection.size();
    return state;
}

Result<RocmTensor> RocmContext::mla_decode_impl(const RocmTensor& query, const RocmKvCache& cache, const RocmWeight& kv_b, size_t layer,
                                                size_t position, const MlaSpec& spec, const RocmDsaState* state) const
{
    if (auto bad = spec.validate()) {
        return compute_error(*bad);
    }
    if (!cache.mla_ || layer >= cache.layers_.size()) {
        return unsupported_layer(layer);
    }
    // `query.rows` query rows that are the last rows of the cache: one for a decode step, a chunk's worth for a prefill
    if (query.rows == 0 || query.cols != spec.q_projection_size || spec.kv_lora_rank != cache.cols_ || spec.qk_rope_head_dim != cache.rope_cols_ ||
        kv_b.rows != spec.kv_projection_size || kv_b.cols != spec.kv_lora_rank) {
        return compute_error("Rocm MLA decode shape mismatch: Q=[" + std::to_string(query.rows) + "," + std::to_string(query.cols) + "] kv_b=[" +
                             std::to_string(kv_b.rows) + "," + std::to_string(kv_b.cols) + "]");
    }
    const size_t ctx = cache.lens_[layer];
    if (ctx == 0 || position + query.rows != ctx) {
        return compute_error("Rocm MLA L" + std::to_string(layer) + " cache length " + std::to_string(ctx) + " does not match position " +
                             std::to_string(position));
    }
    const bool chunk = query.rows > 1;
    const size_t out_cols = spec.num_heads * spec.value_dim();
    // a decode row is written as f32, the rows of a chunk as bf16 (src/backend/rocm/attention.rs:17-19)
    auto out_buf = pooled(query.rows * out_cols * (chunk ? 2 : 4));
    if (out_buf.is_err()) {
        return out_buf.unwrap_err();
    }
    const uint32_t host_meta[4] = {(uint32_t)ctx, 0u, 0u, 0u};
    auto meta = upload_meta(host_meta);
    if (meta.is_err()) {
        return meta.unwrap_err();
    }
    const RocmKvCache::Layer& planes = cache.layers_[layer];
    zllm_mla_decode_args a;
    memset(&a, 0, sizeof(a));
    a.q = query.device.data();
    a.kv_b = (const uint16_t*)kv_b.device.data();
    a.latent_codes = (const int8_t*)planes.a_codes.data();
    a.latent_scales = (const uint16_t*)planes.a_scales.data();
    a.rope_cache = (const uint16_t*)planes.b_codes.data();
    a.tables = (const uint32_t*)cache.table_.data();
    a.ctx_lens = meta.unwrap();
    a.out = out_buf.unwrap().data();
    a.batch = 1;
    a.query_rows = (uint32_t)query.rows;
    a.heads = (uint32_t)spec.num_heads;
    a.q_head_dim = (uint32_t)spec.q_head_dim();
    a.kv_head_dim = (uint32_t)spec.kv_head_dim();
    a.latent_dim = (uint32_t)spec.kv_lora_rank;
    a.rope_dim = (uint32_t)spec.qk_rope_head_dim;
    a.table_stride = (uint32_t)cache.table_host_.size();
    a.max_ctx_len = (uint32_t)ctx;
    a.block_tokens = (uint32_t)cache.block_tokens_;
    a.q_dtype = abi_dtype(query.dtype);
    a.out_dtype = chunk ? ZLLM_DTYPE_BF16 : ZLLM_DTYPE_F32;
    a.out_compact = 1;
    if (state != nullptr) {
        a.selection = (const uint32_t*)state->selection.data();
        a.top_k = (uint32_t)state->top_k;
    }
    if (kv_b.bits != 16) {
        a.kv_b_bits = kv_b.bits;
        a.kv_b_scales = kv_b.scales.data();
        a.kv_b_group = (uint32_t)kv_b.group_size;
        a.kv_b_scale_dtype = kv_b.scale_dtype == DType::F32 ? ZLLM_SCALE_F32 : (kv_b.scale_dtype == DType::F16 ? ZLLM_SCALE_F16 : ZLLM_SCALE_BF16);
    }
    const uint64_t need = zllm_attn_mla_decode_workspace_bytes(&a);
    if (need == 0) {
        return abi_error("zllm_attn_mla_decode_workspace_bytes", -1);
    }
    auto ws = workspace(need);
    if (ws.is_err()) {
        return ws.unwrap_err();
    }
    a.workspace = ws.unwrap();
    a.workspace_bytes = need;
    const int rc = zllm_attn_mla_decode(&a, stream_);
    if (rc != 0) {
        return abi_error("zllm_attn_mla_decode", rc);
    }
    RocmTensor out;
    out.device = out_buf.unwrap();
    out.rows = query.rows;
    out.cols = out_cols;
    out.dtype = chunk ? DType::BF16 : DType::F32;
    return out;
}

Result<RocmTensor> RocmContext::mla_prefill_attention(const RocmTensor& query, const RocmTensor& latent, const RocmTensor& k_rope,
                                                      const RocmWeight& kv_b, RocmKvCache* cache, size_t layer, const MlaSpec& spec) const
{
    if (cache == nullptr) {
        return compute_error("L" + std::to_string(layer) + " ROCm MLA prefill needs a paged cache");
    }
    if (query.rows != latent.rows) {
        return compute_error("Rocm MLA prefill shape mismatch: Q rows=" + std::to_string(query.rows) + " latent rows=" + std::to_string(latent.rows));
    }
    const size_t position = cache->len(layer);
    auto appended = append_mla(*cache, layer, latent, k_rope);
    if (appended.is_err()) {
        return appended.unwrap_err();
    }
    auto out = mla_decode_impl(query, *cache, kv_b, layer, position, spec, nullptr);
    if (out.is_err()) {
        (void)cache->truncate_layer_rows(layer, position); // a failed call leaves the cache length alone
    }
    return out;
}

Result<RocmTensor> RocmContext::mla_prefill_attention_rope(const RocmTensor& query, const RocmTensor& latent, const RocmTensor& k_rope,
                                                           const RocmWeight& kv_b, RocmKvCache* cache, size_t layer, size_t position,
                                                           const std::vector<float>& cos, const std::vector<float>& sin, const MlaSpec& spec) const
{
    if (cache == nullptr) {
        return compute_error("L" + std::to_string(layer) + " ROCm MLA prefill needs a paged cache");
    }
    if (query.rows != latent.rows) {
        return compute_error("Rocm MLA prefill shape mismatch: Q rows=" + std::to_string(query.rows) + " latent rows=" + std::to_string(latent.rows));
    }
    const size_t before = cache->len(layer);
    auto appended = append_mla_rope(*cache, layer, latent, k_rope, spec.qk_rope_head_dim, spec.rotary_layout, position, cos, sin);
    if (appended.is_err()) {
        return appended.unwrap_err();
    }
    auto out = mla_decode_impl(query, *cache, kv_b, layer, before, spec, nullptr);
    if (out.is_err()) {
        (void)cache->truncate_layer_rows(layer, before);
    }
    return out;
}

Result<std::vector<std::optional<MlaLayerSerde>>> RocmContext::download_layers(const RocmKvCache& cache) const
{
    if (!cache.mla_) {
        return compute_error("ROCm KV snapshot: not an MLA cache");
    }
    std::vector<std::optional<MlaLayerSerde>> out;
    for (size_t l = 0; l < cache.layers_.size(); ++l) {
        const RocmKvCache::Layer& planes = cache.layers_[l];
        MlaLayerSerde record;
        record.rows = cache.lens_[l];
        record.latent_cols = cache.cols_;
        record.rope_cols = cache.rope_cols_;
        record.latent_group_size = 64;
        const size_t row_bytes[3] = {cache.cols_, cache.cols_ / 64 * 2, cache.rope_cols_ * 2};
        const void* sources[3] = {planes.a_codes.data(), planes.a_scales.data(), planes.b_codes.data()};
        std::vector<uint8_t> host[3];
        for (int i = 0; i < 3; ++i) {
            host[i].resize(record.rows * row_bytes[i]);
            if (record.rows == 0) {
                continue;
            }
            auto dense = DeviceBuffer::allocate(host[i].size());
            if (dense.is_err()) {
                return dense.unwrap_err();
            }
            zllm_gather_args g;
            memset(&g, 0, sizeof(g));
            g.plane = sources[i];
            g.out = dense.unwrap().data();
            g.table = (const uint32_t*)cache.table_.data();
            g.first = 0;
            g.count = (uint32_t)record.rows;
            g.row_bytes = (uint32_t)row_bytes[i];
            g.block_tokens = (uint32_t)cache.block_tokens_;
            const int code = zllm_attn_gather_rows(&g, stream_);
            if (code != 0) {
                return abi_error("zllm_attn_gather_rows", code);
            }
            hipError_t err = hipMemcpyAsync(host[i].data(), dense.unwrap().data(), host[i].size(), hipMemcpyDeviceToHost, stream_);
            if (err == hipSuccess) {
                err = hipStreamSynchronize(stream_);
            }
            if (err != hipSuccess) {
                return hip_error("KV snapshot download", err);
            }
        }
        record.latent = std::move(host[0]);
        record.latent_scales = std::move(host[1]);
        record.rope = std::move(host[2]);
        out.push_back(std::move(record));
    }
    return out;
}

Result<Unit> RocmContext::upload_layers(RocmKvCache& cache, const std::vector<std::optional<MlaLayerSerde>>& layers) const
{
    if (!cache.mla_ || layers.size() != cache.layers_.size()) {
        return compute_error("ROCm KV snapshot: layer count " + std::to_string(layers.size()) + " does not match the cache");
    }
    for (size_t l = 0; l < layers.size(); ++l) {
        if (!layers[l].has_value()) {
            continue;
        }
        const MlaLayerSerde& record = *layers[l];
        if (record.latent_cols != cache.cols_ || record.rope_cols != cache.rope_cols_ || record.latent_group_size != 64 ||
            !record.latent_scales.has_value() || record.rows > cache.max_tokens_ || record.latent.size() != record.rows * cache.cols_ ||
            record.latent_scales->size() != record.rows * (cache.cols_ / 64) * 2 || record.rope.size() != record.rows * cache.rope_cols_ * 2) {
            return compute_error("L" + std::to_string(l) + " ROCm KV snapshot: record shape does not match the cache");
        }
        if (record.rows != 0) {
            // the restored rows are committed in one step, at the capacity the growth rule gives for them
            // (upload_cache_buffer, src/backend/rocm/mod.rs:324-333)
            auto reserved = cache.reserve_rows(l, record.rows, stream_);
            if (reserved.is_err()) {
                return reserved.unwrap_err();
            }
        }
        RocmKvCache::Layer& planes = cache.layers_[l];
        const size_t row_bytes[3] = {cache.cols_, cache.cols_ / 64 * 2, cache.rope_cols_ * 2};
        void* targets[3] = {planes.a_codes.data(), planes.a_scales.data(), planes.b_codes.data()};
        const std::vector<uint8_t>* host[3] = {&record.latent, &*record.latent_scales, &record.rope};
        for (int i = 0; i < 3 && record.rows != 0; ++i) {
            auto dense = DeviceBuffer::allocate(host[i]->size());
            if (dense.is_err()) {
                return dense.unwrap_err();
            }
            hipError_t err = hipMemcpyAsync(dense.unwrap().data(), host[i]->data(), host[i]->size(), hipMemcpyHostToDevice, stream_);
            if (err != hipSuccess) {
                return hip_error("KV snapshot upload", err);
            }
            zllm_scatter_args sc;
            memset(&sc, 0, sizeof(sc));
            sc.plane = targets[i];
            sc.in = dense.unwrap().data();
            sc.table = (const uint32_t*)cache.table_.data();
            sc.first = 0;
            sc.count = (uint32_t)record.rows;
            sc.row_bytes = (uint32_t)row_bytes[i];
            sc.block_tokens = (uint32_t)cache.block_tokens_;
            const int code = zllm_attn_scatter_rows(&sc, stream_);
            if (code != 0) {
                return abi_error("zllm_attn_scatter_rows", code);
            }
            err = hipStreamSynchronize(stream_);
            if (err != hipSuccess) {
                return hip_error("KV snapshot upload", err);
            }
        }
        cache.lens_[l] = record.rows;
    }
    return Unit{};
}

} // namespace zllm_amd

// Parity of the C++ host layer (zllm_amd/host/rocm_backend.hpp) with the CPU oracle, written the way the
// reference tests its backends: build inputs, call the trait method, compare with the CPU reference
// (src/backend/mod.rs tests around gqa_prefill_attention_cached; tolerance of the attention path:
// max-abs 2e-3, relative 1e-2).  Run by tests/test_gpu_host_backend.py on a GPU box.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <random>
#include <string>
#include <vector>

#include "../../zllm_amd/host/rocm_backend.hpp"

extern "C" {
// oracle/zllm_oracle.c (test infrastructure)
uint16_t zo_f32_to_bf16(float value);
float zo_bf16_to_f32(uint16_t value);
int zo_q8g64_append_paged(int rule, const float* input, int8_t* codes, void* scales, const uint32_t* block_table, uint64_t position,
                          uint64_t rows, uint64_t cols, uint64_t group, uint32_t block_size, uint64_t ring_capacity);
int zo_half_append_paged(int dtype, const float* input, uint16_t* cache, const uint32_t* block_table, uint64_t position, uint64_t rows,
                         uint64_t cols, uint32_t block_size, uint64_t ring_capacity);
int zo_gather_dequant_rows(int format, const void* plane, const void* scales, int scale_dtype, const uint32_t* block_table,
                           uint32_t block_size, uint64_t ring_capacity, uint64_t first, uint64_t count, uint64_t cols, uint64_t group,
                           float* out);
int zo_gather_rows_bytes(const uint8_t* plane, const uint32_t* block_table, uint32_t block_size, uint64_t ring_capacity, uint64_t first,
                         uint64_t count, uint64_t row_bytes, uint8_t* out);
int zo_gqa_prefill_at_visible_f32(const float* query, const float* key, const float* value, uint64_t query_tokens, uint64_t kv_start,
                                  uint64_t kv_end, uint64_t position, uint64_t num_heads, uint64_t num_kv_heads, uint64_t head_dim,
                                  uint64_t window, float score_scale, float softcap, const uint32_t* visible_ends, float* output);
int zo_block_attention_f32(const float* query, const float* key, const float* value, uint64_t query_rows, uint64_t kv_rows, uint64_t num_heads,
                           uint64_t num_kv_heads, uint64_t head_dim, float score_scale, const uint32_t* visible, float* output);
int zo_rope_apply_f32(float* data, uint64_t rows, uint64_t columns, uint64_t head_count, uint64_t rotary_dim, uint64_t position,
                      const float* cosine, const float* sine, uint64_t table_len, int layout, int placement);
typedef struct {
    uint64_t kv_lora_rank, qk_rope_head_dim, q_projection_size, kv_projection_size, num_heads;
} zo_mla_spec;
int zo_mla_absorbed_q8_history(const zo_mla_spec* spec, const uint16_t* query, uint64_t query_rows, uint64_t query_start,
                               const uint8_t* latent_codes, const uint16_t* latent_scales, uint64_t latent_group_size, const uint16_t* rope,
                               uint64_t history_rows, const float* kv_b, const uint32_t* selection, uint64_t width, uint16_t* out_bf16,
                               float* out_f32, float* weighted_f32);
}

using namespace zllm_amd;

static int failures = 0;

#define CHECK(cond, ...)                          \
    do {                                          \
        if (!(cond)) {                            \
            printf("FAIL %s:%d: ", __FILE__, __LINE__); \
            printf(__VA_ARGS__);                  \
            printf("\n");                         \
            ++failures;                           \
        }                                         \
    } while (0)

static std::vector<float> randn(std::mt19937& rng, size_t n, bool bf16_round)
{
    std::normal_distribution<float> dist(0.0f, 1.0f);
    std::vector<float> out(n);
    for (auto& x : out) {
        x = dist(rng);
        if (bf16_round) {
            x = zo_bf16_to_f32(zo_f32_to_bf16(x));
        }
    }
    return out;
}

static void compare(const std::vector<float>& got, const std::vector<float>& want, const char* what)
{
    CHECK(got.size() == want.size(), "%s: size %zu vs %zu", what, got.size(), want.size());
    double max_abs = 0, num = 0, den = 0;
    for (size_t i = 0; i < got.size() && i < want.size(); ++i) {
        const double d = (double)got[i] - want[i];
        max_abs = fmax(max_abs, fabs(d));
        num += d * d;
        den += (double)want[i] * want[i];
        if (!isfinite(got[i])) {
            max_abs = INFINITY;
        }
    }
    const double rel = den > 0 ? sqrt(num / den) : sqrt(num);
    printf("%-58s max-abs %.3e rel %.3e\n", what, max_abs, rel);
    CHECK(max_abs <= 2e-3, "%s: max-abs %.3e > 2e-3", what, max_abs);
    CHECK(rel <= 1e-2, "%s: relative %.3e > 1e-2", what, rel);
}

// ---------------------------------------------------------------------------------------------- GQA
static void test_gqa(const RocmContext& ctx, CausalWindow window, const char* label, TablePolicy policy)
{
    std::mt19937 rng(7);
    GqaSpec spec;
    spec.num_heads = 16;
    spec.num_kv_heads = 4;
    spec.head_dim = 128;
    spec.window = window;
    spec.score_scale = 1.0f / sqrtf(128.0f);
    const size_t kv_cols = spec.num_kv_heads * spec.head_dim, q_cols = spec.num_heads * spec.head_dim;
    const size_t block = 16, max_tokens = 1024;
    auto cache_r = RocmKvCache::new_gqa(2, spec.num_kv_heads, spec.head_dim, block, max_tokens, policy);
    CHECK(cache_r.is_ok(), "cache: %s", cache_r.is_err() ? cache_r.unwrap_err().to_string().c_str() : "");
    if (cache_r.is_err()) {
        return;
    }
    RocmKvCache cache = cache_r.unwrap();
    const size_t pool_rows = cache.block_table().size() * block;
    // the identity table commits rows as they are needed, the scrambled one commits its pool up front
    CHECK(cache.committed_rows(1) == (policy == TablePolicy::Identity ? 0 : pool_rows), "rows committed at creation: %zu", cache.committed_rows(1));
    size_t committed_want = 0;
    // the oracle's copy of layer 1's planes, filled by the oracle's quantizer through the same table
    std::vector<int8_t> k_codes(pool_rows * kv_cols), v_codes(pool_rows * kv_cols);
    std::vector<uint16_t> k_scales(pool_rows * kv_cols / 64), v_scales(pool_rows * kv_cols / 64);
    const size_t layer = 1;
    size_t position = 0;
    const size_t chunks[] = {300, 200, 1, 1, 37, 1};
    for (size_t rows : chunks) {
        const auto q = randn(rng, rows * q_cols, true);
        const auto k = randn(rng, rows * kv_cols, false);
        const auto v = randn(rng, rows * kv_cols, false);
        auto qt = ctx.tensor_from_f32(q, rows, q_cols, DType::BF16);
        auto kt = ctx.tensor_from_f32(k, rows, kv_cols);
        auto vt = ctx.tensor_from_f32(v, rows, kv_cols);
        CHECK(qt.is_ok() && kt.is_ok() && vt.is_ok(), "upload");
        auto out = ctx.gqa_prefill_attention_cached(cache, layer, position, qt.unwrap(), kt.unwrap(), vt.unwrap(), spec, true);
        CHECK(out.is_ok(), "%s rows=%zu: %s", label, rows, out.is_err() ? out.unwrap_err().to_string().c_str() : "");
        if (out.is_err()) {
            return;
        }
        auto got = ctx.tensor_to_f32(out.unwrap());
        CHECK(got.is_ok(), "download");
        zo_q8g64_append_paged(1, k.data(), k_codes.data(), k_scales.data(), cache.block_table().data(), position, rows, kv_cols, 64, block, 0);
        zo_q8g64_append_paged(1, v.data(), v_codes.data(), v_scales.data(), cache.block_table().data(), position, rows, kv_cols, 64, block, 0);
        const size_t total = position + rows;
        std::vector<float> kd(total * kv_cols), vd(total * kv_cols), want(rows * q_cols);
        zo_gather_dequant_rows(0, k_codes.data(), k_scales.data(), 1, cache.block_table().data(), block, 0, 0, total, kv_cols, 64, kd.data());
        zo_gather_dequant_rows(0, v_codes.data(), v_scales.data(), 1, cache.block_table().data(), block, 0, 0, total, kv_cols, 64, vd.data());
        const int rc = zo_gqa_prefill_at_visible_f32(q.data(), kd.data(), vd.data(), rows, 0, total, position, spec.num_heads, spec.num_kv_heads,
                                                     spec.head_dim, window.sliding ? window.size : 0, spec.score_scale, 0.0f, nullptr, want.data());
        CHECK(rc == 0, "oracle rc %d", rc);
        char what[128];
        snprintf(what, sizeof(what), "gqa_prefill_attention_cached %s position=%zu rows=%zu", label, position, rows);
        compare(got.unwrap(), want, what);
        position = total;
        CHECK(cache.len(layer) == position, "cache length %zu vs %zu", cache.len(layer), position);
        if (policy == TablePolicy::Identity) {
            // grow-by-doubling in 64-row multiples (src/backend/rocm/mod.rs:303-313), whole pages
            committed_want = committed_cache_rows(committed_want, total, pool_rows).unwrap();
            CHECK(cache.committed_rows(layer) == committed_want, "committed rows %zu, rule says %zu", cache.committed_rows(layer), committed_want);
            CHECK(cache.committed_rows(0) == 0, "a layer nothing was appended to holds no rows");
        }
    }
    // error behaviour of the reference's body (attention.rs:2213-2229)
    {
        const auto q = randn(rng, q_cols, true);
        const auto k = randn(rng, kv_cols, false);
        auto qt = ctx.tensor_from_f32(q, 1, q_cols);
        auto kt = ctx.tensor_from_f32(k, 1, kv_cols);
        auto stale = ctx.gqa_prefill_attention_cached(cache, layer, position - 1, qt.unwrap(), kt.unwrap(), kt.unwrap(), spec, true);
        CHECK(stale.is_err() && stale.unwrap_err().kind == BackendError::Kind::Compute, "a stale position must be a Compute error");
        auto wrong = ctx.gqa_prefill_attention_cached(cache, layer, position, qt.unwrap(), qt.unwrap(), kt.unwrap(), spec, true);
        CHECK(wrong.is_err() && wrong.unwrap_err().msg.find("shape") != std::string::npos, "a K of the wrong width must be a shape error");
        auto missing = ctx.gqa_prefill_attention_cached(cache, 9, position, qt.unwrap(), kt.unwrap(), kt.unwrap(), spec, true);
        CHECK(missing.is_err() && missing.unwrap_err().kind == BackendError::Kind::UnsupportedLayer && missing.unwrap_err().layer == 9,
              "a layer outside the cache must be UnsupportedLayer");
        CHECK(cache.len(layer) == position, "failed calls must not move the cache length");
    }
}

// ---------------------------------------------------------------------------------------------- MLA
static void test_mla(const RocmContext& ctx)
{
    std::mt19937 rng(11);
    MlaSpec spec;
    spec.kv_lora_rank = 512;
    spec.qk_rope_head_dim = 64;
    spec.num_heads = 16;
    spec.q_projection_size = spec.num_heads * 192;  // nope 128 + rope 64
    spec.kv_projection_size = spec.num_heads * 256; // nope 128 + value 128
    spec.q_lora_rank = 1536;
    CHECK(!spec.validate().has_value(), "spec must validate");
    const size_t block = 64, max_tokens = 700, layer = 0;
    auto cache_r = RocmKvCache::new_mla(1, 512, 64, block, max_tokens, TablePolicy::Scrambled);
    CHECK(cache_r.is_ok(), "cache");
    if (cache_r.is_err()) {
        return;
    }
    RocmKvCache cache = cache_r.unwrap();
    const size_t pool_rows = cache.block_table().size() * block;
    std::vector<int8_t> ref_codes(pool_rows * 512);
    std::vector<uint16_t> ref_scales(pool_rows * 8), ref_rope(pool_rows * 64);
    // rotary tables for 1,024 positions
    const size_t rotary_dim = 64, half = rotary_dim / 2, table_rows = 1024;
    std::vector<float> cos(table_rows * half), sin(table_rows * half);
    for (size_t pos = 0; pos < table_rows; ++pos) {
        for (size_t i = 0; i < half; ++i) {
            const float angle = (float)pos * powf(10000.0f, -2.0f * (float)i / (float)rotary_dim);
            cos[pos * half + i] = cosf(angle);
            sin[pos * half + i] = sinf(angle);
        }
    }
    // a bulk append of rows whose rope is already rotated, then single-row appends with the rotation fused
    const size_t bulk = 555, singles = 3;
    {
        const auto latent = randn(rng, bulk * 512, false);
        const auto rope = randn(rng, bulk * 64, false);
        auto lt = ctx.tensor_from_f32(latent, bulk, 512);
        auto rt = ctx.tensor_from_f32(rope, bulk, 64);
        auto done = ctx.append_mla(cache, layer, lt.unwrap(), rt.unwrap());
        CHECK(done.is_ok(), "append_mla: %s", done.is_err() ? done.unwrap_err().to_string().c_str() : "");
        zo_q8g64_append_paged(0, latent.data(), ref_codes.data(), ref_scales.data(), cache.block_table().data(), 0, bulk, 512, 64, block, 0);
        zo_half_append_paged(0, rope.data(), ref_rope.data(), cache.block_table().data(), 0, bulk, 64, block, 0);
    }
    for (size_t s = 0; s < singles; ++s) {
        const size_t position = bulk + s;
        const auto latent = randn(rng, 512, false);
        auto rope = randn(rng, 64, false);
        auto lt = ctx.tensor_from_f32(latent, 1, 512);
        auto rt = ctx.tensor_from_f32(rope, 1, 64);
        auto done = ctx.append_mla_rope(cache, layer, lt.unwrap(), rt.unwrap(), rotary_dim, RotaryLayout::SplitHalf, position, cos, sin);
        CHECK(done.is_ok(), "append_mla_rope: %s", done.is_err() ? done.unwrap_err().to_string().c_str() : "");
        zo_rope_apply_f32(rope.data(), 1, 64, 1, rotary_dim, position, cos.data(), sin.data(), cos.size(), 0, 1);
        zo_q8g64_append_paged(0, latent.data(), ref_codes.data(), ref_scales.data(), cache.block_table().data(), position, 1, 512, 64, block, 0);
        zo_half_append_paged(0, rope.data(), ref_rope.data(), cache.block_table().data(), position, 1, 64, block, 0);
    }
    const size_t ctx_len = bulk + singles;
    CHECK(cache.len(layer) == ctx_len, "cache length %zu", cache.len(layer));

    const size_t q_cols = spec.q_projection_size;
    const auto q = randn(rng, q_cols, true);
    std::vector<float> kv_b = randn(rng, spec.kv_projection_size * 512, true);
    for (auto& w : kv_b) {
        w *= 0.05f;
        w = zo_bf16_to_f32(zo_f32_to_bf16(w));
    }
    auto qt = ctx.tensor_from_f32(q, 1, q_cols, DType::BF16);
    auto weight = ctx.prepare_mla_kv_b(kv_b, spec.kv_projection_size, 512);
    CHECK(qt.is_ok() && weight.is_ok(), "upload");
    auto out = ctx.mla_decode_attention(qt.unwrap(), cache, weight.unwrap(), layer, ctx_len - 1, spec);
    CHECK(out.is_ok(), "mla_decode_attention: %s", out.is_err() ? out.unwrap_err().to_string().c_str() : "");
    if (out.is_err()) {
        return;
    }
    auto got = ctx.tensor_to_f32(out.unwrap());

    // oracle on the dense history gathered from ITS planes (the device planes are bit-identical: tests/test_gpu_append.py)
    std::vector<uint8_t> codes_dense(ctx_len * 512);
    std::vector<uint16_t> scales_dense(ctx_len * 8), rope_dense(ctx_len * 64), q_bits(q_cols);
    zo_gather_rows_bytes((const uint8_t*)ref_codes.data(), cache.block_table().data(), block, 0, 0, ctx_len, 512, codes_dense.data());
    zo_gather_rows_bytes((const uint8_t*)ref_scales.data(), cache.block_table().data(), block, 0, 0, ctx_len, 16, (uint8_t*)scales_dense.data());
    zo_gather_rows_bytes((const uint8_t*)ref_rope.data(), cache.block_table().data(), block, 0, 0, ctx_len, 128, (uint8_t*)rope_dense.data());
    for (size_t i = 0; i < q_cols; ++i) {
        q_bits[i] = zo_f32_to_bf16(q[i]);
    }
    zo_mla_spec zs = {512, 64, spec.q_projection_size, spec.kv_projection_size, spec.num_heads};
    std::vector<float> want(spec.num_heads * spec.value_dim());
    const int rc = zo_mla_absorbed_q8_history(&zs, q_bits.data(), 1, ctx_len - 1, codes_dense.data(), scales_dense.data(), 64, rope_dense.data(),
                                              ctx_len, kv_b.data(), nullptr, 0, nullptr, want.data(), nullptr);
    CHECK(rc == 0, "oracle rc %d", rc);
    compare(got.unwrap(), want, "mla_decode_attention after append_mla + append_mla_rope");

    // selected-token decode (DecodeBackend::mla_decode_attention_selected): 64 listed positions out of the context
    {
        std::vector<uint32_t> selection;
        for (uint32_t s = 0; s < 64; ++s) {
            selection.push_back((uint32_t)((s * 37u + 5u) % ctx_len)); // 37 and ctx_len are coprime here: distinct positions
        }
        auto state = ctx.dsa_state_from_selection(selection);
        CHECK(state.is_ok(), "dsa_state_from_selection");
        DsaSpec dsa;
        dsa.top_k = selection.size();
        auto picked = ctx.mla_decode_attention_selected(qt.unwrap(), cache, weight.unwrap(), layer, ctx_len - 1, spec, dsa, state.unwrap());
        CHECK(picked.is_ok(), "mla_decode_attention_selected: %s", picked.is_err() ? picked.unwrap_err().to_string().c_str() : "");
        if (picked.is_ok()) {
            std::vector<float> want_sel(spec.num_heads * spec.value_dim());
            const int rc3 = zo_mla_absorbed_q8_history(&zs, q_bits.data(), 1, ctx_len - 1, codes_dense.data(), scales_dense.data(), 64, rope_dense.data(),
                                                       ctx_len, kv_b.data(), selection.data(), selection.size(), nullptr, want_sel.data(), nullptr);
            CHECK(rc3 == 0, "oracle rc %d", rc3);
            compare(ctx.tensor_to_f32(picked.unwrap()).unwrap(), want_sel, "mla_decode_attention_selected, top_k 64");
        }
        dsa.top_k = 63;
        CHECK(ctx.mla_decode_attention_selected(qt.unwrap(), cache, weight.unwrap(), layer, ctx_len - 1, spec, dsa, state.unwrap()).is_err(),
              "a state of another top_k must be refused");
    }

    // session snapshot: download -> wire bytes -> parse -> upload into a second cache (other pages), same result bit for bit
    {
        auto layers = ctx.download_layers(cache);
        CHECK(layers.is_ok(), "download_layers: %s", layers.is_err() ? layers.unwrap_err().to_string().c_str() : "");
        std::vector<uint8_t> bytes;
        for (const auto& record : layers.unwrap()) {
            CHECK(record.has_value() && write_mla_layer(bytes, *record).is_ok(), "write_mla_layer");
        }
        const MlaLayerSerde& first = *layers.unwrap()[layer];
        CHECK(first.rows == ctx_len && first.latent.size() == ctx_len * 512 && memcmp(first.latent.data(), codes_dense.data(), first.latent.size()) == 0 &&
                  memcmp(first.latent_scales->data(), scales_dense.data(), ctx_len * 16) == 0 && memcmp(first.rope.data(), rope_dense.data(), ctx_len * 128) == 0,
              "downloaded layer differs from the oracle's dense history");
        std::vector<std::optional<MlaLayerSerde>> parsed;
        size_t offset = 0;
        for (size_t l = 0; l < cache.layers(); ++l) {
            auto record = read_mla_layer(bytes, offset);
            CHECK(record.is_ok(), "read_mla_layer: %s", record.is_err() ? record.unwrap_err().to_string().c_str() : "");
            parsed.push_back(record.unwrap());
        }
        CHECK(offset == bytes.size(), "wire bytes left over");
        auto other = RocmKvCache::new_mla(cache.layers(), 512, 64, 32, 640); // 32-token pages instead of 64
        CHECK(other.is_ok(), "second cache");
        auto restored = ctx.upload_layers(other.unwrap(), parsed);
        CHECK(restored.is_ok() && other.unwrap().len(layer) == ctx_len, "upload_layers");
        auto again = ctx.mla_decode_attention(qt.unwrap(), other.unwrap(), weight.unwrap(), layer, ctx_len - 1, spec);
        CHECK(again.is_ok(), "decode on the restored cache");
        if (again.is_ok()) {
            auto same = ctx.tensor_to_f32(again.unwrap());
            CHECK(same.unwrap() == got.unwrap(), "restored cache decodes differently");
        }
        std::vector<uint8_t> cut(bytes.begin(), bytes.end() - 1);
        size_t at = 0;
        bool failed = false;
        for (size_t l = 0; l < cache.layers() && !failed; ++l) {
            failed = read_mla_layer(cut, at).is_err();
        }
        CHECK(failed, "a truncated snapshot must be refused");
        // rollback: the logical length moves back, a stale position is refused, a shorter decode works
        CHECK(other.unwrap().truncate_layer_rows(layer, ctx_len + 1).is_err(), "truncate beyond the current length");
        CHECK(other.unwrap().truncate_layer_rows(99, 1).is_err(), "truncate of a layer the cache does not have");
        CHECK(other.unwrap().truncate_layer_rows(layer, 100).is_ok() && other.unwrap().len(layer) == 100, "truncate_layer_rows");
        CHECK(ctx.mla_decode_attention(qt.unwrap(), other.unwrap(), weight.unwrap(), layer, ctx_len - 1, spec).is_err(), "stale position after rollback");
        auto shorter = ctx.mla_decode_attention(qt.unwrap(), other.unwrap(), weight.unwrap(), layer, 99, spec);
        CHECK(shorter.is_ok(), "decode after rollback");
        if (shorter.is_ok()) {
            std::vector<float> want_short(spec.num_heads * spec.value_dim());
            const int rc2 = zo_mla_absorbed_q8_history(&zs, q_bits.data(), 1, 99, codes_dense.data(), scales_dense.data(), 64, rope_dense.data(), 100,
                                                       kv_b.data(), nullptr, 0, nullptr, want_short.data(), nullptr);
            CHECK(rc2 == 0, "oracle rc %d", rc2);
            compare(ctx.tensor_to_f32(shorter.unwrap()).unwrap(), want_short, "mla_decode_attention after truncate_layer_rows(100)");
        }
        CHECK(other.unwrap().truncate_rows(0).is_ok() && other.unwrap().len(layer) == 0, "truncate_rows(0)");
    }

    auto stale = ctx.mla_decode_attention(qt.unwrap(), cache, weight.unwrap(), layer, ctx_len + 5, spec);
    CHECK(stale.is_err(), "a position beyond the cache must be an error");
    MlaSpec bad = spec;
    bad.q_projection_size += 1;
    CHECK(bad.validate().has_value(), "inconsistent head dimensions must not validate");
}


// ---------------------------------------------------------------------------------------------- growth rule, ring, shared KV, visible ends
static void test_growth_rule()
{
    struct Case {
        size_t current, required, limit, want;
    };
    const Case cases[] = {{0, 1, 1000, 64}, {64, 65, 1000, 128}, {128, 129, 200, 200}, {64, 300, 1000, 320}, {100, 50, 1000, 100},
                          {0, 1000, 1000, 1000}, {512, 513, 8192, 1024}};
    for (const Case& c : cases) {
        auto rows = committed_cache_rows(c.current, c.required, c.limit);
        CHECK(rows.is_ok() && rows.unwrap() == c.want, "committed_cache_rows(%zu, %zu, %zu) = %zu, want %zu", c.current, c.required, c.limit,
              rows.is_ok() ? rows.unwrap() : (size_t)0, c.want);
    }
    CHECK(committed_cache_rows(0, 5, 3).is_err() && committed_cache_rows(0, 0, 3).is_err(), "required outside (0, limit] must be refused");
}

// A sliding-window layer that keeps a ring of `window` rows (retain_full_cache == false): a chunk longer than the ring at
// position 0, then decode steps that wrap the ring; the oracle keeps every row and applies the window.
static void test_gqa_ring(const RocmContext& ctx)
{
    std::mt19937 rng(23);
    GqaSpec spec;
    spec.num_heads = 8;
    spec.num_kv_heads = 2;
    spec.head_dim = 128;
    spec.window = CausalWindow::Sliding(96);
    spec.score_scale = 1.0f / sqrtf(128.0f);
    const size_t kv_cols = spec.num_kv_heads * spec.head_dim, q_cols = spec.num_heads * spec.head_dim;
    const size_t block = 16, max_tokens = 2048, layer = 0;
    auto cache_r = RocmKvCache::new_gqa(1, spec.num_kv_heads, spec.head_dim, block, max_tokens);
    CHECK(cache_r.is_ok(), "ring cache");
    if (cache_r.is_err()) {
        return;
    }
    RocmKvCache cache = cache_r.unwrap();
    std::vector<float> all_k, all_v; // the oracle's history: raw rows, quantized through an identity table below
    size_t position = 0;
    const size_t chunks[] = {300, 1, 1, 1, 1, 1};
    for (size_t rows : chunks) {
        const auto q = randn(rng, rows * q_cols, true);
        const auto k = randn(rng, rows * kv_cols, false);
        const auto v = randn(rng, rows * kv_cols, false);
        auto out = ctx.gqa_prefill_attention_cached(cache, layer, position, ctx.tensor_from_f32(q, rows, q_cols, DType::BF16).unwrap(),
                                                    ctx.tensor_from_f32(k, rows, kv_cols).unwrap(), ctx.tensor_from_f32(v, rows, kv_cols).unwrap(), spec,
                                                    false);
        CHECK(out.is_ok(), "ring rows=%zu: %s", rows, out.is_err() ? out.unwrap_err().to_string().c_str() : "");
        if (out.is_err()) {
            return;
        }
        all_k.insert(all_k.end(), k.begin(), k.end());
        all_v.insert(all_v.end(), v.begin(), v.end());
        const size_t total = position + rows;
        std::vector<int8_t> kc(total * kv_cols), vc(total * kv_cols);
        std::vector<uint16_t> ks(total * kv_cols / 64), vs(total * kv_cols / 64);
        zo_q8g64_append_paged(1, all_k.data(), kc.data(), ks.data(), nullptr, 0, total, kv_cols, 64, block, 0);
        zo_q8g64_append_paged(1, all_v.data(), vc.data(), vs.data(), nullptr, 0, total, kv_cols, 64, block, 0);
        std::vector<float> kd(total * kv_cols), vd(total * kv_cols), want(rows * q_cols);
        zo_gather_dequant_rows(0, kc.data(), ks.data(), 1, nullptr, block, 0, 0, total, kv_cols, 64, kd.data());
        zo_gather_dequant_rows(0, vc.data(), vs.data(), 1, nullptr, block, 0, 0, total, kv_cols, 64, vd.data());
        const int rc = zo_gqa_prefill_at_visible_f32(q.data(), kd.data(), vd.data(), rows, 0, total, position, spec.num_heads, spec.num_kv_heads,
                                                     spec.head_dim, 96, spec.score_scale, 0.0f, nullptr, want.data());
        CHECK(rc == 0, "oracle rc %d", rc);
        char what[128];
        snprintf(what, sizeof(what), "gqa_prefill_attention_cached ring(96) position=%zu rows=%zu", position, rows);
        compare(ctx.tensor_to_f32(out.unwrap()).unwrap(), want, what);
        position = total;
    }
    CHECK(cache.ring_capacity(layer) == 96 && cache.committed_rows(layer) <= 128, "ring of 96 rows in %zu committed rows", cache.committed_rows(layer));
    // a multi-token chunk at a non-zero position of a draining sliding layer is refused, as on the reference's CPU backend
    const auto q2 = randn(rng, 2 * q_cols, true);
    const auto k2 = randn(rng, 2 * kv_cols, false);
    auto refused = ctx.gqa_prefill_attention_cached(cache, layer, position, ctx.tensor_from_f32(q2, 2, q_cols).unwrap(),
                                                    ctx.tensor_from_f32(k2, 2, kv_cols).unwrap(), ctx.tensor_from_f32(k2, 2, kv_cols).unwrap(), spec, false);
    CHECK(refused.is_err() && cache.len(layer) == position, "multi-token chunk on a wrapped ring must be refused and leave the length alone");
}

// gqa_prefill_attention_cached_from (a layer that shares another layer's K/V) and _visible (explicit visible ends)
static void test_gqa_shared_and_visible(const RocmContext& ctx)
{
    std::mt19937 rng(29);
    GqaSpec spec;
    spec.num_heads = 8;
    spec.num_kv_heads = 2;
    spec.head_dim = 128;
    spec.window = CausalWindow::Full();
    spec.score_scale = 1.0f / sqrtf(128.0f);
    const size_t kv_cols = spec.num_kv_heads * spec.head_dim, q_cols = spec.num_heads * spec.head_dim;
    const size_t block = 16, prefix = 150, rows = 48, total = prefix + rows;
    auto cache_r = RocmKvCache::new_gqa(2, spec.num_kv_heads, spec.head_dim, block, 512, TablePolicy::Scrambled);
    CHECK(cache_r.is_ok(), "cache");
    if (cache_r.is_err()) {
        return;
    }
    RocmKvCache cache = cache_r.unwrap();
    const auto k = randn(rng, total * kv_cols, false);
    const auto v = randn(rng, total * kv_cols, false);
    const auto q0 = randn(rng, prefix * q_cols, true);
    const auto q = randn(rng, rows * q_cols, true);
    std::vector<float> k_head(k.begin(), k.begin() + prefix * kv_cols), v_head(v.begin(), v.begin() + prefix * kv_cols);
    std::vector<float> k_tail(k.begin() + prefix * kv_cols, k.end()), v_tail(v.begin() + prefix * kv_cols, v.end());
    auto first = ctx.gqa_prefill_attention_cached(cache, 1, 0, ctx.tensor_from_f32(q0, prefix, q_cols).unwrap(),
                                                  ctx.tensor_from_f32(k_head, prefix, kv_cols).unwrap(), ctx.tensor_from_f32(v_head, prefix, kv_cols).unwrap(),
                                                  spec, true);
    CHECK(first.is_ok(), "prefix");
    // rows of a visual block read to the end of their 16-row block
    std::vector<uint32_t> ends(rows);
    for (size_t r = 0; r < rows; ++r) {
        ends[r] = (uint32_t)std::min(prefix + (r / 16 + 1) * 16, total);
    }
    auto qt = ctx.tensor_from_f32(q, rows, q_cols);
    auto seen = ctx.gqa_prefill_attention_cached_visible(cache, 1, prefix, qt.unwrap(), ctx.tensor_from_f32(k_tail, rows, kv_cols).unwrap(),
                                                         ctx.tensor_from_f32(v_tail, rows, kv_cols).unwrap(), spec, ends, true);
    CHECK(seen.is_ok(), "visible: %s", seen.is_err() ? seen.unwrap_err().to_string().c_str() : "");
    std::vector<int8_t> kc(total * kv_cols), vc(total * kv_cols);
    std::vector<uint16_t> ks(total * kv_cols / 64), vs(total * kv_cols / 64);
    zo_q8g64_append_paged(1, k.data(), kc.data(), ks.data(), nullptr, 0, total, kv_cols, 64, block, 0);
    zo_q8g64_append_paged(1, v.data(), vc.data(), vs.data(), nullptr, 0, total, kv_cols, 64, block, 0);
    std::vector<float> kd(total * kv_cols), vd(total * kv_cols), want(rows * q_cols);
    zo_gather_dequant_rows(0, kc.data(), ks.data(), 1, nullptr, block, 0, 0, total, kv_cols, 64, kd.data());
    zo_gather_dequant_rows(0, vc.data(), vs.data(), 1, nullptr, block, 0, 0, total, kv_cols, 64, vd.data());
    int rc = zo_gqa_prefill_at_visible_f32(q.data(), kd.data(), vd.data(), rows, 0, total, prefix, spec.num_heads, spec.num_kv_heads, spec.head_dim, 0,
                                           spec.score_scale, 0.0f, ends.data(), want.data());
    CHECK(rc == 0, "oracle rc %d", rc);
    if (seen.is_ok()) {
        compare(ctx.tensor_to_f32(seen.unwrap()).unwrap(), want, "gqa_prefill_attention_cached_visible, 16-row blocks");
    }
    // a layer that shares layer 1's K/V sees the same visual blocks: the rows are in the cache already, so the bits are the same
    auto shared_seen = ctx.gqa_prefill_attention_cached_from_visible(cache, 1, prefix, qt.unwrap(), spec, ends);
    CHECK(shared_seen.is_ok(), "cached_from_visible: %s", shared_seen.is_err() ? shared_seen.unwrap_err().to_string().c_str() : "");
    if (shared_seen.is_ok() && seen.is_ok()) {
        CHECK(ctx.tensor_to_f32(shared_seen.unwrap()).unwrap() == ctx.tensor_to_f32(seen.unwrap()).unwrap(),
              "gqa_prefill_attention_cached_from_visible must give the bits of the appending call");
    }
    CHECK(ctx.gqa_prefill_attention_cached_from_visible(cache, 1, prefix, qt.unwrap(), spec, std::vector<uint32_t>(rows - 1, 1u)).is_err(),
          "one visible end too few must be refused");
    // layer 0 shares layer 1's K/V: the same chunk, causal, nothing appended
    auto shared = ctx.gqa_prefill_attention_cached_from(cache, 1, prefix, qt.unwrap(), spec);
    CHECK(shared.is_ok(), "cached_from: %s", shared.is_err() ? shared.unwrap_err().to_string().c_str() : "");
    rc = zo_gqa_prefill_at_visible_f32(q.data(), kd.data(), vd.data(), rows, 0, total, prefix, spec.num_heads, spec.num_kv_heads, spec.head_dim, 0,
                                       spec.score_scale, 0.0f, nullptr, want.data());
    CHECK(rc == 0, "oracle rc %d", rc);
    if (shared.is_ok()) {
        compare(ctx.tensor_to_f32(shared.unwrap()).unwrap(), want, "gqa_prefill_attention_cached_from layer 1");
    }
    CHECK(cache.len(0) == 0 && cache.len(1) == total, "shared-KV attention must not append");
    CHECK(ctx.gqa_prefill_attention_cached_from(cache, 1, prefix + 1, qt.unwrap(), spec).is_err(), "a source layer shorter than position + rows must be refused");
    CHECK(ctx.gqa_prefill_attention_cached_from(cache, 7, prefix, qt.unwrap(), spec).is_err(), "a source layer outside the cache must be refused");
}

// MlaPrefillBackend::mla_prefill_attention: two chunks, each appended and attended causally; bf16 rows for a chunk
static void test_mla_prefill(const RocmContext& ctx)
{
    std::mt19937 rng(31);
    MlaSpec spec;
    spec.kv_lora_rank = 512;
    spec.qk_rope_head_dim = 64;
    spec.num_heads = 16;
    spec.q_projection_size = spec.num_heads * 192;
    spec.kv_projection_size = spec.num_heads * 256;
    spec.q_lora_rank = 1536;
    const size_t block = 64, layer = 0;
    auto cache_r = RocmKvCache::new_mla(1, 512, 64, block, 1024);
    CHECK(cache_r.is_ok(), "cache");
    if (cache_r.is_err()) {
        return;
    }
    RocmKvCache cache = cache_r.unwrap();
    std::vector<float> kv_b = randn(rng, spec.kv_projection_size * 512, true);
    for (auto& w : kv_b) {
        w = zo_bf16_to_f32(zo_f32_to_bf16(w * 0.05f));
    }
    auto weight = ctx.prepare_mla_kv_b(kv_b, spec.kv_projection_size, 512);
    std::vector<float> all_latent, all_rope;
    size_t position = 0;
    const size_t chunks[] = {90, 37, 1};
    for (size_t rows : chunks) {
        const auto q = randn(rng, rows * spec.q_projection_size, true);
        const auto latent = randn(rng, rows * 512, false);
        const auto rope = randn(rng, rows * 64, false);
        auto out = ctx.mla_prefill_attention(ctx.tensor_from_f32(q, rows, spec.q_projection_size, DType::BF16).unwrap(),
                                             ctx.tensor_from_f32(latent, rows, 512).unwrap(), ctx.tensor_from_f32(rope, rows, 64).unwrap(), weight.unwrap(),
                                             &cache, layer, spec);
        CHECK(out.is_ok(), "mla_prefill_attention rows=%zu: %s", rows, out.is_err() ? out.unwrap_err().to_string().c_str() : "");
        if (out.is_err()) {
            return;
        }
        CHECK(out.unwrap().dtype == (rows > 1 ? DType::BF16 : DType::F32), "a chunk comes back as bf16, one row as f32");
        all_latent.insert(all_latent.end(), latent.begin(), latent.end());
        all_rope.insert(all_rope.end(), rope.begin(), rope.end());
        const size_t total = position + rows;
        std::vector<int8_t> codes(total * 512);
        std::vector<uint16_t> scales(total * 8), rope_bits(total * 64), q_bits(q.size());
        zo_q8g64_append_paged(0, all_latent.data(), codes.data(), scales.data(), nullptr, 0, total, 512, 64, block, 0);
        zo_half_append_paged(0, all_rope.data(), rope_bits.data(), nullptr, 0, total, 64, block, 0);
        for (size_t i = 0; i < q.size(); ++i) {
            q_bits[i] = zo_f32_to_bf16(q[i]);
        }
        zo_mla_spec zs = {512, 64, spec.q_projection_size, spec.kv_projection_size, spec.num_heads};
        std::vector<float> want(rows * spec.num_heads * spec.value_dim());
        const int rc = zo_mla_absorbed_q8_history(&zs, q_bits.data(), rows, position, (const uint8_t*)codes.data(), scales.data(), 64, rope_bits.data(),
                                                  total, kv_b.data(), nullptr, 0, nullptr, want.data(), nullptr);
        CHECK(rc == 0, "oracle rc %d", rc);
        auto got = ctx.tensor_to_f32(out.unwrap()).unwrap();
        if (rows > 1) { // bf16 rows: within one bf16 step of the oracle's unrounded value, then the attention bound
            double worst = 0;
            for (size_t i = 0; i < got.size(); ++i) {
                worst = fmax(worst, fabs((double)got[i] - want[i]) - fabs((double)want[i]) * 0.0078125);
            }
            printf("%-58s worst excess over a bf16 step %.3e\n", "mla_prefill_attention chunk (bf16 rows)", worst);
            CHECK(worst <= 2e-3, "mla_prefill_attention rows=%zu: %.3e beyond a bf16 step", rows, worst);
        } else {
            compare(got, want, "mla_prefill_attention, one row");
        }
        position = total;
        CHECK(cache.len(layer) == position, "cache length %zu vs %zu", cache.len(layer), position);
    }
    CHECK(ctx.mla_prefill_attention(ctx.tensor_from_f32(std::vector<float>(spec.q_projection_size), 1, spec.q_projection_size).unwrap(),
                                    ctx.tensor_from_f32(std::vector<float>(512), 1, 512).unwrap(), ctx.tensor_from_f32(std::vector<float>(64), 1, 64).unwrap(),
                                    weight.unwrap(), nullptr, layer, spec)
              .is_err(),
          "a prefill without a cache must be refused");
}

// Backend::gqa_prefill_attention{,_visible}: a chunk over its own dense K/V, compared with the oracle on the f32 K/V the
// reference's device path reads (src/backend/rocm/attention.rs:2151-2199) -- the f16 planes in between must stay inside the bound
static void test_gqa_uncached(const RocmContext& ctx)
{
    std::mt19937 rng(41);
    struct Case {
        size_t heads, kv_heads, dim, rows;
        CausalWindow window;
        DType q_dtype;
    };
    const Case cases[] = {{16, 4, 128, 300, CausalWindow::Full(), DType::BF16},
                          {8, 2, 128, 777, CausalWindow::Sliding(200), DType::F32},
                          {8, 4, 256, 130, CausalWindow::Full(), DType::BF16},
                          {4, 1, 128, 1, CausalWindow::Full(), DType::F32}};
    for (const Case& c : cases) {
        GqaSpec spec;
        spec.num_heads = c.heads;
        spec.num_kv_heads = c.kv_heads;
        spec.head_dim = c.dim;
        spec.window = c.window;
        spec.score_scale = 1.0f / sqrtf((float)c.dim);
        const size_t q_cols = c.heads * c.dim, kv_cols = c.kv_heads * c.dim;
        const auto q = randn(rng, c.rows * q_cols, c.q_dtype == DType::BF16);
        const auto k = randn(rng, c.rows * kv_cols, false);
        const auto v = randn(rng, c.rows * kv_cols, false);
        auto qt = ctx.tensor_from_f32(q, c.rows, q_cols, c.q_dtype);
        auto kt = ctx.tensor_from_f32(k, c.rows, kv_cols);
        auto vt = ctx.tensor_from_f32(v, c.rows, kv_cols);
        auto out = ctx.gqa_prefill_attention(qt.unwrap(), kt.unwrap(), vt.unwrap(), spec);
        CHECK(out.is_ok(), "gqa_prefill_attention: %s", out.is_err() ? out.unwrap_err().to_string().c_str() : "");
        std::vector<float> want(c.rows * q_cols);
        int rc = zo_gqa_prefill_at_visible_f32(q.data(), k.data(), v.data(), c.rows, 0, c.rows, 0, c.heads, c.kv_heads, c.dim,
                                               c.window.sliding ? c.window.size : 0, spec.score_scale, 0.0f, nullptr, want.data());
        CHECK(rc == 0, "oracle rc %d", rc);
        char what[128];
        snprintf(what, sizeof(what), "gqa_prefill_attention %zux%zu d=%zu rows=%zu%s", c.heads, c.kv_heads, c.dim, c.rows, c.window.sliding ? " sliding" : "");
        if (out.is_ok()) {
            compare(ctx.tensor_to_f32(out.unwrap()).unwrap(), want, what);
        }
        // right-padded text: the rows of the first 100 tokens (or all) see to the end of that stretch
        std::vector<uint32_t> ends(c.rows);
        const size_t text = std::min<size_t>(c.rows, 100);
        for (size_t r = 0; r < c.rows; ++r) {
            ends[r] = (uint32_t)(r < text ? text : r + 1);
        }
        auto seen = ctx.gqa_prefill_attention_visible(qt.unwrap(), kt.unwrap(), vt.unwrap(), spec, ends);
        CHECK(seen.is_ok(), "gqa_prefill_attention_visible: %s", seen.is_err() ? seen.unwrap_err().to_string().c_str() : "");
        rc = zo_gqa_prefill_at_visible_f32(q.data(), k.data(), v.data(), c.rows, 0, c.rows, 0, c.heads, c.kv_heads, c.dim,
                                           c.window.sliding ? c.window.size : 0, spec.score_scale, 0.0f, ends.data(), want.data());
        CHECK(rc == 0, "oracle rc %d", rc);
        snprintf(what, sizeof(what), "gqa_prefill_attention_visible %zux%zu d=%zu rows=%zu", c.heads, c.kv_heads, c.dim, c.rows);
        if (seen.is_ok()) {
            compare(ctx.tensor_to_f32(seen.unwrap()).unwrap(), want, what);
        }
        ends.pop_back();
        CHECK(ctx.gqa_prefill_attention_visible(qt.unwrap(), kt.unwrap(), vt.unwrap(), spec, ends).is_err(), "one visible end too few must be refused");
        CHECK(ctx.gqa_prefill_attention(qt.unwrap(), qt.unwrap(), vt.unwrap(), spec).is_err() || c.heads == c.kv_heads, "a K of the wrong width must be refused");
    }
}

// BlockAttentionBackend: the reference's own vectors (src/attention/block.rs:125-141), varlen segments, free ranges, the
// prefix + suffix form, and the offsets and ranges BlockAttentionSpec refuses
static void test_block_attention(const RocmContext& ctx)
{
    const size_t d = 128;
    const GqaGeometry one{1, 1, d};
    {
        // zero queries: every row is the mean of the values it sees
        const float values5[] = {2, 4, 6, 20, 40}, values3[] = {2, 6, 10};
        auto varlen = BlockAttentionSpec::varlen(one, 3, 5, {0, 2, 3}, {0, 3, 5}, 1.0f);
        CHECK(varlen.is_ok(), "varlen offsets of the reference's test");
        BlockAttentionSpec free_ranges;
        free_ranges.geometry = one;
        free_ranges.score_scale = 1.0f;
        free_ranges.visible = {{0, 2}, {1, 3}};
        struct Vec {
            const float* values;
            size_t kv_rows, q_rows;
            const BlockAttentionSpec* spec;
            float want[3];
        } vectors[] = {{values5, 5, 3, &varlen.unwrap(), {4, 4, 30}}, {values3, 3, 2, &free_ranges, {4, 8, 0}}};
        for (const Vec& vec : vectors) {
            std::vector<float> v(vec.kv_rows * d, 0.0f), zeros_kv(vec.kv_rows * d, 0.0f), zeros_q(vec.q_rows * d, 0.0f);
            for (size_t r = 0; r < vec.kv_rows; ++r) {
                v[r * d] = vec.values[r];
            }
            auto out = ctx.block_attention(ctx.tensor_from_f32(zeros_q, vec.q_rows, d).unwrap(), ctx.tensor_from_f32(zeros_kv, vec.kv_rows, d).unwrap(),
                                           ctx.tensor_from_f32(v, vec.kv_rows, d).unwrap(), *vec.spec);
            CHECK(out.is_ok(), "block_attention vector: %s", out.is_err() ? out.unwrap_err().to_string().c_str() : "");
            if (out.is_ok()) {
                const auto got = ctx.tensor_to_f32(out.unwrap()).unwrap();
                for (size_t r = 0; r < vec.q_rows; ++r) {
                    CHECK(fabsf(got[r * d] - vec.want[r]) <= 2e-3f * vec.want[r], "block vector row %zu: %g, the reference holds %g", r, got[r * d], vec.want[r]);
                    CHECK(got[r * d + 1] == 0.0f, "block vector row %zu column 1: %g", r, got[r * d + 1]);
                }
            }
        }
        // the offsets the reference's test refuses
        const std::vector<size_t> bad[][2] = {{{0, 2}, {0, 5}}, {{0, 0, 3}, {0, 3, 5}}, {{1, 2, 3}, {0, 3, 5}},
                                              {{0, 4, 3}, {0, 3, 5}}, {{0, 2, 3}, {0, 5}}, {{0, 2, 3}, {0, 5, 5}}};
        for (const auto& pair : bad) {
            CHECK(BlockAttentionSpec::varlen(one, 3, 5, pair[0], pair[1], 1.0f).is_err(), "varlen offsets that must be refused");
        }
    }
    std::mt19937 rng(43);
    const GqaGeometry geometry{8, 2, 128};
    const size_t q_cols = 8 * 128, kv_cols = 2 * 128;
    const float scale = 1.0f / sqrtf(128.0f);
    // isolated sequences packed into one call, query and KV segments of different lengths
    {
        const std::vector<size_t> q_off = {0, 1, 40, 340, 357}, kv_off = {0, 700, 733, 1500, 1501};
        const size_t q_rows = q_off.back(), kv_rows = kv_off.back();
        auto spec = BlockAttentionSpec::varlen(geometry, q_rows, kv_rows, q_off, kv_off, scale);
        CHECK(spec.is_ok(), "varlen spec");
        const auto q = randn(rng, q_rows * q_cols, true);
        const auto k = randn(rng, kv_rows * kv_cols, false);
        const auto v = randn(rng, kv_rows * kv_cols, false);
        std::vector<uint32_t> flat;
        for (const auto& range : spec.unwrap().visible) {
            flat.push_back((uint32_t)range.first);
            flat.push_back((uint32_t)range.second);
        }
        std::vector<float> want(q_rows * q_cols);
        const int rc = zo_block_attention_f32(q.data(), k.data(), v.data(), q_rows, kv_rows, 8, 2, 128, scale, flat.data(), want.data());
        CHECK(rc == 0, "oracle rc %d", rc);
        auto qt = ctx.tensor_from_f32(q, q_rows, q_cols, DType::BF16);
        auto out = ctx.block_attention(qt.unwrap(), ctx.tensor_from_f32(k, kv_rows, kv_cols).unwrap(), ctx.tensor_from_f32(v, kv_rows, kv_cols).unwrap(),
                                       spec.unwrap());
        CHECK(out.is_ok(), "block_attention varlen: %s", out.is_err() ? out.unwrap_err().to_string().c_str() : "");
        if (out.is_ok()) {
            compare(ctx.tensor_to_f32(out.unwrap()).unwrap(), want, "block_attention, varlen segments 357 x 1501");
        }
        // the same K/V handed over as a resident prefix and a short suffix
        const size_t cut = 1437;
        std::vector<float> k_head(k.begin(), k.begin() + cut * kv_cols), k_tail(k.begin() + cut * kv_cols, k.end());
        std::vector<float> v_head(v.begin(), v.begin() + cut * kv_cols), v_tail(v.begin() + cut * kv_cols, v.end());
        auto split = ctx.block_attention_prefix_suffix(qt.unwrap(), ctx.tensor_from_f32(k_head, cut, kv_cols, DType::BF16).unwrap(),
                                                       ctx.tensor_from_f32(v_head, cut, kv_cols, DType::BF16).unwrap(),
                                                       ctx.tensor_from_f32(k_tail, kv_rows - cut, kv_cols).unwrap(),
                                                       ctx.tensor_from_f32(v_tail, kv_rows - cut, kv_cols).unwrap(), spec.unwrap());
        CHECK(split.is_ok(), "block_attention_prefix_suffix: %s", split.is_err() ? split.unwrap_err().to_string().c_str() : "");
        {
            // the same rows as three segments, the middle one a single row
            auto kt = ctx.tensor_from_f32(k_head, cut, kv_cols, DType::BF16).unwrap(), vt = ctx.tensor_from_f32(v_head, cut, kv_cols, DType::BF16).unwrap();
            std::vector<float> k_one(k_tail.begin(), k_tail.begin() + kv_cols), v_one(v_tail.begin(), v_tail.begin() + kv_cols);
            std::vector<float> k_rest(k_tail.begin() + kv_cols, k_tail.end()), v_rest(v_tail.begin() + kv_cols, v_tail.end());
            auto k1 = ctx.tensor_from_f32(k_one, 1, kv_cols).unwrap(), v1 = ctx.tensor_from_f32(v_one, 1, kv_cols).unwrap();
            auto k2 = ctx.tensor_from_f32(k_rest, kv_rows - cut - 1, kv_cols).unwrap(), v2 = ctx.tensor_from_f32(v_rest, kv_rows - cut - 1, kv_cols).unwrap();
            auto three = ctx.block_attention_segments(qt.unwrap(), {&kt, &k1, &k2}, {&vt, &v1, &v2}, spec.unwrap());
            CHECK(three.is_ok(), "block_attention_segments: %s", three.is_err() ? three.unwrap_err().to_string().c_str() : "");
            if (three.is_ok() && split.is_ok()) {
                CHECK(ctx.tensor_to_f32(three.unwrap()).unwrap() == ctx.tensor_to_f32(split.unwrap()).unwrap(), "three segments must give the bits of two");
            }
            CHECK(ctx.block_attention_segments(qt.unwrap(), {&kt, &k1}, {&vt}, spec.unwrap()).is_err(), "unequal K / V segment counts must be refused");
        }
        if (split.is_ok()) {
            // the prefix arrives as bf16 here (a cache kept in bf16): the oracle reads what the planes hold
            std::vector<float> k_seen = k, v_seen = v;
            for (size_t i = 0; i < cut * kv_cols; ++i) {
                k_seen[i] = zo_bf16_to_f32(zo_f32_to_bf16(k[i]));
                v_seen[i] = zo_bf16_to_f32(zo_f32_to_bf16(v[i]));
            }
            const int rc2 = zo_block_attention_f32(q.data(), k_seen.data(), v_seen.data(), q_rows, kv_rows, 8, 2, 128, scale, flat.data(), want.data());
            CHECK(rc2 == 0, "oracle rc %d", rc2);
            compare(ctx.tensor_to_f32(split.unwrap()).unwrap(), want, "block_attention_prefix_suffix, bf16 prefix 1437 + f32 suffix 64");
        }
    }
    // free ranges (not monotone, not causal), one-key rows, more query rows than KV rows
    {
        const size_t q_rows = 200, kv_rows = 90;
        BlockAttentionSpec spec;
        spec.geometry = geometry;
        spec.score_scale = scale;
        std::vector<uint32_t> flat;
        for (size_t r = 0; r < q_rows; ++r) {
            const size_t start = rng() % kv_rows;
            const size_t end = r % 7 == 0 ? start + 1 : start + 1 + rng() % (kv_rows - start);
            spec.visible.emplace_back(start, end);
            flat.push_back((uint32_t)start);
            flat.push_back((uint32_t)end);
        }
        const auto q = randn(rng, q_rows * q_cols, false);
        const auto k = randn(rng, kv_rows * kv_cols, false);
        const auto v = randn(rng, kv_rows * kv_cols, false);
        std::vector<float> want(q_rows * q_cols);
        const int rc = zo_block_attention_f32(q.data(), k.data(), v.data(), q_rows, kv_rows, 8, 2, 128, scale, flat.data(), want.data());
        CHECK(rc == 0, "oracle rc %d", rc);
        auto out = ctx.block_attention(ctx.tensor_from_f32(q, q_rows, q_cols).unwrap(), ctx.tensor_from_f32(k, kv_rows, kv_cols).unwrap(),
                                       ctx.tensor_from_f32(v, kv_rows, kv_cols).unwrap(), spec);
        CHECK(out.is_ok(), "block_attention free ranges: %s", out.is_err() ? out.unwrap_err().to_string().c_str() : "");
        if (out.is_ok()) {
            compare(ctx.tensor_to_f32(out.unwrap()).unwrap(), want, "block_attention, free ranges, 200 rows over 90 keys");
        }
        auto qt = ctx.tensor_from_f32(q, q_rows, q_cols).unwrap(), kt = ctx.tensor_from_f32(k, kv_rows, kv_cols).unwrap();
        BlockAttentionSpec bad = spec;
        bad.visible[5] = {7, 7};
        CHECK(ctx.block_attention(qt, kt, kt, bad).is_err(), "an empty range must be refused");
        bad.visible[5] = {7, kv_rows + 1};
        CHECK(ctx.block_attention(qt, kt, kt, bad).is_err(), "a range past the KV rows must be refused");
        bad = spec;
        bad.visible.pop_back();
        CHECK(ctx.block_attention(qt, kt, kt, bad).is_err(), "one range too few must be refused");
        bad = spec;
        bad.score_scale = 0.0f;
        CHECK(ctx.block_attention(qt, kt, kt, bad).is_err(), "a score scale of zero must be refused");
        CHECK(ctx.block_attention(qt, qt, kt, spec).is_err(), "a K of the wrong width must be refused");
    }
}

// A decode loop in steady state: after the first steps the context neither allocates device memory, nor uploads rotary
// tables again, nor waits for its stream -- outputs come from the pool, tables stay resident, small arrays ride the pinned ring
static void test_steady_state_counters(const RocmContext& ctx)
{
    std::mt19937 rng(47);
    MlaSpec spec;
    spec.kv_lora_rank = 512;
    spec.qk_rope_head_dim = 64;
    spec.num_heads = 16;
    spec.q_projection_size = spec.num_heads * 192;
    spec.kv_projection_size = spec.num_heads * 256;
    spec.q_lora_rank = 1536;
    const size_t half = 32, table_rows = 4096;
    std::vector<float> cos(table_rows * half), sin(table_rows * half);
    for (size_t pos = 0; pos < table_rows; ++pos) {
        for (size_t i = 0; i < half; ++i) {
            const float angle = (float)pos * powf(10000.0f, -2.0f * (float)i / 64.0f);
            cos[pos * half + i] = cosf(angle);
            sin[pos * half + i] = sinf(angle);
        }
    }
    auto cache_r = RocmKvCache::new_mla(1, 512, 64, 64, 2048, TablePolicy::Scrambled);
    CHECK(cache_r.is_ok(), "cache");
    RocmKvCache cache = cache_r.unwrap();
    std::vector<float> kv_b = randn(rng, spec.kv_projection_size * 512, true);
    auto weight = ctx.prepare_mla_kv_b(kv_b, spec.kv_projection_size, 512);
    auto latent = ctx.tensor_from_f32(randn(rng, 512, false), 1, 512);
    auto rope = ctx.tensor_from_f32(randn(rng, 64, false), 1, 64);
    auto query = ctx.tensor_from_f32(randn(rng, spec.q_projection_size, true), 1, spec.q_projection_size, DType::BF16);
    GqaSpec gqa;
    gqa.num_heads = 8;
    gqa.num_kv_heads = 2;
    gqa.head_dim = 128;
    gqa.score_scale = 1.0f / sqrtf(128.0f);
    auto gqa_cache_r = RocmKvCache::new_gqa(1, 2, 128, 16, 2048, TablePolicy::Scrambled);
    CHECK(gqa_cache_r.is_ok(), "cache");
    RocmKvCache gqa_cache = gqa_cache_r.unwrap();
    auto gq = ctx.tensor_from_f32(randn(rng, 8 * 128, true), 1, 8 * 128, DType::BF16);
    auto gk = ctx.tensor_from_f32(randn(rng, 2 * 128, false), 1, 2 * 128);
    HostCounters settled;
    const size_t steps = 150, warm = 20;
    for (size_t step = 0; step < steps; ++step) {
        if (step == warm) {
            settled = ctx.counters();
        }
        auto appended = ctx.append_mla_rope(cache, 0, latent.unwrap(), rope.unwrap(), 64, RotaryLayout::SplitHalf, step, cos, sin);
        CHECK(appended.is_ok(), "append_mla_rope step %zu: %s", step, appended.is_err() ? appended.unwrap_err().to_string().c_str() : "");
        auto out = ctx.mla_decode_attention(query.unwrap(), cache, weight.unwrap(), 0, step, spec);
        CHECK(out.is_ok(), "mla_decode_attention step %zu", step);
        const std::vector<uint32_t> ends = {(uint32_t)(step + 1)};
        auto gout = ctx.gqa_prefill_attention_cached_visible(gqa_cache, 0, step, gq.unwrap(), gk.unwrap(), gk.unwrap(), gqa, ends, true);
        CHECK(gout.is_ok(), "gqa decode step %zu: %s", step, gout.is_err() ? gout.unwrap_err().to_string().c_str() : "");
    }
    const HostCounters after = ctx.counters();
    printf("steady state over %zu steps: allocations %zu -> %zu, rope uploads %zu -> %zu, stream waits %zu -> %zu, staged uploads %zu -> %zu\n",
           steps - warm, settled.device_allocations, after.device_allocations, settled.rope_table_uploads, after.rope_table_uploads,
           settled.stream_waits, after.stream_waits, settled.staged_uploads, after.staged_uploads);
    CHECK(after.device_allocations == settled.device_allocations, "a decode loop in steady state must not allocate device memory");
    // the first call committed 16,384 elements, 512 positions of 32: nothing more to send for positions 20..149
    CHECK(after.rope_table_uploads == settled.rope_table_uploads && settled.rope_table_uploads >= 1, "rotary tables must stay resident: %zu uploads",
          after.rope_table_uploads - settled.rope_table_uploads);
    // 130 steps of two metadata records each: the 256-record ring wraps once
    CHECK(after.stream_waits - settled.stream_waits <= 1, "a decode loop in steady state must not wait for its stream: %zu waits",
          after.stream_waits - settled.stream_waits);
    CHECK(after.staged_uploads - settled.staged_uploads == steps - warm, "visible ends must travel through the pinned ring");
    CHECK(ctx.synchronize().is_ok(), "synchronize");
}

// MLA at another latent / rope width with kv_b as W8A16 and W4A16 codes (RocmQuantizedWeight, src/backend/rocm/attention.rs:181-192):
// the oracle gets the f32 values the codes stand for
static void test_mla_other_widths_and_quantized_weights(const RocmContext& ctx)
{
    std::mt19937 rng(53);
    struct Case {
        size_t latent, rope, nope, value, heads, rows;
        unsigned bits;
        size_t group;
    };
    const Case cases[] = {{128, 32, 64, 64, 6, 300, 8, 64}, {512, 64, 128, 128, 16, 700, 8, 128}, {512, 64, 128, 128, 8, 200, 4, 32}, {256, 128, 32, 96, 3, 90, 16, 0}};
    for (const Case& c : cases) {
        MlaSpec spec;
        spec.kv_lora_rank = c.latent;
        spec.qk_rope_head_dim = c.rope;
        spec.num_heads = c.heads;
        spec.q_projection_size = c.heads * (c.nope + c.rope);
        spec.kv_projection_size = c.heads * (c.nope + c.value);
        spec.q_lora_rank = 64;
        CHECK(!spec.validate().has_value(), "spec must validate");
        auto cache_r = RocmKvCache::new_mla(1, c.latent, c.rope, 16, 1024, TablePolicy::Scrambled);
        CHECK(cache_r.is_ok(), "cache: %s", cache_r.is_err() ? cache_r.unwrap_err().to_string().c_str() : "");
        if (cache_r.is_err()) {
            return;
        }
        RocmKvCache cache = cache_r.unwrap();
        const auto latent = randn(rng, c.rows * c.latent, false);
        const auto rope = randn(rng, c.rows * c.rope, false);
        auto appended = ctx.append_mla(cache, 0, ctx.tensor_from_f32(latent, c.rows, c.latent).unwrap(), ctx.tensor_from_f32(rope, c.rows, c.rope).unwrap());
        CHECK(appended.is_ok(), "append_mla: %s", appended.is_err() ? appended.unwrap_err().to_string().c_str() : "");
        std::vector<float> kv_b = randn(rng, spec.kv_projection_size * c.latent, true);
        for (auto& w : kv_b) {
            w = zo_bf16_to_f32(zo_f32_to_bf16(w * 0.05f));
        }
        auto weight = c.bits == 16 ? ctx.prepare_mla_kv_b(kv_b, spec.kv_projection_size, c.latent)
                                   : ctx.prepare_mla_kv_b_quantized(kv_b, spec.kv_projection_size, c.latent, c.bits, c.group);
        CHECK(weight.is_ok(), "weight: %s", weight.is_err() ? weight.unwrap_err().to_string().c_str() : "");
        if (weight.is_err()) {
            return;
        }
        std::vector<float> seen = kv_b;
        if (c.bits != 16) {
            auto values = ctx.dequantized_kv_b(weight.unwrap());
            CHECK(values.is_ok(), "dequantized_kv_b");
            seen = values.unwrap();
            double worst = 0;
            for (size_t i = 0; i < seen.size(); ++i) {
                worst = fmax(worst, fabs((double)seen[i] - kv_b[i]));
            }
            CHECK(worst < (c.bits == 8 ? 2e-3 : 3e-2), "the codes are %.3e from the weights", worst);
        }
        const auto q = randn(rng, spec.q_projection_size, true);
        auto out = ctx.mla_decode_attention(ctx.tensor_from_f32(q, 1, spec.q_projection_size, DType::BF16).unwrap(), cache, weight.unwrap(), 0,
                                            c.rows - 1, spec);
        CHECK(out.is_ok(), "mla_decode_attention: %s", out.is_err() ? out.unwrap_err().to_string().c_str() : "");
        if (out.is_err()) {
            return;
        }
        std::vector<int8_t> codes(c.rows * c.latent);
        std::vector<uint16_t> scales(c.rows * c.latent / 64), rope_bits(c.rows * c.rope), q_bits(q.size());
        zo_q8g64_append_paged(0, latent.data(), codes.data(), scales.data(), nullptr, 0, c.rows, c.latent, 64, 16, 0);
        zo_half_append_paged(0, rope.data(), rope_bits.data(), nullptr, 0, c.rows, c.rope, 16, 0);
        for (size_t i = 0; i < q.size(); ++i) {
            q_bits[i] = zo_f32_to_bf16(q[i]);
        }
        zo_mla_spec zs = {c.latent, c.rope, spec.q_projection_size, spec.kv_projection_size, c.heads};
        std::vector<float> want(c.heads * c.value);
        const int rc = zo_mla_absorbed_q8_history(&zs, q_bits.data(), 1, c.rows - 1, (const uint8_t*)codes.data(), scales.data(), 64, rope_bits.data(),
                                                  c.rows, seen.data(), nullptr, 0, nullptr, want.data(), nullptr);
        CHECK(rc == 0, "oracle rc %d", rc);
        char what[128];
        snprintf(what, sizeof(what), "mla_decode_attention latent=%zu rope=%zu kv_b %u-bit", c.latent, c.rope, c.bits);
        compare(ctx.tensor_to_f32(out.unwrap()).unwrap(), want, what);
    }
    CHECK(ctx.prepare_mla_kv_b_quantized(std::vector<float>(64 * 128), 64, 128, 8, 48).is_err(), "a group that does not divide the columns must be refused");
    CHECK(ctx.prepare_mla_kv_b_quantized(std::vector<float>(64 * 128), 64, 128, 5, 64).is_err(), "five-bit codes must be refused");
}

int main()
{
    auto ctx = RocmContext::create(0);
    if (ctx.is_err()) {
        printf("FAIL context: %s\n", ctx.unwrap_err().to_string().c_str());
        return 2;
    }
    // CausalWindow known answers of the reference's tests (src/attention/gqa.rs:290-330)
    CHECK(CausalWindow::Full().key_range(5, 10) == std::make_pair((size_t)0, (size_t)6), "full window");
    CHECK(CausalWindow::Sliding(4).key_range(9, 10) == std::make_pair((size_t)6, (size_t)10), "sliding window");
    CHECK(CausalWindow::Sliding(4).key_range(1, 10) == std::make_pair((size_t)0, (size_t)2), "sliding window, short history");
    CHECK(CausalWindow::Sliding(1024).cache_capacity(8192) == 1024 && CausalWindow::Full().cache_capacity(8192) == 8192, "cache capacity");
    test_growth_rule();
    test_gqa(ctx.unwrap(), CausalWindow::Full(), "full", TablePolicy::Scrambled);
    test_gqa(ctx.unwrap(), CausalWindow::Sliding(128), "sliding(128)", TablePolicy::Scrambled);
    test_gqa(ctx.unwrap(), CausalWindow::Full(), "full, growing planes", TablePolicy::Identity);
    test_gqa_ring(ctx.unwrap());
    test_gqa_shared_and_visible(ctx.unwrap());
    test_mla(ctx.unwrap());
    test_mla_prefill(ctx.unwrap());
    test_gqa_uncached(ctx.unwrap());
    test_block_attention(ctx.unwrap());
    test_mla_other_widths_and_quantized_weights(ctx.unwrap());
    test_steady_state_counters(ctx.unwrap());
    printf(failures == 0 ? "ALL PASSED\n" : "%d FAILED\n", failures);
    return failures == 0 ? 0 : 1;
}

// C ABI of the attention hot path: argument validation, workspace carving, launches.
// Nothing here allocates, frees or synchronises.
#include "../../include/zllm_attn.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>

#include "kernels.hpp"

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char* format, ...)
{
    va_list args;
    va_start(args, format);
    vsnprintf(g_error, sizeof(g_error), format, args);
    va_end(args);
    return code;
}

int hip_status(hipError_t err, const char* what)
{
    if (err == hipSuccess) {
        return 0;
    }
    snprintf(g_error, sizeof(g_error), "%s: %s", what, hipGetErrorString(err));
    return (int)err;
}

// Compute units of the current device, asked once per device; 256 (MI355X) where there is no device to ask, so that the
// host-only planning calls still answer.
unsigned int compute_units()
{
    constexpr int kKnown = 64;
    static std::atomic<unsigned int> known[kKnown];
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kKnown) {
        (void)hipGetLastError();
        return 256u;
    }
    unsigned int units = known[device].load(std::memory_order_relaxed);
    if (units == 0u) {
        int count = 0;
        if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0) {
            (void)hipGetLastError();
            return 256u;
        }
        units = (unsigned int)count;
        known[device].store(units, std::memory_order_relaxed);
    }
    return units;
}

} // namespace

// Split records of zllm_attn_gqa_decode_static: one copy of this array lives on every GPU the library's code object
// is loaded on, from load to process end.  In host code the name below is only a handle for hipGetSymbolAddress --
// it is never passed to a kernel or a memory call; the device address found for each GPU is.
constexpr uint64_t kStaticScratchBytes = 16ull << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_of_device[kMaxDevices];

// Device address of `scratch` on `device`, which must be the current device.  Looked up once per device; two threads
// racing through the first call find the same address.
int resolve_static_scratch(int device, void** base)
{
    if (device < 0 || device >= kMaxDevices) {
        return fail(-1, "static scratch: device index %d out of range", device);
    }
    void* known = g_scratch_of_device[device].load(std::memory_order_acquire);
    if (known == nullptr) {
        void* found = nullptr;
        const hipError_t err = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
        if (err != hipSuccess) {
            return hip_status(err, "hipGetSymbolAddress(scratch)");
        }
        if (found == nullptr) {
            return fail(-1, "static scratch: no device address on device %d", device);
        }
        g_scratch_of_device[device].store(found, std::memory_order_release);
        known = found;
    }
    *base = known;
    return 0;
}

int static_scratch_of_current_device(void** base)
{
    int device = -1;
    const hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) {
        return hip_status(err, "hipGetDevice");
    }
    return resolve_static_scratch(device, base);
}

unsigned int shift_of(unsigned int block_tokens)
{
    unsigned int shift = 0;
    while ((1u << shift) < block_tokens) {
        ++shift;
    }
    return shift;
}

uint64_t align_up(uint64_t value, uint64_t to)
{
    return (value + to - 1) / to * to;
}

// head dimensions that Q8g64 groups divide, up to the reference's limit of 256 (tensor/attention.rs:1022)
bool valid_head_dim(uint32_t d)
{
    return d == 64 || d == 128 || d == 192 || d == 256;
}

// Tokens per KV split.  `units` (sequence, head-block) pairs each cut their keys into the same number of splits, one
// workgroup per split, and the launch runs in rounds of one workgroup per CU: workgroups beyond the last full round run
// alone while the other CUs idle, which is what a split count that is merely rounded up costs a batch that does not
// divide the CU count.  So the candidates are the split counts that fill 1, 2, ... 8 rounds, each priced as
// rounds x (tokens of a split + what a workgroup's prologue and epilogue cost, about two 32-token steps), and the
// cheapest is taken, the fewest rounds among equals.  `min_chunk` keeps the partial records and their merge a few
// percent of the KV bytes a split reads.
void plan_splits(uint32_t max_len, uint64_t units, uint32_t units_per_group, uint32_t min_chunk, uint32_t* chunk_tokens, uint32_t* max_chunks)
{
    // `units_per_group` of a pair's splits share one workgroup (GQA decode with few KV heads)
    constexpr uint64_t kFixedTokens = 64;
    const uint64_t cus = compute_units();
    uint64_t best_chunk = align_up(max_len < min_chunk ? min_chunk : max_len, 32); // one split per pair
    uint64_t best_cost = ~(uint64_t)0;
    for (uint64_t rounds = 1; rounds <= 8; ++rounds) {
        const uint64_t per_unit = rounds * cus * units_per_group / units;
        if (per_unit == 0) {
            continue;
        }
        uint64_t chunk = ((uint64_t)max_len + per_unit - 1) / per_unit;
        chunk = align_up(chunk < min_chunk ? min_chunk : chunk, 32);
        const uint64_t splits = ((uint64_t)max_len + chunk - 1) / chunk;
        const uint64_t groups = (splits * units + units_per_group - 1) / units_per_group;
        const uint64_t launched = (groups + cus - 1) / cus;
        const uint64_t cost = launched * (chunk + kFixedTokens);
        if (cost < best_cost) {
            best_cost = cost;
            best_chunk = chunk;
        }
    }
    *chunk_tokens = (uint32_t)best_chunk;
    const uint64_t chunks = ((uint64_t)max_len + best_chunk - 1) / best_chunk;
    *max_chunks = (uint32_t)(chunks == 0 ? 1 : chunks);
}

// Token positions are 32-bit in the kernels, which also round them up to steps and splits: lengths stay below 2^31.
constexpr uint32_t kMaxTokens = 0x7fffff00u;

int validate_gqa_decode(const zllm_gqa_decode_args* a)
{
    if (a == nullptr) {
        return fail(-1, "GQA decode: null args");
    }
    // shape rules of try_gqa_decode_cached_f32 (tensor/attention.rs:1022-1024)
    if (a->batch == 0 || a->num_heads == 0 || a->num_kv_heads == 0 || a->num_heads % a->num_kv_heads != 0 ||
        !valid_head_dim(a->head_dim)) {
        return fail(-1, "GQA decode: invalid shape batch=%u heads=%u/%u dim=%u", a->batch, a->num_heads, a->num_kv_heads, a->head_dim);
    }
    // the split merge indexes the rows of the call (sequences, or the rows of a prefill chunk that runs as decode items) with
    // the grid's second dimension
    if (a->batch > 65535u) {
        return fail(-1, "GQA decode: batch=%u exceeds 65535 rows per call", a->batch);
    }
    if (a->block_tokens == 0 || a->max_kv_len == 0 || a->max_kv_len > kMaxTokens) {
        return fail(-1, "GQA decode: block_tokens=%u max_kv_len=%u must be non-zero, max_kv_len below 2^31", a->block_tokens, a->max_kv_len);
    }
    if (!isfinite(a->score_scale) || a->score_scale <= 0.0f || !(a->softcap >= 0.0f) || !isfinite(a->softcap)) {
        return fail(-1, "GQA decode: invalid score_scale=%g softcap=%g", (double)a->score_scale, (double)a->softcap);
    }
    if (a->kv_format != ZLLM_KV_Q8G64 && a->kv_format != ZLLM_KV_F16) {
        return fail(-1, "GQA decode: unknown kv_format %d", a->kv_format);
    }
    if (a->kv_format == ZLLM_KV_Q8G64 && (a->scale_dtype < ZLLM_SCALE_BF16 || a->scale_dtype > ZLLM_SCALE_F32)) {
        return fail(-1, "GQA decode: Q8g64 scales must be bf16, f16 or f32 (got %d)", a->scale_dtype);
    }
    if (a->kv_format == ZLLM_KV_F16 && a->head_dim != 128 && a->head_dim != 256) {
        return fail(-1, "GQA decode: f16 KV supports head_dim 128 and 256");
    }
    if (a->q_dtype < ZLLM_DTYPE_F32 || a->q_dtype > ZLLM_DTYPE_F16) {
        return fail(-1, "GQA decode: unknown q_dtype %d", a->q_dtype);
    }
    if (a->stages > ZLLM_STAGE_MERGE) {
        return fail(-1, "GQA decode: unknown stages %u", a->stages);
    }
    return 0;
}

// Shortest GQA split: two 32-token steps.  A short visible range (a sliding-window layer, a short context) is
// latency-bound -- a workgroup walks its steps one memory round trip after the other -- so it is cut into as many
// splits as there are CUs before the splits are allowed to grow; the partial records this adds are a few percent of
// the KV bytes even at 64 tokens per split.
constexpr uint64_t kMinGqaChunk = 64;

// The head_dim-128 Q8g64 kernel that streams pages straight into LDS keeps a split's block-table entries in two
// registers per lane: a split of at most 127 pages.  A longer split is cut into equal shorter ones (further whole rounds
// of workgroups), so that a long batch keeps that kernel.
void cap_split_for_page_registers(const zllm_gqa_decode_args* a, uint32_t* chunk_tokens, uint32_t* max_chunks)
{
    const bool pow2 = (a->block_tokens & (a->block_tokens - 1u)) == 0;
    if (a->kv_format != ZLLM_KV_Q8G64 || a->head_dim != 128 || a->scale_dtype == ZLLM_SCALE_F32 || a->ring_capacity != 0 || !pow2 ||
        a->block_tokens < 16u) {
        return;
    }
    const uint64_t limit = ((uint64_t)127u * a->block_tokens) & ~(uint64_t)31u;
    if (*chunk_tokens <= limit) {
        return;
    }
    const uint64_t parts = (*chunk_tokens + limit - 1) / limit;
    const uint64_t chunk = align_up((*chunk_tokens + parts - 1) / parts, 32);
    *chunk_tokens = (uint32_t)chunk;
    *max_chunks = (uint32_t)((a->max_kv_len + chunk - 1) / chunk);
}

// Rows of the split record arrays.  A plan made for equal lengths keeps [sequence][max_chunks] rows, which a workgroup
// and the merge address without reading anything.  A ragged plan (total_kv_tokens given and below batch x max_kv_len) numbers
// its records like its work items, densely over the live splits: sequence b has ceil((len_b - first_b rounded down to 32) /
// chunk_tokens) of them, so total / chunk_tokens + 2 x batch rows hold them all, however long the longest sequence is.
struct GqaSplitPlan {
    uint32_t chunk_tokens, max_chunks;
    uint64_t record_rows;
    bool dense;
};

GqaSplitPlan plan_gqa_decode(const zllm_gqa_decode_args* a)
{
    GqaSplitPlan plan;
    const uint64_t cus = compute_units();
    const uint32_t max_waves = zllm::gqa_decode_max_waves(a->head_dim);
    const uint32_t waves = a->num_kv_heads < max_waves ? a->num_kv_heads : max_waves;
    const uint32_t kvh_blocks = (a->num_kv_heads + waves - 1) / waves;
    const uint32_t head_blocks = (a->num_heads / a->num_kv_heads + 15) / 16;
    const uint32_t items_per_group = zllm::gqa_decode_items_per_group(a->head_dim, a->num_kv_heads);
    const uint64_t columns = (uint64_t)a->batch * kvh_blocks * head_blocks;
    const uint64_t uniform_total = (uint64_t)a->batch * a->max_kv_len;
    plan.dense = false;
    if (a->total_kv_tokens != 0 && a->total_kv_tokens < uniform_total && cus * items_per_group > 2 * columns) {
        // ragged batch: sum_b ceil(len_b / chunk) <= total / chunk + batch, so size the splits for the
        // workgroups that will really run and keep them within one round of the CUs
        const uint64_t slots = cus * items_per_group / (kvh_blocks * head_blocks) - a->batch;
        uint64_t chunk = (a->total_kv_tokens + slots - 1) / slots;
        chunk = align_up(chunk < kMinGqaChunk ? kMinGqaChunk : chunk, 32);
        plan.chunk_tokens = (uint32_t)chunk;
        plan.max_chunks = (uint32_t)((a->max_kv_len + chunk - 1) / chunk);
        plan.dense = true;
    } else {
        plan_splits(a->max_kv_len, columns, items_per_group, kMinGqaChunk, &plan.chunk_tokens, &plan.max_chunks);
    }
    cap_split_for_page_registers(a, &plan.chunk_tokens, &plan.max_chunks);
    plan.record_rows = (uint64_t)a->batch * plan.max_chunks;
    if (plan.dense) {
        const uint64_t live = a->total_kv_tokens / plan.chunk_tokens + 2ull * a->batch;
        if (live < plan.record_rows) {
            plan.record_rows = live;
        } else {
            plan.dense = false; // nothing to save: keep the rows that need no lookup
        }
    }
    return plan;
}

struct GqaWorkspace {
    uint64_t stats, first_rows, total;
};

GqaWorkspace gqa_workspace(const zllm_gqa_decode_args* a, const GqaSplitPlan& plan)
{
    GqaWorkspace w;
    const uint64_t rows = plan.record_rows * a->num_heads;
    w.stats = align_up(rows * a->head_dim * 4, 256);
    w.first_rows = w.stats + align_up(rows * 8, 256);
    w.total = w.first_rows + (plan.dense ? align_up((uint64_t)a->batch * 4, 256) : 0);
    return w;
}

// query rows per sequence: 0 and 1 both mean a decode step
uint32_t mla_query_rows(const zllm_mla_decode_args* a)
{
    return a->query_rows == 0 ? 1u : a->query_rows;
}

int validate_mla_decode(const zllm_mla_decode_args* a)
{
    if (a == nullptr) {
        return fail(-1, "MLA decode: null args");
    }
    // shape rules of try_paged_mla_attention_ct_inner (paged_mla.rs:2940-2949)
    if (a->batch == 0 || a->heads == 0 || a->q_head_dim == 0 || a->kv_head_dim == 0 || a->rope_dim > a->q_head_dim ||
        a->q_head_dim - a->rope_dim > a->kv_head_dim || a->q_head_dim > 1024) {
        return fail(-1, "MLA decode: invalid shape batch=%u heads=%u q_head=%u kv_head=%u rope=%u", a->batch, a->heads, a->q_head_dim,
                    a->kv_head_dim, a->rope_dim);
    }
    {
        // project_value writes value_dim columns per head into a slot of stride q_head_dim (strided output) or
        // value_dim (compact): an empty or overlong value part has nowhere to go
        const uint32_t value_dim = a->kv_head_dim - (a->q_head_dim - a->rope_dim);
        if (value_dim == 0 || (!a->out_compact && value_dim > a->q_head_dim)) {
            return fail(-1, "MLA decode: value_dim=%u must be non-zero and, for strided output, at most q_head_dim=%u", value_dim,
                        a->q_head_dim);
        }
    }
    // latent rows are Q8g64 (a scale per 64 columns); a lane of the vector-ALU kernels owns up to 16 latent and 4 rope columns
    if (a->latent_dim == 0 || a->latent_dim % 64u != 0 || a->latent_dim > 1024u || a->rope_dim % 2u != 0 || a->rope_dim > 256u) {
        return fail(-1, "MLA decode: latent_dim must be a multiple of 64 up to 1024 and rope_dim even up to 256 (got %u + %u)", a->latent_dim,
                    a->rope_dim);
    }
    if (a->kv_b_bits != 0u && a->kv_b_bits != 16u && a->kv_b_bits != 32u && a->kv_b_bits != 8u && a->kv_b_bits != 4u) {
        return fail(-1, "MLA decode: kv_b_bits must be 0 / 16 (bf16), 32 (f32), 8 or 4 (got %u)", a->kv_b_bits);
    }
    if ((a->kv_b_bits == 8u || a->kv_b_bits == 4u) &&
        (a->kv_b_scales == nullptr || a->kv_b_group == 0u || a->latent_dim % a->kv_b_group != 0 || a->kv_b_scale_dtype < ZLLM_SCALE_BF16 ||
         a->kv_b_scale_dtype > ZLLM_SCALE_F32)) {
        return fail(-1, "MLA decode: %u-bit kv_b needs scales, a group size that divides latent_dim=%u (got %u) and a scale dtype", a->kv_b_bits,
                    a->latent_dim, a->kv_b_group);
    }
    if (a->block_tokens == 0 || a->max_ctx_len == 0 || a->max_ctx_len > kMaxTokens) {
        return fail(-1, "MLA decode: block_tokens=%u max_ctx_len=%u must be non-zero, max_ctx_len below 2^31", a->block_tokens, a->max_ctx_len);
    }
    if ((a->q_dtype != ZLLM_DTYPE_F32 && a->q_dtype != ZLLM_DTYPE_BF16) || (a->out_dtype != ZLLM_DTYPE_F32 && a->out_dtype != ZLLM_DTYPE_BF16)) {
        return fail(-1, "MLA decode: q_dtype / out_dtype must be f32 or bf16");
    }
    if (a->stage_mask > 31u) {
        return fail(-1, "MLA decode: unknown stage_mask %u", a->stage_mask);
    }
    if (a->selection != nullptr && a->top_k == 0) {
        return fail(-1, "MLA decode: a selection needs top_k > 0");
    }
    // query rows over the whole call index the grid's third dimension
    if ((uint64_t)a->batch * mla_query_rows(a) > 65535u) {
        return fail(-1, "MLA decode: batch=%u x query_rows=%u exceeds 65535 query rows per call", a->batch, a->query_rows);
    }
    return 0;
}

struct MlaSplitPlan {
    uint32_t chunk_tokens, max_chunks;
    uint64_t record_rows; // rows of the record arrays
    bool dense;           // numbered over the live splits (see GqaSplitPlan)
};

MlaSplitPlan plan_mla_decode(const zllm_mla_decode_args* a)
{
    MlaSplitPlan plan;
    // one workgroup per CU: the partial kernel owns a whole CU (LDS tile + 512 registers per lane)
    // 64 heads per workgroup; the vector-ALU kernel of the other latent / rope widths runs one head per workgroup
    const uint32_t head_blocks = a->latent_dim == 512u && a->rope_dim == 64u ? (a->heads + 63) / 64 : a->heads;
    // with a selection no sequence attends to more than top_k tokens (shorter contexts stay dense)
    const uint32_t longest = a->selection != nullptr && a->top_k < a->max_ctx_len ? a->top_k : a->max_ctx_len;
    const uint64_t query_rows = mla_query_rows(a);
    const uint64_t per_sequence = query_rows * head_blocks; // workgroups per split of a sequence
    const uint64_t cus = compute_units();
    const uint64_t uniform_total = (uint64_t)a->batch * a->max_ctx_len;
    plan.dense = false;
    if (a->selection == nullptr && a->total_ctx_tokens != 0 && a->total_ctx_tokens < uniform_total && cus > 2 * a->batch * per_sequence) {
        // ragged batch, as in plan_gqa_decode: sum_b ceil(len_b / chunk) <= total / chunk + batch
        const uint64_t slots = cus / per_sequence - a->batch;
        uint64_t chunk = (a->total_ctx_tokens + slots - 1) / slots;
        chunk = align_up(chunk < 64 ? 64 : chunk, 32);
        plan.chunk_tokens = (uint32_t)chunk;
        plan.max_chunks = (uint32_t)(((uint64_t)longest + chunk - 1) / chunk);
        plan.dense = true;
    } else {
        plan_splits(longest, (uint64_t)a->batch * per_sequence, 1, 64, &plan.chunk_tokens, &plan.max_chunks);
    }
    const uint64_t rows = (uint64_t)a->batch * query_rows;
    plan.record_rows = rows * plan.max_chunks;
    if (plan.dense) {
        // every query row of a sequence sees at most the sequence's tokens: query_rows x (total / chunk) + one per row
        const uint64_t live = query_rows * (a->total_ctx_tokens / plan.chunk_tokens) + rows;
        if (live < plan.record_rows && live <= UINT32_MAX) {
            plan.record_rows = live;
        } else {
            plan.dense = false;
        }
    }
    return plan;
}

struct MlaWorkspace {
    uint64_t absorbed, partial, stats, weighted, first_rows, total;
};

MlaWorkspace mla_workspace(const zllm_mla_decode_args* a, const MlaSplitPlan& plan)
{
    MlaWorkspace w;
    const uint64_t rows = (uint64_t)a->batch * mla_query_rows(a) * a->heads;
    const uint64_t records = plan.record_rows * a->heads;
    w.absorbed = 0;
    w.partial = align_up(rows * (a->latent_dim + a->rope_dim) * 2, 256);
    w.stats = w.partial + align_up(records * a->latent_dim * 4, 256);
    w.weighted = w.stats + align_up(records * 8, 256);
    w.first_rows = w.weighted + align_up(rows * a->latent_dim * 4, 256);
    w.total = w.first_rows + (plan.dense ? align_up((uint64_t)a->batch * mla_query_rows(a) * 4, 256) : 0);
    return w;
}

} // namespace

extern "C" {

int zllm_attn_init(int device, int* cu_count)
{
    hipDeviceProp_t prop;
    hipError_t err = hipGetDeviceProperties(&prop, device);
    if (err != hipSuccess) {
        return hip_status(err, "hipGetDeviceProperties");
    }
    if (cu_count != nullptr) {
        *cu_count = prop.multiProcessorCount;
    }
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        return fail(-2, "zllm_attn is built for gfx950 only; device %d is %s", device, prop.gcnArchName);
    }
    // the static scratch array of zllm_attn_gqa_decode_static: its address on this device, found with the device current
    int current = -1;
    err = hipGetDevice(&current);
    if (err != hipSuccess) {
        return hip_status(err, "hipGetDevice");
    }
    if (current != device) {
        err = hipSetDevice(device);
        if (err != hipSuccess) {
            return hip_status(err, "hipSetDevice");
        }
    }
    void* base = nullptr;
    const int found = resolve_static_scratch(device, &base);
    if (current != device) {
        (void)hipSetDevice(current);
    }
    return found;
}

const char* zllm_attn_last_error(void)
{
    return g_error;
}

/* ---- host layout arithmetic ------------------------------------------------------------- */

void zllm_attn_key_range(uint64_t window, uint64_t query_position, uint64_t key_end, uint64_t* start, uint64_t* end)
{
    uint64_t causal_end = query_position + 1 < key_end ? query_position + 1 : key_end;
    uint64_t s = 0;
    if (window != 0) {
        s = query_position + 1 > window ? query_position + 1 - window : 0;
    }
    *start = s < causal_end ? s : causal_end;
    *end = causal_end;
}

uint64_t zllm_kv_bytes_per_token(int kind, uint64_t a, uint64_t b, uint64_t group)
{
    if (group == 0) {
        return 0;
    }
    if (kind == 0) {
        if (a == 0 || b == 0 || a % group != 0) {
            return 0;
        }
        return a + (a / group) * 2 + b * 2;
    }
    if (a == 0 || b == 0 || b % group != 0) {
        return 0;
    }
    return 2 * (a * b) + 4 * (a * (b / group));
}

uint64_t zllm_kv_layout_offsets(int kind, uint64_t a, uint64_t b, uint64_t group, uint64_t layer_count, uint64_t capacity,
                                uint64_t layer, uint64_t offsets[5])
{
    const uint64_t per_token = zllm_kv_bytes_per_token(kind, a, b, group);
    if (per_token == 0 || capacity == 0 || layer_count == 0 || layer >= layer_count) {
        return 0;
    }
    const uint64_t stride = capacity * per_token;
    const uint64_t base = layer * stride;
    offsets[0] = base;
    if (kind == 0) {
        const uint64_t codes = capacity * a;
        const uint64_t scales = capacity * (a / group) * 2;
        offsets[1] = base;
        offsets[2] = base + codes;
        offsets[3] = base + codes + scales;
        offsets[4] = 0;
    } else {
        const uint64_t codes = capacity * a * b;
        const uint64_t scales = capacity * a * (b / group) * 2;
        offsets[1] = base;
        offsets[2] = base + codes;
        offsets[3] = base + codes + scales;
        offsets[4] = base + 2 * codes + scales;
    }
    return layer_count * stride;
}

int zllm_kv_ring_write_plan(uint64_t capacity, uint64_t max_sequence_len, uint64_t position, uint64_t count, uint64_t plan[6])
{
    if (count == 0 || capacity == 0 || position + count > max_sequence_len) {
        return fail(-1, "ring write plan: capacity=%llu position=%llu count=%llu max=%llu", (unsigned long long)capacity,
                    (unsigned long long)position, (unsigned long long)count, (unsigned long long)max_sequence_len);
    }
    const uint64_t end = position + count;
    const uint64_t oldest_kept = end > capacity ? end - capacity : 0;
    const uint64_t write_start = position > oldest_kept ? position : oldest_kept;
    const uint64_t tokens = end - write_start;
    const uint64_t first_slot = write_start % capacity;
    const uint64_t first_count = tokens < capacity - first_slot ? tokens : capacity - first_slot;
    plan[0] = end;
    plan[1] = write_start - position;
    plan[2] = tokens;
    plan[3] = first_slot;
    plan[4] = first_count;
    plan[5] = tokens - first_count;
    return 0;
}

/* ---- appends ---------------------------------------------------------------------------- */

int zllm_attn_q8g64_append(const zllm_q8_append_args* a, zllm_stream_t stream)
{
    if (a == nullptr || a->src == nullptr || a->codes == nullptr || a->scales == nullptr) {
        return fail(-1, "Q8g64 append: null pointer");
    }
    if (a->cols == 0 || a->cols % ZLLM_GROUP_SIZE != 0 || a->block_tokens == 0) {
        return fail(-1, "Q8g64 append: cols=%u must be a non-zero multiple of 64, block_tokens=%u non-zero", a->cols, a->block_tokens);
    }
    if (a->rule < ZLLM_QUANT_ROCM_MLA || a->rule > ZLLM_QUANT_CUDA_GQA || a->src_dtype < ZLLM_DTYPE_F32 || a->src_dtype > ZLLM_DTYPE_F16) {
        return fail(-1, "Q8g64 append: unknown rule %d or src_dtype %d", a->rule, a->src_dtype);
    }
    if ((uint64_t)a->position + a->rows > 0xffffffffull) {
        return fail(-1, "Q8g64 append: position + rows overflows u32");
    }
    zllm::Q8AppendParams p{a->src, (signed char*)a->codes, a->scales, a->table, a->positions, a->position, a->rows, a->cols,
                           a->block_tokens, a->ring_capacity, a->src_dtype, a->rule};
    return hip_status(zllm::launch_q8g64_append(p, (hipStream_t)stream), "Q8g64 append launch");
}

int zllm_attn_gqa_prologue(const zllm_gqa_prologue_args* a, zllm_stream_t stream)
{
    if (a == nullptr || a->q == nullptr || a->k == nullptr || a->v == nullptr || a->q_out == nullptr || a->k_codes == nullptr ||
        a->k_scales == nullptr || a->v_codes == nullptr || a->v_scales == nullptr) {
        return fail(-1, "GQA prologue: null pointer");
    }
    // shape rules of rmsnorm_heads (src/backend/cpu/attention.rs:463-467) and apply_f32 (src/attention/rope.rs:121-138)
    if (a->rows == 0 || a->num_heads == 0 || a->num_kv_heads == 0 || a->head_dim == 0 || a->head_dim % ZLLM_GROUP_SIZE != 0 ||
        a->head_dim > 256 || a->block_tokens == 0) {
        return fail(-1, "GQA prologue: invalid shape rows=%u heads=%u/%u head_dim=%u block_tokens=%u", a->rows, a->num_heads,
                    a->num_kv_heads, a->head_dim, a->block_tokens);
    }
    if (a->rotary_dim % 2 != 0 || a->rotary_dim > a->head_dim) {
        return fail(-1, "GQA prologue: rotary_dim=%u must be even and at most head_dim=%u", a->rotary_dim, a->head_dim);
    }
    if (a->rotary_dim != 0 && (a->cosine == nullptr || a->sine == nullptr || (uint64_t)a->position + a->rows > a->rope_table_rows)) {
        return fail(-1, "GQA prologue: RoPE table of %u rows cannot serve position %u + %u rows", a->rope_table_rows, a->position, a->rows);
    }
    if ((a->q_norm != nullptr || a->k_norm != nullptr) && !(a->eps > 0.0f && a->eps < INFINITY)) {
        return fail(-1, "GQA prologue: eps must be finite and positive");
    }
    if (a->rule < ZLLM_QUANT_ROCM_MLA || a->rule > ZLLM_QUANT_CUDA_GQA || a->src_dtype < ZLLM_DTYPE_F32 || a->src_dtype > ZLLM_DTYPE_F16 ||
        (a->q_out_dtype != ZLLM_DTYPE_F32 && a->q_out_dtype != ZLLM_DTYPE_BF16)) {
        return fail(-1, "GQA prologue: unknown rule %d, src_dtype %d or q_out_dtype %d", a->rule, a->src_dtype, a->q_out_dtype);
    }
    if ((uint64_t)a->position + a->rows > 0xffffffffull) {
        return fail(-1, "GQA prologue: position + rows overflows u32");
    }
    zllm::GqaPrologueParams p{a->q, a->k, a->v, a->q_norm, a->k_norm, a->cosine, a->sine, a->q_out, (signed char*)a->k_codes, a->k_scales,
                              (signed char*)a->v_codes, a->v_scales, a->table, a->positions, a->rows, a->num_heads, a->num_kv_heads,
                              a->head_dim, a->rotary_dim, a->position, a->block_tokens, a->ring_capacity, a->eps, a->weight_offset,
                              a->src_dtype, a->q_out_dtype, a->rule, a->split_half};
    return hip_status(zllm::launch_gqa_prologue(p, (hipStream_t)stream), "GQA prologue launch");
}

int zllm_attn_half_append(const zllm_half_append_args* a, zllm_stream_t stream)
{
    if (a == nullptr || a->src == nullptr || a->cache == nullptr) {
        return fail(-1, "half append: null pointer");
    }
    if (a->cols == 0 || a->block_tokens == 0) {
        return fail(-1, "half append: cols and block_tokens must be non-zero");
    }
    if (a->dst_dtype != ZLLM_DTYPE_BF16 && a->dst_dtype != ZLLM_DTYPE_F16) {
        return fail(-1, "half append: dst_dtype must be bf16 or f16");
    }
    if (a->src_dtype < ZLLM_DTYPE_F32 || a->src_dtype > ZLLM_DTYPE_F16) {
        return fail(-1, "half append: unknown src_dtype %d", a->src_dtype);
    }
    zllm::HalfAppendParams p{a->src, (unsigned short*)a->cache, a->table, a->position, a->rows, a->cols, a->block_tokens,
                             a->ring_capacity, a->src_dtype, a->dst_dtype};
    return hip_status(zllm::launch_half_append(p, (hipStream_t)stream), "half append launch");
}

int zllm_attn_mla_append(const zllm_mla_append_args* a, zllm_stream_t stream)
{
    if (a == nullptr || a->latent == nullptr || a->k_rope == nullptr || a->latent_codes == nullptr || a->latent_scales == nullptr ||
        a->rope_cache == nullptr) {
        return fail(-1, "MLA append: null pointer");
    }
    if (a->latent_cols == 0 || a->latent_cols % ZLLM_GROUP_SIZE != 0 || a->rope_cols == 0 || a->block_tokens == 0) {
        return fail(-1, "MLA append: latent_cols=%u (multiple of 64) rope_cols=%u block_tokens=%u", a->latent_cols, a->rope_cols,
                    a->block_tokens);
    }
    if (a->rotary_dim > a->rope_cols || a->rotary_dim % 2 != 0 || (a->rotary_dim != 0 && (a->cosine == nullptr || a->sine == nullptr))) {
        return fail(-1, "MLA append: rotary_dim=%u invalid for rope_cols=%u (or missing cos/sin)", a->rotary_dim, a->rope_cols);
    }
    if (a->rotary_layout != ZLLM_ROTARY_INTERLEAVED && a->rotary_layout != ZLLM_ROTARY_SPLIT_HALF) {
        return fail(-1, "MLA append: unknown rotary layout %d", a->rotary_layout);
    }
    zllm::MlaAppendParams p{a->latent, a->k_rope, a->cosine, a->sine, (signed char*)a->latent_codes, a->latent_scales, a->rope_cache,
                            a->table, a->positions, a->position, a->rope_position, a->rows, a->latent_cols, a->rope_cols,
                            a->rotary_dim, a->rotary_layout == ZLLM_ROTARY_SPLIT_HALF ? 1u : 0u, a->block_tokens};
    return hip_status(zllm::launch_mla_append(p, (hipStream_t)stream), "MLA append launch");
}

int zllm_attn_gather_rows(const zllm_gather_args* a, zllm_stream_t stream)
{
    if (a == nullptr || a->plane == nullptr || a->out == nullptr) {
        return fail(-1, "gather rows: null pointer");
    }
    if (a->block_tokens == 0) {
        return fail(-1, "gather rows: block_tokens must be non-zero");
    }
    zllm::GatherParams p{a->plane, a->out, a->table, a->first, a->count, a->row_bytes, a->block_tokens, a->ring_capacity};
    return hip_status(zllm::launch_gather_rows(p, (hipStream_t)stream), "gather rows launch");
}

int zllm_attn_scatter_rows(const zllm_scatter_args* a, zllm_stream_t stream)
{
    if (a == nullptr || a->plane == nullptr || a->in == nullptr) {
        return fail(-1, "scatter rows: null pointer");
    }
    if (a->block_tokens == 0) {
        return fail(-1, "scatter rows: block_tokens must be non-zero");
    }
    zllm::ScatterParams p{a->plane, a->in, a->table, a->first, a->count, a->row_bytes, a->block_tokens, a->ring_capacity};
    return hip_status(zllm::launch_scatter_rows(p, (hipStream_t)stream), "scatter rows launch");
}

/* ---- KV snapshot wire format (host) ----------------------------------------------------- */

static bool mla_record_shape_ok(const zllm_mla_layer_record* r)
{
    // download_device (src/backend/rocm/kv_cache.rs:3373-3388): Q8 codes are one byte per element with bf16 scales per
    // group, the bf16 mode has two bytes per element and no scales
    if (r->ownership > ZLLM_KV_OWNERSHIP_INTERLEAVED) {
        return false;
    }
    if (r->latent_group_size == 0) {
        return r->latent_scales == nullptr && r->latent_scales_bytes == 0 && r->latent_bytes == r->rows * r->latent_cols * 2 &&
               r->rope_bytes == r->rows * r->rope_cols * 2;
    }
    return r->latent_cols % r->latent_group_size == 0 && r->latent_bytes == r->rows * r->latent_cols &&
           r->latent_scales != nullptr && r->latent_scales_bytes == r->rows * (r->latent_cols / r->latent_group_size) * 2 &&
           r->rope_bytes == r->rows * r->rope_cols * 2;
}

uint64_t zllm_kv_mla_layer_wire_bytes(const zllm_mla_layer_record* r)
{
    if (r == nullptr || !mla_record_shape_ok(r)) {
        return 0;
    }
    return 8 + 1 + 3 * 8 + (8 + r->latent_bytes) + 1 + (r->latent_scales != nullptr ? 8 + r->latent_scales_bytes : 0) + (8 + r->rope_bytes);
}

static uint8_t* put_u64(uint8_t* at, uint64_t value)
{
    for (int i = 0; i < 8; ++i) {
        at[i] = (uint8_t)(value >> (8 * i));
    }
    return at + 8;
}

static uint8_t* put_blob(uint8_t* at, const uint8_t* bytes, uint64_t len)
{
    at = put_u64(at, len);
    if (len != 0) {
        memcpy(at, bytes, len);
    }
    return at + len;
}

int zllm_kv_mla_layer_write(const zllm_mla_layer_record* r, uint8_t* out, uint64_t capacity, uint64_t* written)
{
    const uint64_t need = zllm_kv_mla_layer_wire_bytes(r);
    if (need == 0 || out == nullptr) {
        return fail(-1, "MLA layer write: record lengths do not match its shape");
    }
    if (capacity < need) {
        return fail(-1, "MLA layer write: %llu bytes needed, %llu given", (unsigned long long)need, (unsigned long long)capacity);
    }
    uint8_t* at = put_u64(out, r->rows);
    *at++ = (uint8_t)r->ownership;
    at = put_u64(at, r->latent_cols);
    at = put_u64(at, r->rope_cols);
    at = put_u64(at, r->latent_group_size);
    at = put_blob(at, r->latent, r->latent_bytes);
    if (r->latent_scales != nullptr) {
        *at++ = 1;
        at = put_blob(at, r->latent_scales, r->latent_scales_bytes);
    } else {
        *at++ = 0;
    }
    at = put_blob(at, r->rope, r->rope_bytes);
    if (written != nullptr) {
        *written = (uint64_t)(at - out);
    }
    return 0;
}

namespace {
struct WireReader {
    const uint8_t* at;
    uint64_t remaining;
    bool ok = true;
    uint64_t u64()
    {
        if (remaining < 8) {
            ok = false;
            return 0;
        }
        uint64_t value = 0;
        for (int i = 0; i < 8; ++i) {
            value |= (uint64_t)at[i] << (8 * i);
        }
        at += 8;
        remaining -= 8;
        return value;
    }
    uint8_t byte()
    {
        if (remaining < 1) {
            ok = false;
            return 0;
        }
        --remaining;
        return *at++;
    }
    const uint8_t* blob(uint64_t* len)
    {
        *len = u64();
        if (!ok || *len > remaining) { // "blob longer than what is left" (rocm_swap.rs:1195-1203)
            ok = false;
            return nullptr;
        }
        const uint8_t* start = at;
        at += *len;
        remaining -= *len;
        return start;
    }
};
} // namespace

int zllm_kv_mla_layer_read(const uint8_t* in, uint64_t len, zllm_mla_layer_record* r, uint64_t* consumed)
{
    if (in == nullptr || r == nullptr) {
        return fail(-1, "MLA layer read: null pointer");
    }
    WireReader reader{in, len};
    memset(r, 0, sizeof(*r));
    r->rows = reader.u64();
    r->ownership = reader.byte();
    r->latent_cols = reader.u64();
    r->rope_cols = reader.u64();
    r->latent_group_size = reader.u64();
    r->latent = reader.blob(&r->latent_bytes);
    const uint8_t flag = reader.byte();
    if (reader.ok && flag > 1) {
        return fail(-1, "MLA layer read: flag byte %u", flag);
    }
    if (flag == 1) {
        r->latent_scales = reader.blob(&r->latent_scales_bytes);
    }
    r->rope = reader.blob(&r->rope_bytes);
    if (!reader.ok) {
        return fail(-1, "MLA layer read: record truncated (%llu bytes given)", (unsigned long long)len);
    }
    if (r->ownership > ZLLM_KV_OWNERSHIP_INTERLEAVED) {
        return fail(-1, "MLA layer read: ownership byte %u", r->ownership);
    }
    if (consumed != nullptr) {
        *consumed = len - reader.remaining;
    }
    if (!mla_record_shape_ok(r)) {
        return fail(-2, "MLA layer read: blob lengths do not match rows=%llu latent=%llu rope=%llu group=%llu", (unsigned long long)r->rows,
                    (unsigned long long)r->latent_cols, (unsigned long long)r->rope_cols, (unsigned long long)r->latent_group_size);
    }
    return 0;
}

/* ---- GQA decode ------------------------------------------------------------------------- */

uint64_t zllm_attn_gqa_decode_workspace_bytes(const zllm_gqa_decode_args* a)
{
    if (validate_gqa_decode(a) != 0) {
        return 0;
    }
    return gqa_workspace(a, plan_gqa_decode(a)).total;
}

// The decode call over a workspace that is either the caller's or the library's static array.
static int gqa_decode_over(const zllm_gqa_decode_args* a, void* workspace, uint64_t workspace_bytes, zllm_stream_t stream,
                           bool table_shared = false, int out_dtype = ZLLM_DTYPE_F32)
{
    if (a->q == nullptr || a->k_plane == nullptr || a->v_plane == nullptr || a->kv_lens == nullptr || a->out == nullptr ||
        workspace == nullptr || (a->kv_format == ZLLM_KV_Q8G64 && (a->k_scales == nullptr || a->v_scales == nullptr))) {
        return fail(-1, "GQA decode: null pointer");
    }
    if ((((uintptr_t)a->q | (uintptr_t)a->k_plane | (uintptr_t)a->v_plane | (uintptr_t)workspace | (uintptr_t)a->out) & 15u) != 0 ||
        (((uintptr_t)a->k_scales | (uintptr_t)a->v_scales) & 3u) != 0) {
        return fail(-1, "GQA decode: q, cache planes, out and workspace must be 16-byte aligned (scale planes 4-byte)");
    }
    const uint64_t need = zllm_attn_gqa_decode_workspace_bytes(a);
    if (workspace_bytes < need) {
        return fail(-1, "GQA decode: workspace %llu bytes, need %llu", (unsigned long long)workspace_bytes, (unsigned long long)need);
    }
    if (a->tables != nullptr && (uint64_t)a->table_stride * a->block_tokens < a->max_kv_len && a->ring_capacity == 0) {
        return fail(-1, "GQA decode: table_stride=%u pages of %u tokens cannot cover max_kv_len=%u", a->table_stride, a->block_tokens,
                    a->max_kv_len);
    }
    zllm::GqaDecodeParams p;
    memset(&p, 0, sizeof(p));
    p.q = a->q;
    p.k_plane = (const unsigned char*)a->k_plane;
    p.k_scales = (const unsigned char*)a->k_scales;
    p.v_plane = (const unsigned char*)a->v_plane;
    p.v_scales = (const unsigned char*)a->v_scales;
    p.tables = a->tables;
    p.kv_lens = a->kv_lens;
    p.first_visible = a->first_visible;
    p.out = a->out;
    const GqaSplitPlan plan = plan_gqa_decode(a);
    const GqaWorkspace layout = gqa_workspace(a, plan);
    p.chunk_tokens = plan.chunk_tokens;
    p.max_chunks = plan.max_chunks;
    p.partial = (float*)workspace;
    p.stats = (float*)((char*)workspace + layout.stats);
    if (plan.dense) {
        p.record_rows = (unsigned int)plan.record_rows;
        p.first_rows = (unsigned int*)((char*)workspace + layout.first_rows);
    }
    p.batch = a->batch;
    p.num_heads = a->num_heads;
    p.num_kv_heads = a->num_kv_heads;
    p.head_dim = a->head_dim;
    p.group = a->num_heads / a->num_kv_heads;
    p.table_stride = a->table_stride;
    p.table_shared = table_shared ? 1u : 0u;
    p.out_dtype = out_dtype;
    p.block_tokens = a->block_tokens;
    p.block_shift = shift_of(a->block_tokens);
    p.ring_capacity = a->ring_capacity;
    p.score_scale = a->score_scale;
    p.softcap = a->softcap;
    p.q_dtype = a->q_dtype;
    if (a->gate != nullptr) {
        // shape rule of sigmoid_gate (src/backend/cpu/context.rs:420-422)
        if ((a->gate_cols != 1 && a->gate_cols != a->num_heads * a->head_dim) || (a->gate_dtype != ZLLM_DTYPE_F32 && a->gate_dtype != ZLLM_DTYPE_BF16)) {
            return fail(-1, "GQA decode: gate_cols=%u must be 1 or %u, gate_dtype f32 or bf16", a->gate_cols, a->num_heads * a->head_dim);
        }
        p.gate = a->gate;
        p.gate_cols = a->gate_cols;
        p.gate_dtype = a->gate_dtype;
    }
    return hip_status(zllm::launch_gqa_decode(p, a->kv_format, a->scale_dtype, a->stages, (hipStream_t)stream), "GQA decode launch");
}

int zllm_attn_gqa_decode_split_plan(const zllm_gqa_decode_args* a, uint32_t* chunk_tokens, uint32_t* max_chunks)
{
    const int rc = validate_gqa_decode(a);
    if (rc != 0) {
        return rc;
    }
    const GqaSplitPlan plan = plan_gqa_decode(a);
    if (chunk_tokens != nullptr) {
        *chunk_tokens = plan.chunk_tokens;
    }
    if (max_chunks != nullptr) {
        *max_chunks = plan.max_chunks;
    }
    return 0;
}

int zllm_attn_gqa_decode_record_layout(const zllm_gqa_decode_args* a, zllm_split_record_layout* out)
{
    const int rc = validate_gqa_decode(a);
    if (rc != 0) {
        return rc;
    }
    if (out == nullptr) {
        return fail(-1, "GQA decode record layout: null output");
    }
    const GqaSplitPlan plan = plan_gqa_decode(a);
    const GqaWorkspace layout = gqa_workspace(a, plan);
    out->record_rows = plan.record_rows;
    out->partial_offset = 0;
    out->stats_offset = layout.stats;
    out->first_rows_offset = plan.dense ? layout.first_rows : 0;
    out->chunk_tokens = plan.chunk_tokens;
    out->max_chunks = plan.max_chunks;
    out->dense = plan.dense ? 1u : 0u;
    return 0;
}

int zllm_attn_gqa_decode(const zllm_gqa_decode_args* a, zllm_stream_t stream)
{
    const int rc = validate_gqa_decode(a);
    if (rc != 0) {
        return rc;
    }
    return gqa_decode_over(a, a->workspace, a->workspace_bytes, stream);
}

uint64_t zllm_attn_static_scratch_bytes(void)
{
    return kStaticScratchBytes;
}

int zllm_attn_gqa_decode_static(const zllm_gqa_decode_args* a, zllm_stream_t stream)
{
    const int rc = validate_gqa_decode(a);
    if (rc != 0) {
        return rc;
    }
    const uint64_t need = zllm_attn_gqa_decode_workspace_bytes(a);
    if (need > kStaticScratchBytes) {
        return fail(-1, "GQA decode (static scratch): the split records of this call need %llu bytes, the static array holds %llu",
                    (unsigned long long)need, (unsigned long long)kStaticScratchBytes);
    }
    void* base = nullptr;
    const int found = static_scratch_of_current_device(&base);
    if (found != 0) {
        return found;
    }
    return gqa_decode_over(a, base, kStaticScratchBytes, stream);
}

/* ---- MLA decode ------------------------------------------------------------------------- */

uint64_t zllm_attn_mla_decode_workspace_bytes(const zllm_mla_decode_args* a)
{
    if (validate_mla_decode(a) != 0) {
        return 0;
    }
    return mla_workspace(a, plan_mla_decode(a)).total;
}

int zllm_attn_mla_decode_record_layout(const zllm_mla_decode_args* a, zllm_split_record_layout* out)
{
    const int rc = validate_mla_decode(a);
    if (rc != 0) {
        return rc;
    }
    if (out == nullptr) {
        return fail(-1, "MLA decode record layout: null output");
    }
    const MlaSplitPlan plan = plan_mla_decode(a);
    const MlaWorkspace w = mla_workspace(a, plan);
    out->record_rows = plan.record_rows;
    out->partial_offset = w.partial;
    out->stats_offset = w.stats;
    out->first_rows_offset = plan.dense ? w.first_rows : 0;
    out->chunk_tokens = plan.chunk_tokens;
    out->max_chunks = plan.max_chunks;
    out->dense = plan.dense ? 1u : 0u;
    return 0;
}

int zllm_attn_mla_decode(const zllm_mla_decode_args* a, zllm_stream_t stream)
{
    const int rc = validate_mla_decode(a);
    if (rc != 0) {
        return rc;
    }
    if (a->q == nullptr || a->kv_b == nullptr || a->latent_codes == nullptr || a->latent_scales == nullptr || a->rope_cache == nullptr ||
        a->ctx_lens == nullptr || a->out == nullptr || a->workspace == nullptr) {
        return fail(-1, "MLA decode: null pointer");
    }
    // the kernels read weights, codes, rope and the workspace as 16-byte vectors
    if ((((uintptr_t)a->kv_b | (uintptr_t)a->latent_codes | (uintptr_t)a->rope_cache | (uintptr_t)a->workspace) & 15u) != 0 ||
        (((uintptr_t)a->latent_scales) & 1u) != 0 || (((uintptr_t)a->out | (uintptr_t)a->q) & 3u) != 0) {
        return fail(-1, "MLA decode: kv_b, latent codes, rope cache and workspace must be 16-byte aligned (q and out 4-byte, scales 2-byte)");
    }
    zllm::MlaDecodeParams p;
    memset(&p, 0, sizeof(p));
    const MlaSplitPlan plan = plan_mla_decode(a);
    p.chunk_tokens = plan.chunk_tokens;
    p.max_chunks = plan.max_chunks;
    const MlaWorkspace w = mla_workspace(a, plan);
    if (a->workspace_bytes < w.total) {
        return fail(-1, "MLA decode: workspace %llu bytes, need %llu", (unsigned long long)a->workspace_bytes, (unsigned long long)w.total);
    }
    if (a->tables != nullptr && (uint64_t)a->table_stride * a->block_tokens < a->max_ctx_len) {
        return fail(-1, "MLA decode: table_stride=%u pages of %u tokens cannot cover max_ctx_len=%u", a->table_stride, a->block_tokens,
                    a->max_ctx_len);
    }
    char* ws = (char*)a->workspace;
    p.q = a->q;
    p.kv_b = a->kv_b;
    p.latent_codes = (const signed char*)a->latent_codes;
    p.latent_scales = a->latent_scales;
    p.rope_cache = a->rope_cache;
    p.tables = a->tables;
    p.ctx_lens = a->ctx_lens;
    p.out = a->out;
    p.absorbed = (unsigned short*)(ws + w.absorbed);
    p.partial = (float*)(ws + w.partial);
    p.stats = (float*)(ws + w.stats);
    p.weighted = (float*)(ws + w.weighted);
    if (plan.dense) {
        p.record_rows = (unsigned int)plan.record_rows;
        p.first_rows = (unsigned int*)(ws + w.first_rows);
    }
    p.query_rows = mla_query_rows(a);
    p.batch = a->batch * p.query_rows; // the kernels index query rows; a row finds its sequence by division
    p.heads = a->heads;
    p.q_head_dim = a->q_head_dim;
    p.kv_head_dim = a->kv_head_dim;
    p.latent_dim = a->latent_dim;
    p.rope_dim = a->rope_dim;
    p.nope_dim = a->q_head_dim - a->rope_dim;
    p.value_dim = a->kv_head_dim - p.nope_dim;
    p.table_stride = a->table_stride;
    p.block_tokens = a->block_tokens;
    p.block_shift = shift_of(a->block_tokens);
    // 1 / sqrt(q_head_dim): the reference's scale (src/attention/mla.rs:109, kernel/cpu/mla.rs:790)
    p.score_scale = 1.0f / sqrtf((float)a->q_head_dim);
    p.q_dtype = a->q_dtype;
    p.out_dtype = a->out_dtype;
    p.out_compact = a->out_compact;
    p.selection = a->selection;
    p.selection_counts = a->selection_counts;
    p.top_k = a->top_k;
    p.kv_b_scales = a->kv_b_scales;
    p.kv_b_bits = a->kv_b_bits == 0u ? 16u : a->kv_b_bits;
    p.kv_b_group = a->kv_b_group;
    p.kv_b_scale_dtype = a->kv_b_scale_dtype;
    return hip_status(zllm::launch_mla_decode(p, a->stage_mask, (hipStream_t)stream), "MLA decode launch");
}

/* ---- GQA chunked prefill ---------------------------------------------------------------- */

static int validate_gqa_prefill(const zllm_gqa_prefill_args* a)
{
    if (a == nullptr) {
        return fail(-1, "GQA prefill: null args");
    }
    // shape rules of try_block_attention_resident_f32 (tensor/attention.rs:727-745)
    if (a->rows == 0 || a->num_heads == 0 || a->num_kv_heads == 0 || a->num_heads % a->num_kv_heads != 0) {
        return fail(-1, "GQA prefill: invalid shape rows=%u heads=%u/%u", a->rows, a->num_heads, a->num_kv_heads);
    }
    // head dimensions of the reference's block attention that a Q8g64 group divides (tensor/attention.rs:727-745)
    if (!valid_head_dim(a->head_dim) || (a->kv_format != ZLLM_KV_Q8G64 && a->kv_format != ZLLM_KV_F16) ||
        (a->kv_format == ZLLM_KV_F16 && a->head_dim != 128 && a->head_dim != 256)) {
        return fail(-1, "GQA prefill: head_dim 64 / 128 / 192 / 256 over a Q8g64 cache or 128 / 256 over an f16 cache (got dim=%u format=%d)",
                    a->head_dim, a->kv_format);
    }
    if (a->num_heads / a->num_kv_heads > 256) {
        return fail(-1, "GQA prefill: at most 256 query heads per KV head");
    }
    if (a->kv_format == ZLLM_KV_Q8G64 && (a->scale_dtype < ZLLM_SCALE_BF16 || a->scale_dtype > ZLLM_SCALE_F32)) {
        return fail(-1, "GQA prefill: Q8g64 scales must be bf16, f16 or f32 (got %d)", a->scale_dtype);
    }
    if (a->table != nullptr && a->table_stride != 0 && (uint64_t)a->table_stride * a->block_tokens < (uint64_t)a->position + a->rows) {
        return fail(-1, "GQA prefill: table_stride=%u pages of %u tokens cannot cover position + rows = %llu", a->table_stride,
                    a->block_tokens, (unsigned long long)a->position + a->rows);
    }
    if (a->block_tokens == 0 || (uint64_t)a->position + a->rows > kMaxTokens) {
        return fail(-1, "GQA prefill: block_tokens must be non-zero and position + rows stay below 2^31");
    }
    if (!isfinite(a->score_scale) || a->score_scale <= 0.0f || !(a->softcap >= 0.0f) || !isfinite(a->softcap)) {
        return fail(-1, "GQA prefill: invalid score_scale=%g softcap=%g", (double)a->score_scale, (double)a->softcap);
    }
    if (a->q_dtype < ZLLM_DTYPE_F32 || a->q_dtype > ZLLM_DTYPE_F16 || a->out_dtype < ZLLM_DTYPE_F32 || a->out_dtype > ZLLM_DTYPE_F16) {
        return fail(-1, "GQA prefill: unknown q_dtype %d / out_dtype %d", a->q_dtype, a->out_dtype);
    }
    // explicit row ranges (BlockAttentionSpec::visible, src/attention/block.rs:10-16) come as two arrays and replace the
    // causal window altogether
    if (a->visible_starts != nullptr && (a->visible_ends == nullptr || a->window != 0)) {
        return fail(-1, "GQA prefill: visible_starts needs visible_ends and window == 0 (got window=%u)", a->window);
    }
    return 0;
}

// KV splits of a chunk kernel launch (zllm::GqaPrefillParams::max_chunks).  A workgroup is one row tile of one KV head
// walking the tile's whole visible range; a short chunk over a long prefix has few such workgroups, so the range is cut
// as a decode call's is -- whole rounds of the CUs, splits of at least 256 tokens (a workgroup first loads and
// normalises a tile of queries) -- and the parts meet in the split merge.  The records are
// rows x splits x heads x head_dim floats: a plan whose records would pass 256 MiB keeps fewer splits.
void plan_prefill_splits(const zllm_gqa_prefill_args* a, uint32_t* chunk_tokens, uint32_t* max_chunks)
{
    const uint32_t group = a->num_heads / a->num_kv_heads;
    const bool half_tiles = zllm::gqa_prefill_half_tiles(a->rows, a->position, a->window, a->num_heads, a->num_kv_heads, a->head_dim, a->kv_format,
                                                         a->scale_dtype, a->q_dtype);
    const uint32_t columns = a->head_dim == 256 || half_tiles ? 128u : 256u; // (row, head-in-group) pairs of a workgroup
    const uint32_t tile_rows = columns / group > 0 ? columns / group : 1u;
    const uint64_t tiles = ((uint64_t)a->rows + tile_rows - 1) / tile_rows;
    uint64_t longest = (uint64_t)a->position + a->rows; // keys the last row tile may see
    if (a->window != 0 && (uint64_t)a->window + tile_rows + 32 < longest) {
        longest = (uint64_t)a->window + tile_rows + 32;
    }
    plan_splits((uint32_t)longest, tiles * a->num_kv_heads, 1, 256, chunk_tokens, max_chunks);
    const uint64_t record_bytes = (uint64_t)a->rows * a->num_heads * a->head_dim * 4;
    const uint64_t most = record_bytes == 0 ? 1 : ((uint64_t)256 << 20) / record_bytes;
    if (*max_chunks > most) {
        const uint64_t keep = most < 1 ? 1 : most;
        const uint64_t chunk = align_up((longest + keep - 1) / keep, 32);
        *chunk_tokens = (uint32_t)chunk;
        *max_chunks = (uint32_t)((longest + chunk - 1) / chunk);
    }
}

struct PrefillSplitRecords {
    uint64_t partial, stats, total;
};

PrefillSplitRecords prefill_split_records(const zllm_gqa_prefill_args* a, uint32_t max_chunks)
{
    PrefillSplitRecords w;
    const uint64_t records = (uint64_t)a->rows * max_chunks * a->num_heads;
    w.partial = 0;
    w.stats = align_up(records * a->head_dim * 4, 256);
    w.total = w.stats + align_up(records * 8, 256);
    return w;
}

// Q8g64 caches (scales of any type) and f16 caches run the matrix-core chunk kernels, which keep all of their state on
// chip (head_dim 64 / 128 / 256, f16: 128 / 256).  What is left runs each row of the chunk as one item of the split-KV
// decode kernels (row r is a sequence of position + r + 1 tokens over the same block table): more than 128 query heads
// per KV head at head_dim 256 (a workgroup has 128 columns there), and f32 queries outside gqa_prefill_q8 (head_dim 128,
// 16-bit scales).  The chunk kernels carry a query as f16, exact for bf16 and f16 activations; an f32 query loses 13
// bits, which large logits and outlier channels turn into errors past the 2e-3 bound (measured 2.6e-3 at head_dim 256
// and 6e-3 at head_dim 64 with a doubled score scale), and the decode kernels' query is wider.  That route re-reads the
// KV bytes per row, so it is bound by the cache bandwidth rather than the matrix cores; it needs the rows' ranges and
// the split records.
static bool prefill_rows_as_decode_items(const zllm_gqa_prefill_args* a)
{
    const bool q8 = a->kv_format == ZLLM_KV_Q8G64;
    if (a->q_dtype == ZLLM_DTYPE_F32 && !(q8 && a->head_dim == 128 && a->scale_dtype != ZLLM_SCALE_F32)) {
        return true;
    }
    if (a->head_dim == 192) {
        return true; // no chunk kernel is built for three scale groups a head
    }
    return a->head_dim == 256 && a->num_heads / a->num_kv_heads > 128u;
}

static void prefill_decode_args(const zllm_gqa_prefill_args* a, zllm_gqa_decode_args* d)
{
    memset(d, 0, sizeof(*d));
    d->q = a->q;
    d->k_plane = a->k_plane;
    d->k_scales = a->k_scales;
    d->v_plane = a->v_plane;
    d->v_scales = a->v_scales;
    d->tables = a->table;
    d->batch = a->rows;
    d->num_heads = a->num_heads;
    d->num_kv_heads = a->num_kv_heads;
    d->head_dim = a->head_dim;
    d->max_kv_len = a->position + a->rows;
    const uint64_t pages = ((uint64_t)a->position + a->rows + a->block_tokens - 1) / a->block_tokens;
    d->table_stride = a->table_stride != 0 ? a->table_stride : (uint32_t)pages;
    // sum of the rows' visible lengths (an upper bound when rows carry explicit visible ends): tunes the split size
    uint64_t total = 0;
    for (uint32_t r = 0; r < a->rows; ++r) {
        const uint64_t end = (uint64_t)a->position + r + 1;
        total += a->visible_ends != nullptr ? (uint64_t)a->position + a->rows : (a->window != 0 && end > a->window ? a->window : end);
    }
    d->total_kv_tokens = total > 0xffffffffull ? 0u : (uint32_t)total;
    d->block_tokens = a->block_tokens;
    d->score_scale = a->score_scale;
    d->softcap = a->softcap;
    d->kv_format = a->kv_format;
    d->scale_dtype = a->scale_dtype;
    d->q_dtype = a->q_dtype;
    d->gate = a->gate;
    d->gate_cols = a->gate_cols;
    d->gate_dtype = a->gate_dtype;
}

// Workspace of the route that runs the chunk's rows as items of the decode kernels: the rows' ranges, then the split records
static uint64_t prefill_decode_route_bytes(const zllm_gqa_prefill_args* a)
{
    zllm_gqa_decode_args d;
    prefill_decode_args(a, &d);
    const uint64_t records = zllm_attn_gqa_decode_workspace_bytes(&d);
    return records == 0 ? 0 : align_up((uint64_t)a->rows * 8, 256) + records;
}

// A chunk of very few rows is a decode step in all but name (the reference decodes through this entry with one row,
// src/backend/rocm/attention.rs:2202-2231): the chunk kernel would run row tiles that are all but empty.  With the
// decode route's workspace such a chunk runs as decode items instead, each row re-reading the cache.  Measured on 32
// query / 8 KV heads of 128 (us, decode items against the chunk kernel with KV splits): one row over 32 K tokens 24 / 71,
// two 33 / 73, four 56 / 74, eight 104 / 78; eight rows over 2 K tokens 20 / 33 -- about 15 us + 0.34 ns per row and
// token against 28 us + 1.5 ns per token (0.8 ns with half-size row tiles).
static bool few_rows_as_decode_items(const zllm_gqa_prefill_args* a)
{
    if (a->rows > 16u) {
        return false;
    }
    uint64_t tokens = (uint64_t)a->position + a->rows;
    if (a->window != 0 && tokens > a->window) {
        tokens = a->window;
    }
    // the chunk kernel's half-size row tiles (Q8g64 with 16-bit scales at head_dim 128, a chunk whose pairs fit one) walk
    // a key in 0.8 ns: eight rows over 32 K tokens 54 us, where they would cost 104 as decode items
    const bool half_tiles = zllm::gqa_prefill_half_tiles(a->rows, a->position, a->window, a->num_heads, a->num_kv_heads, a->head_dim, a->kv_format,
                                                         a->scale_dtype, a->q_dtype);
    return (uint64_t)a->rows * tokens * 34u < tokens * (half_tiles ? 80u : 150u) + 1300000u;
}

uint64_t zllm_attn_gqa_prefill_workspace_bytes(const zllm_gqa_prefill_args* a)
{
    if (validate_gqa_prefill(a) != 0) {
        return 0;
    }
    if (prefill_rows_as_decode_items(a)) {
        return prefill_decode_route_bytes(a);
    }
    uint32_t chunk_tokens, max_chunks;
    plan_prefill_splits(a, &chunk_tokens, &max_chunks);
    const uint64_t splits = max_chunks > 1 ? prefill_split_records(a, max_chunks).total : 0; /* unsplit, the chunk kernel keeps all of its state on chip */
    const uint64_t items = few_rows_as_decode_items(a) ? prefill_decode_route_bytes(a) : 0;
    return splits > items ? splits : items;
}

int zllm_attn_gqa_prefill_chunk(const zllm_gqa_prefill_args* a, zllm_stream_t stream)
{
    const int rc = validate_gqa_prefill(a);
    if (rc != 0) {
        return rc;
    }
    if (a->q == nullptr || a->k_plane == nullptr || a->v_plane == nullptr || a->out == nullptr ||
        (a->kv_format == ZLLM_KV_Q8G64 && (a->k_scales == nullptr || a->v_scales == nullptr))) {
        return fail(-1, "GQA prefill: null pointer");
    }
    // the kernel reads codes as 8-byte vectors and scales as 4-byte words, and stores the output as 16- or 8-byte vectors
    if ((((uintptr_t)a->q | (uintptr_t)a->k_plane | (uintptr_t)a->v_plane | (uintptr_t)a->out) & 15u) != 0 ||
        (((uintptr_t)a->k_scales | (uintptr_t)a->v_scales) & 3u) != 0) {
        return fail(-1, "GQA prefill: q, cache planes and out must be 16-byte aligned (scale planes 4-byte)");
    }
    if (a->gate != nullptr &&
        ((a->gate_cols != 1 && a->gate_cols != a->num_heads * a->head_dim) || (a->gate_dtype != ZLLM_DTYPE_F32 && a->gate_dtype != ZLLM_DTYPE_BF16))) {
        return fail(-1, "GQA prefill: gate_cols=%u must be 1 or %u, gate_dtype f32 or bf16", a->gate_cols, a->num_heads * a->head_dim);
    }
    bool as_items = prefill_rows_as_decode_items(a);
    if (!as_items && few_rows_as_decode_items(a)) {
        const uint64_t need = prefill_decode_route_bytes(a);
        as_items = need != 0 && a->workspace != nullptr && a->workspace_bytes >= need && ((uintptr_t)a->workspace & 15u) == 0;
    }
    if (as_items) {
        zllm_gqa_decode_args d;
        prefill_decode_args(a, &d);
        if (validate_gqa_decode(&d) != 0) {
            return -1;
        }
        const uint64_t need = prefill_decode_route_bytes(a);
        if (a->workspace == nullptr || a->workspace_bytes < need || ((uintptr_t)a->workspace & 15u) != 0) {
            return fail(-1, "GQA prefill: this geometry needs a 16-byte aligned workspace of %llu bytes (got %llu)", (unsigned long long)need,
                        (unsigned long long)a->workspace_bytes);
        }
        uint32_t* lens = (uint32_t*)a->workspace;
        uint32_t* first = lens + a->rows;
        int rc2 = hip_status(zllm::launch_prefill_row_ranges(lens, first, a->visible_ends, a->visible_starts, a->rows, a->position, a->window, (hipStream_t)stream),
                             "GQA prefill row ranges launch");
        if (rc2 != 0) {
            return rc2;
        }
        d.kv_lens = lens;
        d.first_visible = first;
        d.out = (float*)a->out;
        const uint64_t head_bytes = align_up((uint64_t)a->rows * 8, 256);
        return gqa_decode_over(&d, (char*)a->workspace + head_bytes, a->workspace_bytes - head_bytes, stream, /*table_shared=*/true, a->out_dtype);
    }
    zllm::GqaPrefillParams p;
    memset(&p, 0, sizeof(p));
    p.visible_ends = a->visible_ends;
    p.visible_starts = a->visible_starts;
    p.q = a->q;
    p.k_plane = (const unsigned char*)a->k_plane;
    p.k_scales = (const unsigned char*)a->k_scales;
    p.v_plane = (const unsigned char*)a->v_plane;
    p.v_scales = (const unsigned char*)a->v_scales;
    p.table = a->table;
    p.out = a->out;
    p.rows = a->rows;
    p.position = a->position;
    p.window = a->window;
    p.num_heads = a->num_heads;
    p.num_kv_heads = a->num_kv_heads;
    p.head_dim = a->head_dim;
    p.group = a->num_heads / a->num_kv_heads;
    p.block_tokens = a->block_tokens;
    p.block_shift = shift_of(a->block_tokens);
    p.score_scale = a->score_scale;
    p.softcap = a->softcap;
    p.q_dtype = a->q_dtype;
    p.out_dtype = a->out_dtype;
    if (a->gate != nullptr) {
        if ((a->gate_cols != 1 && a->gate_cols != a->num_heads * a->head_dim) || (a->gate_dtype != ZLLM_DTYPE_F32 && a->gate_dtype != ZLLM_DTYPE_BF16)) {
            return fail(-1, "GQA prefill: gate_cols=%u must be 1 or %u, gate_dtype f32 or bf16", a->gate_cols, a->num_heads * a->head_dim);
        }
        p.gate = a->gate;
        p.gate_cols = a->gate_cols;
        p.gate_dtype = a->gate_dtype;
    }
    // KV splits when the chunk has too few row tiles for the device and the caller brought the room for their records
    uint32_t chunk_tokens = 0, max_chunks = 1;
    plan_prefill_splits(a, &chunk_tokens, &max_chunks);
    if (max_chunks > 1) {
        const PrefillSplitRecords w = prefill_split_records(a, max_chunks);
        if (a->workspace != nullptr && a->workspace_bytes >= w.total && ((uintptr_t)a->workspace & 15u) == 0) {
            p.partial = (float*)((char*)a->workspace + w.partial);
            p.stats = (float*)((char*)a->workspace + w.stats);
            p.chunk_tokens = chunk_tokens;
            p.max_chunks = max_chunks;
        }
    }
    const int launched = hip_status(zllm::launch_gqa_prefill(p, a->kv_format, a->scale_dtype, (hipStream_t)stream), "GQA prefill launch");
    if (launched != 0 || p.max_chunks <= 1) {
        return launched;
    }
    zllm::GqaDecodeParams m;
    memset(&m, 0, sizeof(m));
    m.out = (float*)a->out;
    m.out_dtype = a->out_dtype;
    m.partial = p.partial;
    m.stats = p.stats;
    m.batch = a->rows;
    m.num_heads = a->num_heads;
    m.head_dim = a->head_dim;
    m.chunk_tokens = chunk_tokens;
    m.max_chunks = max_chunks;
    m.fixed_chunks = max_chunks;
    m.gate = p.gate;
    m.gate_cols = p.gate_cols;
    m.gate_dtype = p.gate_dtype;
    return hip_status(zllm::launch_split_merge(m, (hipStream_t)stream), "GQA prefill split merge launch");
}

} // extern "C"

/*
 * CPU oracle for the zLLM attention hot path — TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the reference's CPU algorithms for GQA / MLA
 * attention over a Q8g64 paged KV cache.  It is the checker for the HIP path
 * and the timed "cpu_baseline" of the benchmark; the product library never
 * links, loads or calls it.
 *
 * Every function names the reference file:line it follows (paths relative to
 * the zllm-lab/zllm tree).  The reference is Rust and cannot be compiled in
 * this environment, so each function is pinned by the reference's own
 * known-answer tests (tests/test_oracle_known_answers.py) and by independent
 * float64 NumPy checks (tests/test_oracle_math.py).
 *
 * Parity status:
 *   - pinned: key_range, paged_row, layout arithmetic, ring write plan, bf16 /
 *     f16 conversions, the three Q8g64 quantizer rules, GQA head attention,
 *     MLA reference / absorbed-Q8 attention, RoPE apply; the direct-over-Q8
 *     GQA decode (the benchmark's second CPU mode) by equality with the pinned
 *     dequantise-then-f32 routine and by float64 NumPy.
 *   - parity unpinned: the attention-logit soft-cap (the reference has no such
 *     operation; defined here as s <- cap * tanh(s / cap) after the score
 *     scale), and the bit-level float summation order of the reference's SIMD
 *     `dot` (results are compared by tolerance, never bit-for-bit).
 *
 * Build: gcc -O2 -fPIC -shared -fopenmp -ffp-contract=off (see oracle/Makefile).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ZO_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ */
/* 16-bit float conversions                                                  */
/* ------------------------------------------------------------------------ */

/* src/kernel/rocm/hip/hiprtc.rs:62-67 (zllm_bf16_to_f32). */
ZO_API float zo_bf16_to_f32(uint16_t value)
{
    uint32_t bits = ((uint32_t)value) << 16;
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

/* src/kernel/rocm/hip/hiprtc.rs:69-75 (zllm_f32_to_bf16): round to nearest even
 * by adding 0x7fff + lsb; NaN is not special-cased (same as the reference). */
ZO_API uint16_t zo_f32_to_bf16(float value)
{
    uint32_t bits;
    memcpy(&bits, &value, 4);
    uint32_t rounding = 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)((bits + rounding) >> 16);
}

/* src/kernel/rocm/hip/hiprtc.rs:77-102 (zllm_f16_to_f32), subnormals included. */
ZO_API float zo_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exponent = ((uint32_t)h >> 10) & 0x1fu;
    uint32_t mantissa = (uint32_t)h & 0x03ffu;
    uint32_t value;
    if (exponent == 0) {
        if (mantissa == 0) {
            value = sign;
        } else {
            exponent = 113;
            while ((mantissa & 0x0400u) == 0) {
                mantissa <<= 1;
                --exponent;
            }
            value = sign | (exponent << 23) | ((mantissa & 0x03ffu) << 13);
        }
    } else if (exponent == 31) {
        value = sign | 0x7f800000u | (mantissa << 13);
    } else {
        value = sign | ((exponent + 112) << 23) | (mantissa << 13);
    }
    float out;
    memcpy(&out, &value, 4);
    return out;
}

/* IEEE binary32 -> binary16, round to nearest even.  This is what Metal's
 * `half(scale)` (src/kernel/metal/attention/mod.rs:123) and the `half` crate's
 * `f16::from_f32` compute. */
ZO_API uint16_t zo_f32_to_f16(float value)
{
    uint32_t x;
    memcpy(&x, &value, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 0xff) {
        return (uint16_t)(sign | 0x7c00u | (man ? (0x0200u | (man >> 13)) : 0));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 31) {
        return (uint16_t)(sign | 0x7c00u);
    }
    if (e <= 0) {
        if (e < -10) {
            return (uint16_t)sign;
        }
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) {
            half_man++;
        }
        return (uint16_t)(sign | half_man);
    }
    uint32_t half_bits = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half_bits & 1u))) {
        half_bits++;
    }
    return (uint16_t)(sign | half_bits);
}

/* src/kernel/rocm/hip/hiprtc.rs:104-116 (zllm_scale): 0 = bf16, 1 = f16, 2 = f32. */
static float zo_scale_at(const void* scales, size_t index, int scale_dtype)
{
    if (scale_dtype == 0) {
        return zo_bf16_to_f32(((const uint16_t*)scales)[index]);
    }
    if (scale_dtype == 1) {
        return zo_f16_to_f32(((const uint16_t*)scales)[index]);
    }
    return ((const float*)scales)[index];
}

/* ------------------------------------------------------------------------ */
/* Visible ranges, paging, layout arithmetic (integers, exact)              */
/* ------------------------------------------------------------------------ */

/* src/attention/gqa.rs:54-62 (CausalWindow::key_range).  window == 0 means
 * CausalWindow::Full, otherwise Sliding{size = window}. */
ZO_API void zo_key_range(uint64_t window, uint64_t query_position, uint64_t key_end,
                         uint64_t* start_out, uint64_t* end_out)
{
    uint64_t causal_end = query_position + 1;
    if (causal_end > key_end) {
        causal_end = key_end;
    }
    uint64_t start = 0;
    if (window != 0) {
        uint64_t upto = query_position + 1;
        start = upto > window ? upto - window : 0;
    }
    if (start > causal_end) {
        start = causal_end;
    }
    *start_out = start;
    *end_out = causal_end;
}

/* src/attention/gqa.rs:65-68 (key_range_with_visible_end). */
ZO_API void zo_key_range_with_visible_end(uint64_t window, uint64_t query_position, uint64_t key_end,
                                          uint64_t visible_end, uint64_t* start_out, uint64_t* end_out)
{
    uint64_t start, end;
    zo_key_range(window, query_position, key_end, &start, &end);
    uint64_t e = visible_end > end ? visible_end : end;
    if (e > key_end) {
        e = key_end;
    }
    *start_out = start;
    *end_out = e;
}

/* src/attention/gqa.rs:70-75 (cache_capacity). */
ZO_API uint64_t zo_cache_capacity(uint64_t window, uint64_t max_sequence_len)
{
    if (window == 0) {
        return max_sequence_len;
    }
    return window < max_sequence_len ? window : max_sequence_len;
}

/* src/kernel/rocm/hip/attention/paged_mla/source.hip:46-54 (paged_row). */
ZO_API uint64_t zo_paged_row(const uint32_t* block_table, uint32_t token, uint32_t block_size)
{
    if (block_table == NULL) {
        return token;
    }
    return (uint64_t)block_table[token / block_size] * block_size + token % block_size;
}

/* src/kv_cache/mod.rs:570-585 (KvCacheSpec::bytes_per_token) and :121-163
 * (MlaRecordLayout).  kind 0 = MLA (a = kv_lora_rank, b = qk_rope_head_dim),
 * kind 1 = GQA (a = num_kv_heads, b = head_dim).  Returns 0 on invalid input. */
ZO_API uint64_t zo_bytes_per_token(int kind, uint64_t a, uint64_t b, uint64_t group)
{
    if (kind == 0) {
        if (a == 0 || b == 0 || group == 0 || a % group != 0) {
            return 0;
        }
        return a + (a / group) * 2 + b * 2;
    }
    if (group == 0 || b % group != 0) {
        return 0;
    }
    uint64_t columns = a * b;
    uint64_t groups = a * (b / group);
    return columns * 2 + groups * 4;
}

/* src/kv_cache/mod.rs:179-331 (KvCacheLayout::new and the layer_* offsets),
 * Int8 format.  For MLA writes {base, codes, scales, rope}; for GQA writes
 * {base, key codes, key scales, value codes, value scales}.  Returns
 * total_bytes (0 on invalid input). */
ZO_API uint64_t zo_layout_offsets(int kind, uint64_t a, uint64_t b, uint64_t group,
                                  uint64_t layer_count, uint64_t capacity, uint64_t layer,
                                  uint64_t* offsets)
{
    uint64_t per_token = zo_bytes_per_token(kind, a, b, group);
    if (per_token == 0 || capacity == 0 || layer_count == 0 || layer >= layer_count) {
        return 0;
    }
    uint64_t layer_stride = capacity * per_token;
    uint64_t base = layer * layer_stride;
    offsets[0] = base;
    if (kind == 0) {
        offsets[1] = base;                                    /* layer_codes_offset  :246-252 */
        offsets[2] = base + capacity * a;                     /* layer_scales_offset :254-261 */
        offsets[3] = base + capacity * (a + (a / group) * 2); /* layer_rope_offset   :263-271 */
    } else {
        uint64_t columns = a * b;
        uint64_t groups = a * (b / group);
        offsets[1] = base;                                              /* :290-293 */
        offsets[2] = base + capacity * columns;                         /* :295-302 */
        offsets[3] = base + capacity * columns + capacity * groups * 2; /* :304-313 */
        offsets[4] = offsets[3] + capacity * columns;                   /* :315-322 */
    }
    return layer_count * layer_stride;
}

/* src/kv_cache/mod.rs:440-455 (HybridGqaCacheLayout::write_plan).  out =
 * {end, source_start, token_count, first_slot, first_count, second_count}.
 * Returns 0 on success, -1 on the reference's error cases. */
ZO_API int zo_ring_write_plan(uint64_t capacity, uint64_t max_sequence_len, uint64_t position,
                              uint64_t count, uint64_t* out)
{
    if (count == 0 || capacity == 0) {
        return -1;
    }
    uint64_t end = position + count;
    if (end > max_sequence_len) {
        return -1;
    }
    uint64_t evicted_before = end > capacity ? end - capacity : 0;
    uint64_t write_start = position > evicted_before ? position : evicted_before;
    uint64_t token_count = end - write_start;
    uint64_t first_slot = write_start % capacity;
    uint64_t first_count = token_count < capacity - first_slot ? token_count : capacity - first_slot;
    out[0] = end;
    out[1] = write_start - position;
    out[2] = token_count;
    out[3] = first_slot;
    out[4] = first_count;
    out[5] = token_count - first_count;
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Q8g64 quantization (three conventions) and paged scatter / gather        */
/* ------------------------------------------------------------------------ */

enum {
    ZO_RULE_ROCM_MLA = 0,  /* bf16 scale, codes divide by the ROUNDED scale */
    ZO_RULE_METAL_GQA = 1, /* f16 scale, codes multiply by 1/UNROUNDED scale */
    ZO_RULE_CUDA_GQA = 2   /* f32 scale, codes multiply by 1/scale          */
};

static float zo_clamp127(float v)
{
    return fmaxf(-127.0f, fminf(127.0f, v));
}

/* Quantize one group of `group` contiguous f32 values.
 *  rule 0: src/kernel/rocm/hip/attention/paged_mla/source.hip:183-201
 *          scale = absmax == 0 ? 1 : absmax * (1/127); stored = bf16(scale);
 *          code = clamp(nearbyint(x / f32(stored)), +-127).
 *  rule 1: src/kernel/metal/attention/mod.rs:114-127
 *          scale = absmax > 0 ? absmax / 127 : 1; stored = half(scale);
 *          code = clamp(rint(x * (1 / scale)), +-127).
 *  rule 2: src/kernel/cuda/attention.rs:331-341 — as rule 1, stored = f32. */
static void zo_quantize_group(int rule, const float* x, size_t group, int8_t* codes, void* scale_slot)
{
    float maximum = 0.0f;
    for (size_t i = 0; i < group; ++i) {
        maximum = fmaxf(maximum, fabsf(x[i]));
    }
    if (rule == ZO_RULE_ROCM_MLA) {
        const float reciprocal_127 = 1.0f / 127.0f;
        float scale = maximum == 0.0f ? 1.0f : maximum * reciprocal_127;
        uint16_t encoded = zo_f32_to_bf16(scale);
        *(uint16_t*)scale_slot = encoded;
        float quant_scale = zo_bf16_to_f32(encoded);
        for (size_t i = 0; i < group; ++i) {
            codes[i] = (int8_t)zo_clamp127(nearbyintf(x[i] / quant_scale));
        }
        return;
    }
    float scale = maximum > 0.0f ? maximum / 127.0f : 1.0f;
    if (rule == ZO_RULE_METAL_GQA) {
        *(uint16_t*)scale_slot = zo_f32_to_f16(scale);
    } else {
        *(float*)scale_slot = scale;
    }
    float inverse = 1.0f / scale;
    for (size_t i = 0; i < group; ++i) {
        codes[i] = (int8_t)zo_clamp127(rintf(x[i] * inverse));
    }
}

/* Quantize `rows` rows of `cols` f32 values and scatter them through the
 * block table: physical row = paged_row(table, position + row, block_size);
 * codes[phys * cols + col], scales[phys * groups + g]
 * (src/kernel/rocm/hip/attention/paged_mla/source.hip:164-202).  ring_capacity
 * > 0 first maps the logical token to `token % ring_capacity`
 * (src/kernel/cuda/attention.rs:82-88, src/kv_cache/mod.rs:528-535). */
ZO_API int zo_q8g64_append_paged(int rule, const float* input, int8_t* codes, void* scales,
                                 const uint32_t* block_table, uint64_t position, uint64_t rows,
                                 uint64_t cols, uint64_t group, uint32_t block_size,
                                 uint64_t ring_capacity)
{
    if (group == 0 || cols == 0 || cols % group != 0 || block_size == 0) {
        return -1;
    }
    size_t groups = cols / group;
    size_t scale_bytes = rule == ZO_RULE_CUDA_GQA ? 4 : 2;
    for (uint64_t row = 0; row < rows; ++row) {
        uint64_t token = position + row;
        if (ring_capacity != 0) {
            token %= ring_capacity;
        }
        uint64_t phys = zo_paged_row(block_table, (uint32_t)token, block_size);
        for (size_t g = 0; g < groups; ++g) {
            zo_quantize_group(rule, input + row * cols + g * group, group,
                              codes + phys * cols + g * group,
                              (uint8_t*)scales + (phys * groups + g) * scale_bytes);
        }
    }
    return 0;
}

/* f32 -> bf16 / f16 scatter through the table
 * (src/kernel/rocm/hip/attention/paged_mla/source.hip:146-162 for bf16;
 * f16 is the CUDA backend's unquantized KV, src/kernel/cuda/attention.rs:82-88).
 * dtype 0 = bf16, 1 = f16. */
ZO_API int zo_half_append_paged(int dtype, const float* input, uint16_t* cache,
                                const uint32_t* block_table, uint64_t position, uint64_t rows,
                                uint64_t cols, uint32_t block_size, uint64_t ring_capacity)
{
    if (cols == 0 || block_size == 0) {
        return -1;
    }
    for (uint64_t row = 0; row < rows; ++row) {
        uint64_t token = position + row;
        if (ring_capacity != 0) {
            token %= ring_capacity;
        }
        uint64_t phys = zo_paged_row(block_table, (uint32_t)token, block_size);
        for (uint64_t c = 0; c < cols; ++c) {
            float v = input[row * cols + c];
            cache[phys * cols + c] = dtype == 0 ? zo_f32_to_bf16(v) : zo_f32_to_f16(v);
        }
    }
    return 0;
}

/* Gather logical tokens [first, first + count) through the table and
 * dequantize to dense f32 rows: x = f32(code) * f32(stored scale)
 * (src/kernel/rocm/hip/attention/paged_mla/source.hip:3704-3719,
 * src/kernel/cuda/attention.rs:391).  format 0 = Q8 codes + scales,
 * 1 = f16 values, 2 = bf16 values. */
ZO_API int zo_gather_dequant_rows(int format, const void* plane, const void* scales, int scale_dtype,
                                  const uint32_t* block_table, uint32_t block_size,
                                  uint64_t ring_capacity, uint64_t first, uint64_t count,
                                  uint64_t cols, uint64_t group, float* out)
{
    if (cols == 0 || block_size == 0 || (format == 0 && (group == 0 || cols % group != 0))) {
        return -1;
    }
    size_t groups = format == 0 ? cols / group : 0;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < (int64_t)count; ++r) {
        uint64_t token = first + (uint64_t)r;
        if (ring_capacity != 0) {
            token %= ring_capacity;
        }
        uint64_t phys = zo_paged_row(block_table, (uint32_t)token, block_size);
        float* dst = out + (size_t)r * cols;
        if (format == 0) {
            const int8_t* src = (const int8_t*)plane + phys * cols;
            for (uint64_t c = 0; c < cols; ++c) {
                dst[c] = (float)src[c] * zo_scale_at(scales, phys * groups + c / group, scale_dtype);
            }
        } else {
            const uint16_t* src = (const uint16_t*)plane + phys * cols;
            for (uint64_t c = 0; c < cols; ++c) {
                dst[c] = format == 1 ? zo_f16_to_f32(src[c]) : zo_bf16_to_f32(src[c]);
            }
        }
    }
    return 0;
}

/* Raw byte gather of plane rows (bit-exact page/index gathering check). */
ZO_API int zo_gather_rows_bytes(const uint8_t* plane, const uint32_t* block_table, uint32_t block_size,
                                uint64_t ring_capacity, uint64_t first, uint64_t count,
                                uint64_t row_bytes, uint8_t* out)
{
    if (block_size == 0) {
        return -1;
    }
    for (uint64_t r = 0; r < count; ++r) {
        uint64_t token = first + r;
        if (ring_capacity != 0) {
            token %= ring_capacity;
        }
        uint64_t phys = zo_paged_row(block_table, (uint32_t)token, block_size);
        memcpy(out + r * row_bytes, plane + phys * row_bytes, row_bytes);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* GQA attention (f32 reference math)                                       */
/* ------------------------------------------------------------------------ */

/* src/kernel/cpu/matmul.rs:114-131 (dot): eight strided partial sums with a
 * fused multiply-add, a horizontal add, then a scalar tail.  The horizontal
 * order of `wide::f32x8::reduce_add` is not reproduced bit-for-bit. */
static float zo_dot8(const float* a, const float* b, size_t n)
{
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t full = n / 8 * 8;
    for (size_t i = 0; i < full; i += 8) {
        for (size_t l = 0; l < 8; ++l) {
            acc[l] = fmaf(a[i + l], b[i + l], acc[l]);
        }
    }
    float tail = 0.0f;
    for (size_t i = full; i < n; ++i) {
        tail += a[i] * b[i];
    }
    float lo = (acc[0] + acc[4]) + (acc[2] + acc[6]);
    float hi = (acc[1] + acc[5]) + (acc[3] + acc[7]);
    return (lo + hi) + tail;
}

/* src/attention/gqa.rs:172-213 (causal_head_range_f32): two-pass softmax,
 * probabilities normalised before the weighted sum, zero output when the
 * denominator is zero or non-finite.  `softcap` > 0 applies
 * s <- softcap * tanh(s / softcap) after the score scale (build extension;
 * parity unpinned, the reference has no logit soft-cap).
 * Returns 0, or -1 for the reference's invalid-argument cases. */
ZO_API int zo_gqa_head_range_f32(const float* query, const float* key, const float* value,
                                 size_t head_dim, size_t kv_stride, size_t range_start,
                                 size_t range_end, float score_scale, float softcap,
                                 float* output, float* scratch_scores)
{
    if (head_dim == 0 || range_start >= range_end || kv_stride < head_dim ||
        !isfinite(score_scale) || score_scale <= 0.0f) {
        return -1;
    }
    size_t count = range_end - range_start;
    float* scores = scratch_scores ? scratch_scores : (float*)malloc(count * sizeof(float));
    float maximum = -INFINITY;
    for (size_t i = 0; i < count; ++i) {
        size_t source = range_start + i;
        float score = zo_dot8(query, key + source * kv_stride, head_dim) * score_scale;
        if (softcap > 0.0f) {
            score = softcap * tanhf(score / softcap);
        }
        maximum = fmaxf(maximum, score);
        scores[i] = score;
    }
    float denominator = 0.0f;
    for (size_t i = 0; i < count; ++i) {
        scores[i] = expf(scores[i] - maximum);
        denominator += scores[i];
    }
    for (size_t c = 0; c < head_dim; ++c) {
        output[c] = 0.0f;
    }
    if (isfinite(denominator) && denominator != 0.0f) {
        for (size_t i = 0; i < count; ++i) {
            float probability = scores[i] / denominator;
            const float* v = value + (range_start + i) * kv_stride;
            for (size_t c = 0; c < head_dim; ++c) {
                output[c] += probability * v[c];
            }
        }
    }
    if (!scratch_scores) {
        free(scores);
    }
    return 0;
}

/* src/attention/gqa.rs:243-282 (prefill_attention_at_visible_with_dot_f32)
 * driven the way src/kernel/cpu/gqa.rs:14-21 drives it.  One task per
 * (token, head) as the reference's rayon `par_chunks_mut(head_dim)` (:269).
 * key/value hold rows [kv_start, kv_end) as dense f32 [rows, kv_heads*head_dim].
 * visible_ends may be NULL.  An empty visible range is an error in the
 * reference (causal_head_range_f32 rejects it); here the row is zero-filled
 * and -2 is returned after the loop so callers can detect it. */
ZO_API int zo_gqa_prefill_at_visible_f32(const float* query, const float* key, const float* value,
                                         uint64_t query_tokens, uint64_t kv_start, uint64_t kv_end,
                                         uint64_t position, uint64_t num_heads, uint64_t num_kv_heads,
                                         uint64_t head_dim, uint64_t window, float score_scale,
                                         float softcap, const uint32_t* visible_ends, float* output)
{
    if (num_heads == 0 || num_kv_heads == 0 || head_dim == 0 || num_heads % num_kv_heads != 0) {
        return -1;
    }
    uint64_t query_cols = num_heads * head_dim;
    uint64_t kv_cols = num_kv_heads * head_dim;
    uint64_t group = num_heads / num_kv_heads;
    int64_t tasks = (int64_t)(query_tokens * num_heads);
    int status = 0;
#pragma omp parallel
    {
        float* scratch = (float*)malloc((size_t)(kv_end - kv_start + 1) * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (int64_t item = 0; item < tasks; ++item) {
            uint64_t token = (uint64_t)item / num_heads;
            uint64_t head = (uint64_t)item % num_heads;
            uint64_t kv_head = head / group;
            uint64_t start, end;
            if (visible_ends) {
                zo_key_range_with_visible_end(window, position + token, kv_end, visible_ends[token], &start, &end);
            } else {
                zo_key_range(window, position + token, kv_end, &start, &end);
            }
            if (start < kv_start) {
                start = kv_start;
            }
            float* out = output + token * query_cols + head * head_dim;
            int rc = -1;
            if (start < end) {
                rc = zo_gqa_head_range_f32(query + token * query_cols + head * head_dim,
                                           key + kv_head * head_dim, value + kv_head * head_dim,
                                           head_dim, kv_cols, start - kv_start, end - kv_start,
                                           score_scale, softcap, out, scratch);
            }
            if (rc != 0) {
                for (uint64_t c = 0; c < head_dim; ++c) {
                    out[c] = 0.0f;
                }
#pragma omp atomic write
                status = -2;
            }
        }
        free(scratch);
    }
    return status;
}

/* The reference's second CPU mode, applied to a GQA cache: attention straight over the Q8g64 rows, values formed as
 * (float)code * scale on the fly and nothing materialised in f32, the way absorbed_attention_row_q8_scalar works over
 * the Q8 latent (src/kernel/cpu/mla.rs:771-829: score pass over the codes, two-pass softmax, weighted sum over the
 * codes again).  One task per (sequence, head).  k_codes / v_codes are dense rows [len, kv_heads * head_dim] of one
 * sequence, scales [len, kv_heads * head_dim / 64] in `scale_dtype`; the last row's query sees [first, len).
 * Same arithmetic as zo_gqa_prefill_at_visible_f32 over the dequantised rows up to the order of the dot product's
 * partial sums (sequential here, eight lanes there). */
ZO_API int zo_gqa_decode_q8_direct(const float* query, const int8_t* k_codes, const void* k_scales, const int8_t* v_codes,
                                   const void* v_scales, int scale_dtype, uint64_t first, uint64_t len, uint64_t num_heads,
                                   uint64_t num_kv_heads, uint64_t head_dim, float score_scale, float softcap, float* output)
{
    if (num_heads == 0 || num_kv_heads == 0 || head_dim == 0 || head_dim % 64 != 0 || num_heads % num_kv_heads != 0 ||
        !isfinite(score_scale) || score_scale <= 0.0f) {
        return -1;
    }
    uint64_t cols = num_kv_heads * head_dim, groups = cols / 64, group = num_heads / num_kv_heads;
    uint64_t count = len > first ? len - first : 0;
#pragma omp parallel
    {
        float* scores = (float*)malloc((size_t)(count + 1) * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (int64_t head = 0; head < (int64_t)num_heads; ++head) {
            uint64_t kv_head = (uint64_t)head / group;
            const float* q = query + (uint64_t)head * head_dim;
            float* out = output + (uint64_t)head * head_dim;
            float maximum = -INFINITY;
            for (uint64_t i = 0; i < count; ++i) {
                uint64_t t = first + i;
                const int8_t* row = k_codes + t * cols + kv_head * head_dim;
                float score = 0.0f;
                for (uint64_t g = 0; g < head_dim / 64; ++g) {
                    float scale = zo_scale_at(k_scales, t * groups + kv_head * (head_dim / 64) + g, scale_dtype);
                    for (uint64_t c = 0; c < 64; ++c) {
                        score += q[g * 64 + c] * ((float)row[g * 64 + c] * scale);
                    }
                }
                score *= score_scale;
                if (softcap > 0.0f) {
                    score = softcap * tanhf(score / softcap);
                }
                maximum = fmaxf(maximum, score);
                scores[i] = score;
            }
            float denominator = 0.0f;
            for (uint64_t i = 0; i < count; ++i) {
                scores[i] = expf(scores[i] - maximum);
                denominator += scores[i];
            }
            for (uint64_t c = 0; c < head_dim; ++c) {
                out[c] = 0.0f;
            }
            if (count != 0 && isfinite(denominator) && denominator != 0.0f) {
                for (uint64_t i = 0; i < count; ++i) {
                    uint64_t t = first + i;
                    float probability = scores[i] / denominator;
                    const int8_t* row = v_codes + t * cols + kv_head * head_dim;
                    for (uint64_t g = 0; g < head_dim / 64; ++g) {
                        float scale = zo_scale_at(v_scales, t * groups + kv_head * (head_dim / 64) + g, scale_dtype);
                        for (uint64_t c = 0; c < 64; ++c) {
                            out[g * 64 + c] += probability * ((float)row[g * 64 + c] * scale);
                        }
                    }
                }
            }
        }
        free(scores);
    }
    return 0;
}

/* src/attention/block.rs:67-119 (attention_f32): explicit per-row visible
 * ranges [visible[2r], visible[2r+1]); same math as the GQA head routine. */
ZO_API int zo_block_attention_f32(const float* query, const float* key, const float* value,
                                  uint64_t query_rows, uint64_t kv_rows, uint64_t num_heads,
                                  uint64_t num_kv_heads, uint64_t head_dim, float score_scale,
                                  const uint32_t* visible, float* output)
{
    if (num_heads == 0 || num_kv_heads == 0 || head_dim == 0 || num_heads % num_kv_heads != 0 ||
        !isfinite(score_scale) || score_scale <= 0.0f) {
        return -1;
    }
    for (uint64_t r = 0; r < query_rows; ++r) {
        if (visible[2 * r] >= visible[2 * r + 1] || visible[2 * r + 1] > kv_rows) {
            return -1; /* block.rs:31-35 */
        }
    }
    uint64_t query_cols = num_heads * head_dim;
    uint64_t kv_cols = num_kv_heads * head_dim;
    uint64_t group = num_heads / num_kv_heads;
    int64_t tasks = (int64_t)(query_rows * num_heads);
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t item = 0; item < tasks; ++item) {
        uint64_t row = (uint64_t)item / num_heads;
        uint64_t head = (uint64_t)item % num_heads;
        uint64_t kv_head = head / group;
        zo_gqa_head_range_f32(query + row * query_cols + head * head_dim, key + kv_head * head_dim,
                              value + kv_head * head_dim, head_dim, kv_cols, visible[2 * row],
                              visible[2 * row + 1], score_scale, 0.0f,
                              output + row * query_cols + head * head_dim, NULL);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* RoPE                                                                      */
/* ------------------------------------------------------------------------ */

/* src/attention/rope.rs:120-164 (apply_f32).  layout 0 = SplitHalf,
 * 1 = Interleaved; placement 0 = Prefix, 1 = Suffix.  In place on `data`.
 * Compiled with -ffp-contract=off: the two products and the add/sub are
 * separately rounded, as in the Rust source. */
ZO_API int zo_rope_apply_f32(float* data, uint64_t rows, uint64_t columns, uint64_t head_count,
                             uint64_t rotary_dim, uint64_t position, const float* cosine,
                             const float* sine, uint64_t table_len, int layout, int placement)
{
    if (head_count == 0 || rotary_dim == 0 || rotary_dim % 2 != 0 || columns % head_count != 0) {
        return -1;
    }
    uint64_t head_dim = columns / head_count;
    if (rotary_dim > head_dim) {
        return -1;
    }
    uint64_t half = rotary_dim / 2;
    if ((position + rows) * half > table_len) {
        return -1;
    }
    for (uint64_t row = 0; row < rows; ++row) {
        const float* cos_row = cosine + (position + row) * half;
        const float* sin_row = sine + (position + row) * half;
        for (uint64_t head = 0; head < head_count; ++head) {
            uint64_t head_start = row * columns + head * head_dim;
            uint64_t start = placement == 0 ? head_start : head_start + head_dim - rotary_dim;
            for (uint64_t pair = 0; pair < half; ++pair) {
                uint64_t ri = layout == 0 ? pair : pair * 2;
                uint64_t ii = layout == 0 ? half + pair : pair * 2 + 1;
                float real = data[start + ri];
                float imaginary = data[start + ii];
                data[start + ri] = real * cos_row[pair] - imaginary * sin_row[pair];
                data[start + ii] = imaginary * cos_row[pair] + real * sin_row[pair];
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Per-head RMSNorm and the sigmoid output gate                               */
/* ------------------------------------------------------------------------ */

/* src/kernel/cpu/vae.rs:297-334 (rmsnorm_heads_with), reached from
 * gemma_rmsnorm_heads / rmsnorm_heads (src/backend/cpu/attention.rs:365-371,
 * 463-470): out = x * (1 / sqrt(sum(x^2) / head_dim + eps)) * (weight + offset),
 * offset 1 for the Gemma form, 0 for the plain form; weight NULL = no weight.
 * The sum of squares runs over eight lane accumulators (element e feeds lane
 * e % 8, chunks in ascending order) that are then added as the `wide` crate's
 * f32x8::reduce_add does on AVX -- lanes (l, l + 4), then (0, 2) and (1, 3),
 * then the two halves -- followed by the tail elements in order.  PARITY
 * UNPINNED at bit level: `wide` is a third-party dependency (not vendored) and
 * its reduction order is taken from its published source; the reference's own
 * tests (src/kernel/cpu/rmsnorm.rs:70-103) hold to 1e-6 / 1e-5 only. */
ZO_API int zo_rmsnorm_heads_f32(const float* input, uint64_t rows, uint64_t head_count, uint64_t head_dim,
                                const float* weight, float eps, float weight_offset, float* out)
{
    if (head_count == 0 || head_dim == 0 || (weight != NULL && (!isfinite(eps) || eps <= 0.0f))) {
        return -1;
    }
    uint64_t lanes = head_dim / 8 * 8;
    for (uint64_t unit = 0; unit < rows * head_count; ++unit) {
        const float* source = input + unit * head_dim;
        float* target = out + unit * head_dim;
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (uint64_t c = 0; c < lanes; c += 8) {
            for (int l = 0; l < 8; ++l) {
                acc[l] += source[c + l] * source[c + l];
            }
        }
        float sum = ((acc[0] + acc[4]) + (acc[2] + acc[6])) + ((acc[1] + acc[5]) + (acc[3] + acc[7]));
        for (uint64_t c = lanes; c < head_dim; ++c) {
            sum += source[c] * source[c];
        }
        float inverse = 1.0f / sqrtf(sum / (float)head_dim + eps);
        for (uint64_t c = 0; c < head_dim; ++c) {
            target[c] = weight != NULL ? source[c] * inverse * (weight[c] + weight_offset) : source[c] * inverse;
        }
    }
    return 0;
}

/* src/backend/cpu/context.rs:419-432 (sigmoid_gate): out = input / (1 + exp(-gate)),
 * one gate per element or one per row (gate_cols == 1). */
ZO_API int zo_sigmoid_gate_f32(const float* input, const float* gate, uint64_t rows, uint64_t cols, uint64_t gate_cols,
                               float* out)
{
    if (gate_cols != 1 && gate_cols != cols) {
        return -1;
    }
    for (uint64_t row = 0; row < rows; ++row) {
        for (uint64_t c = 0; c < cols; ++c) {
            float value = gate[row * gate_cols + (gate_cols == 1 ? 0 : c)];
            out[row * cols + c] = input[row * cols + c] * (1.0f / (1.0f + expf(-value)));
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* MLA attention                                                             */
/* ------------------------------------------------------------------------ */

typedef struct {
    uint64_t kv_lora_rank;
    uint64_t qk_rope_head_dim;
    uint64_t q_projection_size;
    uint64_t kv_projection_size;
    uint64_t num_heads;
} zo_mla_spec;

static float zo_dot_seq(const float* a, const float* b, size_t n)
{
    float s = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        s += a[i] * b[i];
    }
    return s;
}

/* src/attention/mla.rs:73-138 (reference_attention): non-absorbed MLA for one
 * query row over `count` selected rows of projected KV.  Output has
 * q_projection_size entries; only the first value_dim of each head slot are
 * written (:134). */
ZO_API int zo_mla_reference_attention(const float* query, const float* projected_kv,
                                      const float* rope_cache, uint64_t rope_rows,
                                      const uint64_t* rope_indices, uint64_t count,
                                      const zo_mla_spec* spec, float* output)
{
    uint64_t heads = spec->num_heads;
    if (heads == 0 || spec->q_projection_size % heads != 0 || spec->kv_projection_size % heads != 0 || count == 0) {
        return -1;
    }
    uint64_t q_head_dim = spec->q_projection_size / heads;
    uint64_t rope_dim = spec->qk_rope_head_dim;
    if (rope_dim > q_head_dim) {
        return -1;
    }
    uint64_t nope = q_head_dim - rope_dim;
    uint64_t kv_head_dim = spec->kv_projection_size / heads;
    if (nope > kv_head_dim) {
        return -1;
    }
    for (uint64_t i = 0; i < count; ++i) {
        if (rope_dim != 0 && rope_indices[i] >= rope_rows) {
            return -1;
        }
    }
    uint64_t value_dim = kv_head_dim - nope;
    float scale = 1.0f / sqrtf((float)q_head_dim);
    memset(output, 0, spec->q_projection_size * sizeof(float));
    float* scores = (float*)malloc(count * sizeof(float));
    for (uint64_t head = 0; head < heads; ++head) {
        const float* q_nope = query + head * q_head_dim;
        const float* q_rope = q_nope + nope;
        float maximum = -INFINITY;
        for (uint64_t s = 0; s < count; ++s) {
            const float* k_nope = projected_kv + s * spec->kv_projection_size + head * kv_head_dim;
            const float* k_rope = rope_cache + rope_indices[s] * rope_dim;
            float score = (zo_dot_seq(q_nope, k_nope, nope) + zo_dot_seq(q_rope, k_rope, rope_dim)) * scale;
            maximum = fmaxf(maximum, score);
            scores[s] = score;
        }
        float denominator = 0.0f;
        for (uint64_t s = 0; s < count; ++s) {
            scores[s] = expf(scores[s] - maximum);
            denominator += scores[s];
        }
        for (uint64_t v = 0; v < value_dim; ++v) {
            float sum = 0.0f;
            for (uint64_t s = 0; s < count; ++s) {
                sum += scores[s] / denominator *
                       projected_kv[s * spec->kv_projection_size + head * kv_head_dim + nope + v];
            }
            output[head * q_head_dim + v] = sum;
        }
    }
    free(scores);
    return 0;
}

/* src/kernel/cpu/mla.rs:582-686 (mla_attention_selected_bf16_history), scalar
 * arm: bf16 query / projected KV / rope, f32 math, compact bf16 output
 * [rows, heads * value_dim].  selection may be NULL (causal prefix). */
ZO_API int zo_mla_selected_bf16_history(const zo_mla_spec* spec, const uint16_t* query,
                                        uint64_t query_rows, uint64_t query_start,
                                        const uint16_t* projected_kv, const uint16_t* rope,
                                        uint64_t history_rows, const uint32_t* selection,
                                        uint64_t width, uint16_t* output)
{
    uint64_t heads = spec->num_heads;
    uint64_t q_head_dim = spec->q_projection_size / heads;
    uint64_t rope_dim = spec->qk_rope_head_dim;
    uint64_t nope = q_head_dim - rope_dim;
    uint64_t kv_head_dim = spec->kv_projection_size / heads;
    uint64_t value_dim = kv_head_dim - nope;
    uint64_t output_cols = heads * value_dim;
    if (query_rows == 0 || query_start + query_rows != history_rows) {
        return -1;
    }
    float scale = 1.0f / sqrtf((float)q_head_dim);
    for (uint64_t row = 0; row < query_rows; ++row) {
        uint64_t valid_rows = query_start + row + 1;
        const uint32_t* selected = selection ? selection + row * width : NULL;
        uint64_t count = selected ? width : valid_rows;
        float* scores = (float*)malloc(count * sizeof(float));
        for (uint64_t head = 0; head < heads; ++head) {
            const uint16_t* q = query + row * spec->q_projection_size + head * q_head_dim;
            float maximum = -INFINITY;
            for (uint64_t slot = 0; slot < count; ++slot) {
                uint64_t token = selected ? selected[slot] : slot;
                if (token >= valid_rows) {
                    free(scores);
                    return -1;
                }
                uint64_t kv_base = token * spec->kv_projection_size + head * kv_head_dim;
                float score = 0.0f;
                for (uint64_t c = 0; c < nope; ++c) {
                    score += zo_bf16_to_f32(q[c]) * zo_bf16_to_f32(projected_kv[kv_base + c]);
                }
                for (uint64_t c = 0; c < rope_dim; ++c) {
                    score += zo_bf16_to_f32(q[nope + c]) * zo_bf16_to_f32(rope[token * rope_dim + c]);
                }
                score *= scale;
                maximum = fmaxf(maximum, score);
                scores[slot] = score;
            }
            float denominator = 0.0f;
            for (uint64_t slot = 0; slot < count; ++slot) {
                scores[slot] = expf(scores[slot] - maximum);
                denominator += scores[slot];
            }
            for (uint64_t v = 0; v < value_dim; ++v) {
                float sum = 0.0f;
                for (uint64_t slot = 0; slot < count; ++slot) {
                    uint64_t token = selected ? selected[slot] : slot;
                    sum += scores[slot] *
                           zo_bf16_to_f32(projected_kv[token * spec->kv_projection_size + head * kv_head_dim + nope + v]);
                }
                output[row * output_cols + head * value_dim + v] = zo_f32_to_bf16(sum / denominator);
            }
        }
        free(scores);
    }
    return 0;
}

/* src/kernel/cpu/mla.rs:958-1076 (mla_attention_absorbed_q8_history) with the
 * scalar row kernel :771-829 (absorbed_attention_row_q8_scalar).
 *   (1) absorbed[h] = q_nope[h] . W_kv_b[h, 0:nope, :]  -> rounded to bf16 (:1037)
 *   (2) per head / token: s = (sum bf16(absorbed) * (code * scale)
 *                               + sum bf16(q_rope) * bf16(rope)) / sqrt(q_head_dim),
 *       two-pass softmax, weighted[h] = sum (p / den) * (code * scale)   (f32)
 *   (3) out[h, v] = weighted[h] . W_kv_b[h, nope + v, :]  -> bf16 (:1071)
 * Scales are decoded as bf16 (:1021).  History is dense (rows 0..history_rows);
 * a paged cache is gathered first.  Optional outputs: out_bf16
 * [rows, heads*value_dim], out_f32 (same shape, before the final rounding),
 * weighted_f32 [rows, heads*latent].  selection may be NULL. */
ZO_API int zo_mla_absorbed_q8_history(const zo_mla_spec* spec, const uint16_t* query,
                                      uint64_t query_rows, uint64_t query_start,
                                      const uint8_t* latent_codes, const uint16_t* latent_scales,
                                      uint64_t latent_group_size, const uint16_t* rope,
                                      uint64_t history_rows, const float* kv_b,
                                      const uint32_t* selection, uint64_t width,
                                      uint16_t* out_bf16, float* out_f32, float* weighted_f32)
{
    uint64_t heads = spec->num_heads;
    uint64_t latent_dim = spec->kv_lora_rank;
    uint64_t rope_dim = spec->qk_rope_head_dim;
    if (heads == 0 || latent_group_size == 0 || latent_dim % latent_group_size != 0 || query_rows == 0 ||
        query_start + query_rows != history_rows) {
        return -1;
    }
    uint64_t q_head_dim = spec->q_projection_size / heads;
    uint64_t nope = q_head_dim - rope_dim;
    uint64_t kv_head_dim = spec->kv_projection_size / heads;
    uint64_t value_dim = kv_head_dim - nope;
    uint64_t groups = latent_dim / latent_group_size;
    if (selection) {
        for (uint64_t row = 0; row < query_rows; ++row) {
            for (uint64_t s = 0; s < width; ++s) {
                if (selection[row * width + s] >= query_start + row + 1) {
                    return -1;
                }
            }
        }
    }
    float scale = 1.0f / sqrtf((float)q_head_dim);
    int64_t tasks = (int64_t)(query_rows * heads);
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t item = 0; item < tasks; ++item) {
        uint64_t row = (uint64_t)item / heads;
        uint64_t head = (uint64_t)item % heads;
        const uint16_t* q = query + row * spec->q_projection_size + head * q_head_dim;
        /* (1) absorb, matmul_nn (:712-728): out[c] = sum_k q_nope[k] * W[k, c]. */
        float* absorbed = (float*)calloc(latent_dim, sizeof(float));
        const float* w_k = kv_b + head * kv_head_dim * latent_dim;
        for (uint64_t k = 0; k < nope; ++k) {
            float qk = zo_bf16_to_f32(q[k]);
            for (uint64_t c = 0; c < latent_dim; ++c) {
                absorbed[c] += qk * w_k[k * latent_dim + c];
            }
        }
        for (uint64_t c = 0; c < latent_dim; ++c) {
            absorbed[c] = zo_bf16_to_f32(zo_f32_to_bf16(absorbed[c]));
        }
        /* (2) attention over the Q8 history. */
        const uint32_t* selected = selection ? selection + row * width : NULL;
        uint64_t count = selected ? width : query_start + row + 1;
        float* scores = (float*)malloc(count * sizeof(float));
        float maximum = -INFINITY;
        for (uint64_t slot = 0; slot < count; ++slot) {
            uint64_t token = selected ? selected[slot] : slot;
            float score = 0.0f;
            for (uint64_t c = 0; c < latent_dim; ++c) {
                float value = (float)(int8_t)latent_codes[token * latent_dim + c] *
                              zo_bf16_to_f32(latent_scales[token * groups + c / latent_group_size]);
                score += absorbed[c] * value;
            }
            for (uint64_t c = 0; c < rope_dim; ++c) {
                score += zo_bf16_to_f32(q[nope + c]) * zo_bf16_to_f32(rope[token * rope_dim + c]);
            }
            score *= scale;
            maximum = fmaxf(maximum, score);
            scores[slot] = score;
        }
        float denominator = 0.0f;
        for (uint64_t slot = 0; slot < count; ++slot) {
            scores[slot] = expf(scores[slot] - maximum);
            denominator += scores[slot];
        }
        float* weighted = (float*)calloc(latent_dim, sizeof(float));
        for (uint64_t slot = 0; slot < count; ++slot) {
            uint64_t token = selected ? selected[slot] : slot;
            float probability = scores[slot] / denominator;
            for (uint64_t c = 0; c < latent_dim; ++c) {
                float value = (float)(int8_t)latent_codes[token * latent_dim + c] *
                              zo_bf16_to_f32(latent_scales[token * groups + c / latent_group_size]);
                weighted[c] += probability * value;
            }
        }
        if (weighted_f32) {
            memcpy(weighted_f32 + (row * heads + head) * latent_dim, weighted, latent_dim * sizeof(float));
        }
        /* (3) project value, matmul_nt (:754-768). */
        const float* w_v = kv_b + (head * kv_head_dim + nope) * latent_dim;
        for (uint64_t v = 0; v < value_dim; ++v) {
            float sum = zo_dot_seq(weighted, w_v + v * latent_dim, latent_dim);
            uint64_t index = row * heads * value_dim + head * value_dim + v;
            if (out_f32) {
                out_f32[index] = sum;
            }
            if (out_bf16) {
                out_bf16[index] = zo_f32_to_bf16(sum);
            }
        }
        free(weighted);
        free(scores);
        free(absorbed);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Threads (CPU baseline bookkeeping)                                        */
/* ------------------------------------------------------------------------ */

/* Mirrors src/kernel/cpu/mod.rs:29-44 (allowed_parallelism): the worker count
 * follows the process affinity mask.  n <= 0 keeps the OpenMP default. */
ZO_API int zo_set_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) {
        omp_set_num_threads(n);
    }
    return omp_get_max_threads();
#else
    (void)n;
    return 1;
#endif
}

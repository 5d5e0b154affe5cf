// Page appends: Q8g64 quantize + scatter, 16-bit scatter, fused MLA append, row gather.
//
// One wave64 owns one 64-element quantization group, so the group absmax is a
// wave reduction (max is order-independent, hence bit-exact with the reference's
// tree reduction, src/kernel/rocm/hip/attention/paged_mla/source.hip:175-181).
#include "common.hpp"
#include "kernels.hpp"

// Every product and sum in this file is rounded on its own, as in the CPU code these kernels must agree with bit for
// bit.  Expressions of more than one operation are written with plain operators under this pragma: the __fmul_rn /
// __fadd_rn intrinsics are ordinary operators compiled in a header where fusing is allowed, so a product and a sum
// written through them still become one multiply-add.
#pragma clang fp contract(off)

namespace zllm {

__device__ __forceinline__ float wave_max_all(float v)
{
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        v = fmaxf(v, __shfl_xor(v, offset));
    }
    return v;
}

// Quantize one value of a 64-group held one-per-lane; returns the code and
// writes the scale slot from lane 0.
//   rule 0 (paged_mla/source.hip:183-201): scale = absmax * (1/127), stored
//          bf16, code = nearbyint(x / f32(stored)).
//   rule 1 (kernel/metal/attention/mod.rs:114-127): scale = absmax / 127,
//          stored f16, code = rint(x * (1 / scale)).
//   rule 2 (kernel/cuda/attention.rs:331-341): as rule 1, stored f32.
__device__ __forceinline__ signed char quantize_lane(float value, int rule, void* scales, unsigned long long scale_index,
                                                     unsigned int lane)
{
    const float maximum = wave_max_all(fabsf(value));
    float quantized;
    if (rule == 0) {
        const float scale = maximum == 0.0f ? 1.0f : __fmul_rn(maximum, 1.0f / 127.0f);
        const unsigned short encoded = f32_to_bf16_bits(scale);
        if (lane == 0) {
            ((unsigned short*)scales)[scale_index] = encoded;
        }
        quantized = nearbyintf(__fdiv_rn(value, bf16_bits_to_f32(encoded)));
    } else {
        const float scale = maximum > 0.0f ? __fdiv_rn(maximum, 127.0f) : 1.0f;
        if (lane == 0) {
            if (rule == 1) {
                ((unsigned short*)scales)[scale_index] = f32_to_f16_bits(scale);
            } else {
                ((float*)scales)[scale_index] = scale;
            }
        }
        const float inverse = __fdiv_rn(1.0f, scale);
        quantized = rintf(__fmul_rn(value, inverse));
    }
    return (signed char)fmaxf(-127.0f, fminf(127.0f, quantized));
}

__global__ __launch_bounds__(256) void q8g64_append_kernel(Q8AppendParams p)
{
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int groups_per_row = p.cols / 64u;
    const unsigned long long group_index = (unsigned long long)blockIdx.x * 4u + (threadIdx.x >> 6);
    const unsigned long long total_groups = (unsigned long long)p.rows * groups_per_row;
    if (group_index >= total_groups) {
        return;
    }
    const unsigned int row = (unsigned int)(group_index / groups_per_row);
    const unsigned int group = (unsigned int)(group_index - (unsigned long long)row * groups_per_row);
    const unsigned int column = group * 64u + lane;
    const unsigned int position = p.positions != nullptr ? p.positions[0] : p.position;
    const float value = load_as_f32(p.src, (size_t)row * p.cols + column, p.src_dtype);
    const unsigned long long physical = paged_row(p.table, position + row, p.block_tokens, p.ring_capacity);
    const signed char code = quantize_lane(value, p.rule, p.scales, physical * groups_per_row + group, lane);
    p.codes[physical * p.cols + column] = code;
}

__global__ __launch_bounds__(256) void half_append_kernel(HalfAppendParams p)
{
    const unsigned long long index = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
    const unsigned long long elements = (unsigned long long)p.rows * p.cols;
    if (index >= elements) {
        return;
    }
    const unsigned int row = (unsigned int)(index / p.cols);
    const unsigned int column = (unsigned int)(index - (unsigned long long)row * p.cols);
    const unsigned long long physical = paged_row(p.table, p.position + row, p.block_tokens, p.ring_capacity);
    const float value = load_as_f32(p.src, index, p.src_dtype);
    p.cache[physical * p.cols + column] = p.dst_dtype == 1 ? f32_to_bf16_bits(value) : f32_to_f16_bits(value);
}

// Fused MLA append (what paged_cache_append_mla_body computes, paged_mla/source.hip:672-758), laid out the way the
// prologue kernel below is: one wave per token row, four rows per workgroup.  The wave quantizes the row's latent
// groups one after the other (a group is one value per lane), then writes the row's rope columns as bf16: the
// columns in front of the rotary part are copied, and each lane of the rotary part owns whole rotation pairs --
// it loads the pair and its cos / sin once and stores both rotated values.  Products are rounded on their own
// (no fused multiply-add), so the bits do not depend on the compiler's contraction choices.
__global__ __launch_bounds__(256) void mla_append_kernel(MlaAppendParams p)
{
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= p.rows) {
        return;
    }
    const unsigned int position = p.positions != nullptr ? p.positions[0] : p.position;
    const unsigned int rope_position = p.positions != nullptr ? p.positions[1] : p.rope_position;
    const unsigned long long physical = paged_row(p.table, position + row, p.block_tokens, 0);

    const unsigned int groups_per_row = p.latent_cols / 64u;
    const float* latent_row = p.latent + (unsigned long long)row * p.latent_cols;
    signed char* code_row = p.latent_codes + physical * p.latent_cols;
    for (unsigned int group = 0; group < groups_per_row; ++group) {
        const float value = latent_row[group * 64u + lane];
        code_row[group * 64u + lane] = quantize_lane(value, 0, p.latent_scales, physical * groups_per_row + group, lane);
    }

    const float* rope_row = p.k_rope + (unsigned long long)row * p.rope_cols;
    unsigned short* rope_out = p.rope_cache + physical * p.rope_cols;
    const unsigned int plain_cols = p.rope_cols - p.rotary_dim; // stored as they are
    for (unsigned int column = lane; column < plain_cols; column += 64u) {
        rope_out[column] = f32_to_bf16_bits(rope_row[column]);
    }
    const unsigned int pairs = p.rotary_dim / 2u;
    const float* cos_row = p.cosine + (unsigned long long)(rope_position + row) * pairs;
    const float* sin_row = p.sine + (unsigned long long)(rope_position + row) * pairs;
    for (unsigned int i = lane; i < pairs; i += 64u) {
        // split-half keeps the two members of pair i half a rotary block apart, interleaved keeps them adjacent
        const unsigned int first = plain_cols + (p.split_half ? i : 2u * i);
        const unsigned int second = p.split_half ? first + pairs : first + 1u;
        const float x = rope_row[first], y = rope_row[second];
        const float cs = cos_row[i], sn = sin_row[i];
        rope_out[first] = f32_to_bf16_bits(x * cs - y * sn);
        rope_out[second] = f32_to_bf16_bits(y * cs + x * sn);
    }
}

// Pre-attention prologue: one wave per (row, head) of Q, K or V.  The head's values sit one per lane per 64-column
// group (the layout the quantizer wants); the head goes through LDS once for the sum of squares and once for the
// rotation partner.
//   norm   (src/kernel/cpu/vae.rs:297-334): eight accumulators, element e into accumulator e % 8 in ascending order,
//          added as (l, l + 4), (0, 2) | (1, 3), halves -- lanes 0..7 do exactly that, so the sum has the reference
//          restatement's bits; then x * (1 / sqrt(sum / d + eps)) * (weight + offset), every step rounded on its own.
//   rope   (src/attention/rope.rs:120-164): real * cos - imag * sin, imag * cos + real * sin, products rounded
//          separately.
//   K, V   quantize_lane + page scatter, as the append kernel.
template <int GROUPS> __global__ __launch_bounds__(256) void gqa_prologue_kernel(GqaPrologueParams p)
{
    __shared__ float head_lds[4][GROUPS * 64];
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int wave = threadIdx.x >> 6;
    const unsigned int heads_per_row = p.num_heads + 2u * p.num_kv_heads;
    const unsigned long long unit = (unsigned long long)blockIdx.x * 4u + wave;
    if (unit >= (unsigned long long)p.rows * heads_per_row) {
        return;
    }
    const unsigned int row = (unsigned int)(unit / heads_per_row);
    const unsigned int slot = (unsigned int)(unit - (unsigned long long)row * heads_per_row);
    const unsigned int kind = slot < p.num_heads ? 0u : (slot < p.num_heads + p.num_kv_heads ? 1u : 2u); // Q, K, V
    const unsigned int head = kind == 0u ? slot : (kind == 1u ? slot - p.num_heads : slot - p.num_heads - p.num_kv_heads);
    const unsigned int head_count = kind == 0u ? p.num_heads : p.num_kv_heads;
    const void* src = kind == 0u ? p.q : (kind == 1u ? p.k : p.v);
    const float* weight = kind == 0u ? p.q_norm : (kind == 1u ? p.k_norm : nullptr);
    const unsigned int d = GROUPS * 64u;
    const size_t base = ((size_t)row * head_count + head) * d;
    const unsigned int position = p.positions != nullptr ? p.positions[0] : p.position;
    float* lds = head_lds[wave];
    float x[GROUPS];
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
        x[g] = load_as_f32(src, base + g * 64 + lane, p.src_dtype);
    }
    if (kind != 2u && weight != nullptr) {
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            lds[g * 64 + lane] = x[g];
        }
        __builtin_amdgcn_wave_barrier();
        float acc = 0.0f;
        if (lane < 8u) {
            for (unsigned int c = 0; c < d; c += 8u) {
                const float value = lds[c + lane];
                acc = acc + value * value;
            }
        }
        acc = acc + __shfl_xor(acc, 4);
        acc = acc + __shfl_xor(acc, 2);
        acc = acc + __shfl_xor(acc, 1);
        const float sum = __shfl(acc, 0);
        // sqrtf is correctly rounded (hipcc's default); __fsqrt_rn maps to the native approximation
        const float inverse = 1.0f / sqrtf(sum / (float)d + p.eps);
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            x[g] = x[g] * inverse * (weight[g * 64 + lane] + p.weight_offset);
        }
        __builtin_amdgcn_wave_barrier();
    }
    if (kind != 2u && p.rotary_dim != 0u) {
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            lds[g * 64 + lane] = x[g];
        }
        __builtin_amdgcn_wave_barrier();
        const unsigned int half = p.rotary_dim / 2u;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            const unsigned int column = g * 64u + lane;
            if (column < p.rotary_dim) {
                const unsigned int pair = p.split_half ? column % half : column / 2u;
                const unsigned int real_column = p.split_half ? pair : pair * 2u;
                const unsigned int imag_column = p.split_half ? half + pair : pair * 2u + 1u;
                const float real = lds[real_column];
                const float imaginary = lds[imag_column];
                const float c = p.cosine[(size_t)(position + row) * half + pair];
                const float s = p.sine[(size_t)(position + row) * half + pair];
                x[g] = column == real_column ? real * c - imaginary * s : imaginary * c + real * s;
            }
        }
    }
    if (kind == 0u) {
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            if (p.q_out_dtype == 0) {
                ((float*)p.q_out)[base + g * 64 + lane] = x[g];
            } else {
                ((unsigned short*)p.q_out)[base + g * 64 + lane] = f32_to_bf16_bits(x[g]);
            }
        }
        return;
    }
    const unsigned int cols = p.num_kv_heads * d;
    const unsigned int groups_per_row = cols / 64u;
    const unsigned long long physical = paged_row(p.table, position + row, p.block_tokens, p.ring_capacity);
    signed char* codes = kind == 1u ? p.k_codes : p.v_codes;
    void* scales = kind == 1u ? p.k_scales : p.v_scales;
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
        const unsigned int group = head * GROUPS + g;
        const signed char code = quantize_lane(x[g], p.rule, scales, physical * groups_per_row + group, lane);
        codes[physical * cols + group * 64u + lane] = code;
    }
}

// The same prologue with eight lanes per (row, head) unit and eight units per wave, for head_dim 64 / 128 / 256: a lane
// holds head_dim / 8 consecutive values, so the loads and stores are 16-byte vectors (a wave moves 2 to 8 KiB per
// instruction instead of 128 to 256 bytes) and the serial part of the norm -- eight accumulators, each running through
// its head_dim / 8 squares in order -- occupies all 64 lanes instead of eight.  Every sum and product is the one of
// gqa_prologue_kernel, in the same order: the results are the same bits.
template <int N> __device__ __forceinline__ void load_run_as_f32(const void* src, size_t index, int dtype, float (&out)[N])
{
    static_assert(N % 8 == 0, "whole 16-byte vectors");
    if (dtype == 0) {
#pragma unroll
        for (int i = 0; i < N / 4; ++i) {
            const f32x4 v = *(const f32x4*)((const float*)src + index + 4 * i);
            out[4 * i] = v[0], out[4 * i + 1] = v[1], out[4 * i + 2] = v[2], out[4 * i + 3] = v[3];
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < N / 8; ++i) {
        const u32x4 v = *(const u32x4*)((const unsigned short*)src + index + 8 * i);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const unsigned short lo = (unsigned short)(v[w] & 0xffffu), hi = (unsigned short)(v[w] >> 16);
            out[8 * i + 2 * w] = dtype == 1 ? bf16_bits_to_f32(lo) : f16_bits_to_f32(lo);
            out[8 * i + 2 * w + 1] = dtype == 1 ? bf16_bits_to_f32(hi) : f16_bits_to_f32(hi);
        }
    }
}

template <int GROUPS> __global__ __launch_bounds__(256) void gqa_prologue_wide(GqaPrologueParams p)
{
    static_assert(GROUPS == 1 || GROUPS == 2 || GROUPS == 4, "a lane's run must not straddle a 64-column group");
    constexpr int D = GROUPS * 64;
    constexpr int EPL = D / 8;         // values per lane
    constexpr int LPG = 64 / EPL;      // lanes per 64-column group
    __shared__ __align__(16) float unit_lds[4][8][D];
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int wave = threadIdx.x >> 6;
    const unsigned int sub = lane >> 3;  // unit of the wave
    const unsigned int part = lane & 7u; // eighth of the unit; also the accumulator this lane runs in the norm
    const unsigned int heads_per_row = p.num_heads + 2u * p.num_kv_heads;
    const unsigned long long total = (unsigned long long)p.rows * heads_per_row;
    const unsigned long long wanted = ((unsigned long long)blockIdx.x * 4u + wave) * 8u + sub;
    const bool live = wanted < total;
    const unsigned long long unit = live ? wanted : total - 1u; // a lane past the end repeats the last unit and stores nothing
    const unsigned int row = (unsigned int)(unit / heads_per_row);
    const unsigned int slot = (unsigned int)(unit - (unsigned long long)row * heads_per_row);
    const unsigned int kind = slot < p.num_heads ? 0u : (slot < p.num_heads + p.num_kv_heads ? 1u : 2u); // Q, K, V
    const unsigned int head = kind == 0u ? slot : (kind == 1u ? slot - p.num_heads : slot - p.num_heads - p.num_kv_heads);
    const unsigned int head_count = kind == 0u ? p.num_heads : p.num_kv_heads;
    const void* src = kind == 0u ? p.q : (kind == 1u ? p.k : p.v);
    const float* weight = kind == 0u ? p.q_norm : (kind == 1u ? p.k_norm : nullptr);
    const size_t base = ((size_t)row * head_count + head) * D + part * EPL;
    const unsigned int position = p.positions != nullptr ? p.positions[0] : p.position;
    float* lds = unit_lds[wave][sub];
    float x[EPL];
    load_run_as_f32<EPL>(src, base, p.src_dtype, x);
    if (kind != 2u && weight != nullptr) {
#pragma unroll
        for (int i = 0; i < EPL / 4; ++i) {
            *(f32x4*)(lds + part * EPL + 4 * i) = f32x4{x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]};
        }
        __builtin_amdgcn_wave_barrier();
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < EPL; ++k) { // accumulator `part`: elements part, part + 8, ... in ascending order
            const float value = lds[8 * k + part];
            acc = acc + value * value;
        }
        acc = acc + __shfl_xor(acc, 4);
        acc = acc + __shfl_xor(acc, 2);
        acc = acc + __shfl_xor(acc, 1);
        const float sum = __shfl(acc, (int)(lane & ~7u));
        // sqrtf is correctly rounded (hipcc's default); __fsqrt_rn maps to the native approximation
        const float inverse = 1.0f / sqrtf(sum / (float)D + p.eps);
        float w[EPL];
        load_run_as_f32<EPL>(weight, part * EPL, 0, w);
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            x[i] = x[i] * inverse * (w[i] + p.weight_offset);
        }
        __builtin_amdgcn_wave_barrier();
    }
    if (kind != 2u && p.rotary_dim != 0u) {
#pragma unroll
        for (int i = 0; i < EPL / 4; ++i) {
            *(f32x4*)(lds + part * EPL + 4 * i) = f32x4{x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]};
        }
        __builtin_amdgcn_wave_barrier();
        const unsigned int half = p.rotary_dim / 2u;
        const float* cos_row = p.cosine + (size_t)(position + row) * half;
        const float* sin_row = p.sine + (size_t)(position + row) * half;
        if (p.split_half && half % EPL == 0u && (((uintptr_t)p.cosine | (uintptr_t)p.sine) & 15u) == 0) {
            // split halves that are whole runs: the lane's run is all real or all imaginary parts, its partners are the
            // run half a rotary block away, and the angles of the run are consecutive
            const unsigned int start = part * EPL;
            if (start < p.rotary_dim) {
                const bool second = start >= half;
                const unsigned int pair0 = second ? start - half : start;
                float real[EPL], imaginary[EPL], c[EPL], sn[EPL];
                load_run_as_f32<EPL>(lds, pair0, 0, real);
                load_run_as_f32<EPL>(lds, half + pair0, 0, imaginary);
                load_run_as_f32<EPL>(cos_row, pair0, 0, c);
                load_run_as_f32<EPL>(sin_row, pair0, 0, sn);
#pragma unroll
                for (int i = 0; i < EPL; ++i) {
                    x[i] = second ? imaginary[i] * c[i] + real[i] * sn[i] : real[i] * c[i] - imaginary[i] * sn[i];
                }
            }
        } else {
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
            const unsigned int column = part * EPL + i;
            if (column < p.rotary_dim) {
                const unsigned int pair = p.split_half ? column % half : column / 2u;
                const unsigned int real_column = p.split_half ? pair : pair * 2u;
                const unsigned int imag_column = p.split_half ? half + pair : pair * 2u + 1u;
                const float real = lds[real_column];
                const float imaginary = lds[imag_column];
                const float c = cos_row[pair];
                const float sn = sin_row[pair];
                x[i] = column == real_column ? real * c - imaginary * sn : imaginary * c + real * sn;
            }
        }
        }
    }
    if (kind == 0u) {
        if (!live) {
            return;
        }
        if (p.q_out_dtype == 0) {
#pragma unroll
            for (int i = 0; i < EPL / 4; ++i) {
                *(f32x4*)((float*)p.q_out + base + 4 * i) = f32x4{x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]};
            }
        } else {
#pragma unroll
            for (int i = 0; i < EPL / 8; ++i) {
                u32x4 packed;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    packed[w] = (unsigned int)f32_to_bf16_bits(x[8 * i + 2 * w]) | ((unsigned int)f32_to_bf16_bits(x[8 * i + 2 * w + 1]) << 16);
                }
                *(u32x4*)((unsigned short*)p.q_out + base + 8 * i) = packed;
            }
        }
        return;
    }
    // K, V: the 64-column group of this lane's run is held by LPG neighbouring lanes
    float maximum = 0.0f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
        maximum = fmaxf(maximum, fabsf(x[i]));
    }
#pragma unroll
    for (int offset = 1; offset < LPG; offset <<= 1) {
        maximum = fmaxf(maximum, __shfl_xor(maximum, offset));
    }
    const unsigned int cols = p.num_kv_heads * D;
    const unsigned int groups_per_row = cols / 64u;
    const unsigned long long physical = paged_row(p.table, position + row, p.block_tokens, p.ring_capacity);
    signed char* codes = kind == 1u ? p.k_codes : p.v_codes;
    void* scales = kind == 1u ? p.k_scales : p.v_scales;
    const unsigned long long scale_index = physical * groups_per_row + head * GROUPS + part / LPG;
    const bool writer = live && part % LPG == 0u;
    float factor; // rule 0: the stored scale as f32 (divide by it); rules 1, 2: 1 / scale (multiply by it)
    if (p.rule == 0) {
        const float scale = maximum == 0.0f ? 1.0f : __fmul_rn(maximum, 1.0f / 127.0f);
        const unsigned short encoded = f32_to_bf16_bits(scale);
        if (writer) {
            ((unsigned short*)scales)[scale_index] = encoded;
        }
        factor = bf16_bits_to_f32(encoded);
    } else {
        const float scale = maximum > 0.0f ? __fdiv_rn(maximum, 127.0f) : 1.0f;
        if (writer) {
            if (p.rule == 1) {
                ((unsigned short*)scales)[scale_index] = f32_to_f16_bits(scale);
            } else {
                ((float*)scales)[scale_index] = scale;
            }
        }
        factor = __fdiv_rn(1.0f, scale);
    }
    if (!live) {
        return;
    }
    unsigned int packed[EPL / 4];
#pragma unroll
    for (int i = 0; i < EPL / 4; ++i) {
        packed[i] = 0u;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const float value = x[4 * i + b];
            const float quantized = p.rule == 0 ? nearbyintf(__fdiv_rn(value, factor)) : rintf(__fmul_rn(value, factor));
            const int code = (int)fmaxf(-127.0f, fminf(127.0f, quantized));
            packed[i] |= ((unsigned int)code & 0xffu) << (8 * b);
        }
    }
    unsigned int* out = (unsigned int*)(codes + physical * cols + (size_t)head * D + part * EPL);
    if constexpr (EPL == 8) {
        *(u32x2*)out = u32x2{packed[0], packed[1]};
    } else {
#pragma unroll
        for (int i = 0; i < EPL / 16; ++i) {
            *(u32x4*)(out + 4 * i) = u32x4{packed[4 * i], packed[4 * i + 1], packed[4 * i + 2], packed[4 * i + 3]};
        }
    }
}

// The same append with eight lanes per 64-column group and eight values per lane: 16-byte loads, 8-byte code stores.
// The group maximum is a maximum whichever way it is taken, everything after it is quantize_lane's arithmetic.
__global__ __launch_bounds__(256) void q8g64_append_wide(Q8AppendParams p)
{
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int part = lane & 7u;
    const unsigned int groups_per_row = p.cols / 64u;
    const unsigned long long total_groups = (unsigned long long)p.rows * groups_per_row;
    const unsigned long long wanted = ((unsigned long long)blockIdx.x * 4u + (threadIdx.x >> 6)) * 8u + (lane >> 3);
    const bool live = wanted < total_groups;
    const unsigned long long group_index = live ? wanted : total_groups - 1u;
    const unsigned int row = (unsigned int)(group_index / groups_per_row);
    const unsigned int group = (unsigned int)(group_index - (unsigned long long)row * groups_per_row);
    const unsigned int column = group * 64u + part * 8u;
    const unsigned int position = p.positions != nullptr ? p.positions[0] : p.position;
    float x[8];
    load_run_as_f32<8>(p.src, (size_t)row * p.cols + column, p.src_dtype, x);
    float maximum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        maximum = fmaxf(maximum, fabsf(x[i]));
    }
    maximum = fmaxf(maximum, __shfl_xor(maximum, 1));
    maximum = fmaxf(maximum, __shfl_xor(maximum, 2));
    maximum = fmaxf(maximum, __shfl_xor(maximum, 4));
    const unsigned long long physical = paged_row(p.table, position + row, p.block_tokens, p.ring_capacity);
    const unsigned long long scale_index = physical * groups_per_row + group;
    const bool writer = live && part == 0u;
    float factor;
    if (p.rule == 0) {
        const float scale = maximum == 0.0f ? 1.0f : __fmul_rn(maximum, 1.0f / 127.0f);
        const unsigned short encoded = f32_to_bf16_bits(scale);
        if (writer) {
            ((unsigned short*)p.scales)[scale_index] = encoded;
        }
        factor = bf16_bits_to_f32(encoded);
    } else {
        const float scale = maximum > 0.0f ? __fdiv_rn(maximum, 127.0f) : 1.0f;
        if (writer) {
            if (p.rule == 1) {
                ((unsigned short*)p.scales)[scale_index] = f32_to_f16_bits(scale);
            } else {
                ((float*)p.scales)[scale_index] = scale;
            }
        }
        factor = __fdiv_rn(1.0f, scale);
    }
    if (!live) {
        return;
    }
    unsigned int packed[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float quantized = p.rule == 0 ? nearbyintf(__fdiv_rn(x[i], factor)) : rintf(__fmul_rn(x[i], factor));
        const int code = (int)fmaxf(-127.0f, fminf(127.0f, quantized));
        packed[i >> 2] |= ((unsigned int)code & 0xffu) << (8 * (i & 3));
    }
    *(u32x2*)(p.codes + physical * p.cols + column) = u32x2{packed[0], packed[1]};
}

// Eight consecutive values of a row per thread: one or two 16-byte loads, one 16-byte store.
__global__ __launch_bounds__(256) void half_append_wide(HalfAppendParams p)
{
    const unsigned int runs_per_row = p.cols / 8u;
    const unsigned long long index = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= (unsigned long long)p.rows * runs_per_row) {
        return;
    }
    const unsigned int row = (unsigned int)(index / runs_per_row);
    const unsigned int column = (unsigned int)(index - (unsigned long long)row * runs_per_row) * 8u;
    const unsigned long long physical = paged_row(p.table, p.position + row, p.block_tokens, p.ring_capacity);
    float x[8];
    load_run_as_f32<8>(p.src, (size_t)row * p.cols + column, p.src_dtype, x);
    u32x4 packed;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const unsigned int lo = p.dst_dtype == 1 ? f32_to_bf16_bits(x[2 * w]) : f32_to_f16_bits(x[2 * w]);
        const unsigned int hi = p.dst_dtype == 1 ? f32_to_bf16_bits(x[2 * w + 1]) : f32_to_f16_bits(x[2 * w + 1]);
        packed[w] = lo | (hi << 16);
    }
    *(u32x4*)(p.cache + physical * p.cols + column) = packed;
}

template <typename T> __global__ __launch_bounds__(256) void gather_rows_kernel(GatherParams p, unsigned int units_per_row)
{
    const unsigned long long index = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
    const unsigned long long total = (unsigned long long)p.count * units_per_row;
    if (index >= total) {
        return;
    }
    const unsigned int row = (unsigned int)(index / units_per_row);
    const unsigned int unit = (unsigned int)(index - (unsigned long long)row * units_per_row);
    const unsigned long long physical = paged_row(p.table, p.first + row, p.block_tokens, p.ring_capacity);
    ((T*)p.out)[index] = ((const T*)p.plane)[physical * units_per_row + unit];
}

template <typename T> __global__ __launch_bounds__(256) void scatter_rows_kernel(ScatterParams p, unsigned int units_per_row)
{
    const unsigned long long index = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
    const unsigned long long total = (unsigned long long)p.count * units_per_row;
    if (index >= total) {
        return;
    }
    const unsigned int row = (unsigned int)(index / units_per_row);
    const unsigned int unit = (unsigned int)(index - (unsigned long long)row * units_per_row);
    const unsigned long long physical = paged_row(p.table, p.first + row, p.block_tokens, p.ring_capacity);
    ((T*)p.plane)[physical * units_per_row + unit] = ((const T*)p.in)[index];
}

hipError_t launch_scatter_rows(const ScatterParams& p, hipStream_t stream)
{
    if (p.count == 0 || p.row_bytes == 0) {
        return hipSuccess;
    }
    const bool aligned16 = p.row_bytes % 16 == 0 && ((uintptr_t)p.plane % 16 == 0) && ((uintptr_t)p.in % 16 == 0);
    const bool aligned4 = p.row_bytes % 4 == 0 && ((uintptr_t)p.plane % 4 == 0) && ((uintptr_t)p.in % 4 == 0);
    const unsigned int unit = aligned16 ? 16 : (aligned4 ? 4 : 1);
    const unsigned int units_per_row = p.row_bytes / unit;
    const unsigned long long total = (unsigned long long)p.count * units_per_row;
    const dim3 grid((unsigned int)((total + 255) / 256));
    if (unit == 16) {
        scatter_rows_kernel<uint4><<<grid, dim3(256), 0, stream>>>(p, units_per_row);
    } else if (unit == 4) {
        scatter_rows_kernel<unsigned int><<<grid, dim3(256), 0, stream>>>(p, units_per_row);
    } else {
        scatter_rows_kernel<unsigned char><<<grid, dim3(256), 0, stream>>>(p, units_per_row);
    }
    return hipGetLastError();
}

hipError_t launch_q8g64_append(const Q8AppendParams& p, hipStream_t stream)
{
    const unsigned long long groups = (unsigned long long)p.rows * (p.cols / 64u);
    if (groups == 0) {
        return hipSuccess;
    }
    if ((((uintptr_t)p.src | (uintptr_t)p.codes) & 15u) == 0) { // 16-byte loads of the source, 8-byte stores of the codes
        q8g64_append_wide<<<dim3((unsigned int)((groups + 31) / 32)), dim3(256), 0, stream>>>(p);
    } else {
        q8g64_append_kernel<<<dim3((unsigned int)((groups + 3) / 4)), dim3(256), 0, stream>>>(p);
    }
    return hipGetLastError();
}

hipError_t launch_half_append(const HalfAppendParams& p, hipStream_t stream)
{
    const unsigned long long elements = (unsigned long long)p.rows * p.cols;
    if (elements == 0) {
        return hipSuccess;
    }
    if (p.cols % 8u == 0 && (((uintptr_t)p.src | (uintptr_t)p.cache) & 15u) == 0) {
        half_append_wide<<<dim3((unsigned int)((elements / 8 + 255) / 256)), dim3(256), 0, stream>>>(p);
    } else {
        half_append_kernel<<<dim3((unsigned int)((elements + 255) / 256)), dim3(256), 0, stream>>>(p);
    }
    return hipGetLastError();
}

hipError_t launch_gqa_prologue(const GqaPrologueParams& p, hipStream_t stream)
{
    const unsigned long long units = (unsigned long long)p.rows * (p.num_heads + 2u * p.num_kv_heads);
    // vector loads and stores: every tensor and plane 16-byte aligned (rows are multiples of 64 values)
    const uintptr_t pointers = (uintptr_t)p.q | (uintptr_t)p.k | (uintptr_t)p.v | (uintptr_t)p.q_out | (uintptr_t)p.k_codes | (uintptr_t)p.v_codes |
                               (uintptr_t)p.q_norm | (uintptr_t)p.k_norm;
    if ((pointers & 15u) == 0 && p.head_dim != 192u) {
        const dim3 wide_grid((unsigned int)((units + 31) / 32));
        switch (p.head_dim / 64u) {
        case 1: gqa_prologue_wide<1><<<wide_grid, dim3(256), 0, stream>>>(p); break;
        case 2: gqa_prologue_wide<2><<<wide_grid, dim3(256), 0, stream>>>(p); break;
        default: gqa_prologue_wide<4><<<wide_grid, dim3(256), 0, stream>>>(p); break;
        }
        return hipGetLastError();
    }
    const dim3 grid((unsigned int)((units + 3) / 4));
    switch (p.head_dim / 64u) {
    case 1: gqa_prologue_kernel<1><<<grid, dim3(256), 0, stream>>>(p); break;
    case 2: gqa_prologue_kernel<2><<<grid, dim3(256), 0, stream>>>(p); break;
    case 3: gqa_prologue_kernel<3><<<grid, dim3(256), 0, stream>>>(p); break;
    case 4: gqa_prologue_kernel<4><<<grid, dim3(256), 0, stream>>>(p); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_mla_append(const MlaAppendParams& p, hipStream_t stream)
{
    if (p.rows == 0) {
        return hipSuccess;
    }
    mla_append_kernel<<<dim3((p.rows + 3u) / 4u), dim3(256), 0, stream>>>(p);
    return hipGetLastError();
}

hipError_t launch_gather_rows(const GatherParams& p, hipStream_t stream)
{
    if (p.count == 0 || p.row_bytes == 0) {
        return hipSuccess;
    }
    const bool aligned16 = p.row_bytes % 16 == 0 && ((uintptr_t)p.plane % 16 == 0) && ((uintptr_t)p.out % 16 == 0);
    const bool aligned4 = p.row_bytes % 4 == 0 && ((uintptr_t)p.plane % 4 == 0) && ((uintptr_t)p.out % 4 == 0);
    const unsigned int unit = aligned16 ? 16 : (aligned4 ? 4 : 1);
    const unsigned int units_per_row = p.row_bytes / unit;
    const unsigned long long total = (unsigned long long)p.count * units_per_row;
    const dim3 grid((unsigned int)((total + 255) / 256));
    if (unit == 16) {
        gather_rows_kernel<uint4><<<grid, dim3(256), 0, stream>>>(p, units_per_row);
    } else if (unit == 4) {
        gather_rows_kernel<unsigned int><<<grid, dim3(256), 0, stream>>>(p, units_per_row);
    } else {
        gather_rows_kernel<unsigned char><<<grid, dim3(256), 0, stream>>>(p, units_per_row);
    }
    return hipGetLastError();
}

} // namespace zllm

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
    q8g64_append_kernel<<<dim3((unsigned int)((groups + 3) / 4)), dim3(256), 0, stream>>>(p);
    return hipGetLastError();
}

hipError_t launch_half_append(const HalfAppendParams& p, hipStream_t stream)
{
    const unsigned long long elements = (unsigned long long)p.rows * p.cols;
    if (elements == 0) {
        return hipSuccess;
    }
    half_append_kernel<<<dim3((unsigned int)((elements + 255) / 256)), dim3(256), 0, stream>>>(p);
    return hipGetLastError();
}

hipError_t launch_gqa_prologue(const GqaPrologueParams& p, hipStream_t stream)
{
    const unsigned long long units = (unsigned long long)p.rows * (p.num_heads + 2u * p.num_kv_heads);
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

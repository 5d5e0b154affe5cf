// Absorbed MLA decode for the geometries and weight formats the matrix-core kernels do not take: any latent width that
// Q8g64 groups divide (64 .. 1024 columns), any even rope width up to 256, and kv_b as f32, bf16, or 8- / 4-bit codes
// with a scale per row and column group (the formats of paged_weight,
// src/kernel/rocm/hip/attention/paged_mla/source.hip:2-26).  Vector ALU only: the work is a few dot products per
// token, and these shapes are the small ones (the reference's own rank-64 case, src/kernel/cpu/mla.rs:1166-1195).
//
//   absorb   q_abs[h, c] = sum_k q_nope[h, k] * W[h, k, c], k ascending, product and sum rounded separately, result
//            rounded to bf16 -- the arithmetic of the reference's scalar matmul (src/kernel/cpu/mla.rs:712-728, :1037)
//   partial  one workgroup per (split, head, query row): every wave walks tokens of the split, a lane owns the latent
//            columns lane, lane + 64, ...; score = sum_g scale_g (codes_g . q_abs_g) + rope . q_rope, online softmax per
//            wave, the four waves combined at the end; records as the matrix-core kernels write them
//            (un-normalised sum of p x latent, running maximum in base-2 units, sum of p)
//   project  out[h, v] = sum_c merged[h, c] * W[h, nope + v, c]
#include <hip/hip_runtime.h>

#include "common.hpp"
#include "kernels.hpp"
#include "mla_rows.hpp"

namespace zllm {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kMaxLatentPerLane = 16; // latent_dim <= 1024

// Element (row, column) of kv_b [rows, columns]: bits 32 = f32, 16 = bf16, 8 / 4 = codes packed low bits first into
// 32-bit words, value (code - 128) or (code - 8) times the scale of (row, column / group)
__device__ __forceinline__ float weight_at(const MlaDecodeParams& p, unsigned int row, unsigned int column)
{
    const unsigned int columns = p.latent_dim;
    if (p.kv_b_bits == 16u) {
        return bf16_bits_to_f32(p.kv_b[(size_t)row * columns + column]);
    }
    if (p.kv_b_bits == 32u) {
        return ((const float*)p.kv_b)[(size_t)row * columns + column];
    }
    const unsigned int per_word = 32u / p.kv_b_bits;
    const size_t words = ((size_t)columns + per_word - 1u) / per_word;
    const unsigned int word = ((const unsigned int*)p.kv_b)[(size_t)row * words + column / per_word];
    const unsigned int code = (word >> ((column % per_word) * p.kv_b_bits)) & ((1u << p.kv_b_bits) - 1u);
    const int centred = p.kv_b_bits == 4u ? (int)code - 8 : (int)code - 128;
    const size_t at = (size_t)row * (columns / p.kv_b_group) + column / p.kv_b_group;
    float scale;
    if (p.kv_b_scale_dtype == 2) {
        scale = ((const float*)p.kv_b_scales)[at];
    } else if (p.kv_b_scale_dtype == 1) {
        scale = f16_bits_to_f32(((const unsigned short*)p.kv_b_scales)[at]);
    } else {
        scale = bf16_bits_to_f32(((const unsigned short*)p.kv_b_scales)[at]);
    }
    return (float)centred * scale;
}

// grid = (heads, query rows), 256 threads: a thread owns latent columns tid, tid + 256, ...
__global__ __launch_bounds__(256) void mla_absorb_any(MlaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    __shared__ float q_sh[1024];
    const size_t q_base = ((size_t)b * p.heads + head) * p.q_head_dim;
    for (unsigned int i = threadIdx.x; i < p.q_head_dim; i += 256u) {
        // the oracle takes a bf16 query (src/kernel/cpu/mla.rs:958-961)
        q_sh[i] = bf16_bits_to_f32(f32_to_bf16_bits(load_as_f32(p.q, q_base + i, p.q_dtype)));
    }
    __syncthreads();
    unsigned short* qa = p.absorbed + ((size_t)b * p.heads + head) * (p.latent_dim + p.rope_dim);
    for (unsigned int c = threadIdx.x; c < p.latent_dim; c += 256u) {
#pragma clang fp contract(off)
        float acc = 0.0f;
        for (unsigned int k = 0; k < p.nope_dim; ++k) {
            acc = acc + q_sh[k] * weight_at(p, head * p.kv_head_dim + k, c);
        }
        qa[c] = f32_to_bf16_bits(acc);
    }
    for (unsigned int r = threadIdx.x; r < p.rope_dim; r += 256u) {
        qa[p.latent_dim + r] = f32_to_bf16_bits(q_sh[p.nope_dim + r]);
    }
}

struct WaveState {
    float m, l;
    float acc[kMaxLatentPerLane];
};

// grid = (split or dense item, heads, query rows or 1), 256 threads
__global__ __launch_bounds__(256) void mla_partial_any(MlaDecodeParams p)
{
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int wave = threadIdx.x >> 6;
    const unsigned int head = blockIdx.y;
    unsigned int chunk = blockIdx.x;
    unsigned int b = gridDim.z - 1u - blockIdx.z;
    if (p.record_rows != 0u && !mla_locate_split(p, blockIdx.x, lane, b, chunk)) {
        return;
    }
    unsigned int seq;
    unsigned int len = visible_tokens(p.ctx_lens, p.query_rows, b, seq);
    const unsigned int* selected = nullptr;
    if (p.selection != nullptr && p.top_k < len) {
        selected = p.selection + (size_t)b * p.top_k;
        len = p.selection_counts != nullptr ? min(p.selection_counts[b], p.top_k) : p.top_k;
    }
    const unsigned int n_splits = min(p.max_chunks, (len + p.chunk_tokens - 1u) / p.chunk_tokens);
    const unsigned int span = n_splits > 0u ? min(p.chunk_tokens, (((len + n_splits - 1u) / n_splits) + 31u) & ~31u) : p.chunk_tokens;
    const unsigned long long c_start64 = (unsigned long long)chunk * span;
    const size_t row = p.record_rows != 0u ? (size_t)blockIdx.x : (size_t)b * p.max_chunks + chunk;
    const size_t rec = row * p.heads + head;
    if (c_start64 >= len) { // empty split: (max, sum) = (-inf, 0), the merge skips it
        if (threadIdx.x == 0u) {
            p.stats[rec * 2] = kNegInf;
            p.stats[rec * 2 + 1] = 0.0f;
        }
        return;
    }
    const unsigned int c_start = (unsigned int)c_start64;
    const unsigned int c_end = (unsigned int)min((unsigned long long)len, c_start64 + span);
    const unsigned int groups = p.latent_dim / 64u;
    const unsigned int* table = p.tables != nullptr ? p.tables + (size_t)seq * p.table_stride : nullptr;
    const unsigned short* qa = p.absorbed + ((size_t)b * p.heads + head) * (p.latent_dim + p.rope_dim);
    float q_lat[kMaxLatentPerLane];
#pragma unroll
    for (int g = 0; g < kMaxLatentPerLane; ++g) {
        q_lat[g] = (unsigned int)g < groups ? bf16_bits_to_f32(qa[g * 64 + lane]) : 0.0f;
    }
    float q_rope[4]; // rope columns lane, lane + 64, ...
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const unsigned int c = r * 64u + lane;
        q_rope[r] = c < p.rope_dim ? bf16_bits_to_f32(qa[p.latent_dim + c]) : 0.0f;
    }
    const float scale_log2 = p.score_scale * kLog2e;
    WaveState st;
    st.m = kNegInf;
    st.l = 0.0f;
#pragma unroll
    for (int g = 0; g < kMaxLatentPerLane; ++g) {
        st.acc[g] = 0.0f;
    }
    for (unsigned int t = c_start + wave; t < c_end; t += 4u) {
        const unsigned int token = selected != nullptr ? selected[t] : t;
        const unsigned long long phys = table != nullptr ? (unsigned long long)table[token / p.block_tokens] * p.block_tokens + token % p.block_tokens
                                                         : token;
        const signed char* codes = p.latent_codes + phys * p.latent_dim;
        const unsigned short* scales = p.latent_scales + phys * groups;
        const unsigned short* rope = p.rope_cache + phys * p.rope_dim;
        float value[kMaxLatentPerLane];
        float dot = 0.0f;
#pragma unroll
        for (int g = 0; g < kMaxLatentPerLane; ++g) {
            value[g] = 0.0f;
            if ((unsigned int)g < groups) {
                value[g] = (float)codes[g * 64 + lane] * bf16_bits_to_f32(scales[g]);
                dot = fmaf(value[g], q_lat[g], dot);
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const unsigned int c = r * 64u + lane;
            if (c < p.rope_dim) {
                dot = fmaf(bf16_bits_to_f32(rope[c]), q_rope[r], dot);
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            dot += __shfl_xor(dot, off);
        }
        const float s = dot * scale_log2;
        const float nm = fmaxf(st.m, s);
        const float alpha = __builtin_amdgcn_exp2f(st.m - nm); // m = -inf -> 0
        const float w = __builtin_amdgcn_exp2f(s - nm);
        st.l = st.l * alpha + w;
        st.m = nm;
#pragma unroll
        for (int g = 0; g < kMaxLatentPerLane; ++g) {
            st.acc[g] = st.acc[g] * alpha + w * value[g];
        }
    }
    // the four waves' states into one
    __shared__ float sh_m[4], sh_l[4];
    __shared__ float sh_acc[4][1024];
    if (lane == 0u) {
        sh_m[wave] = st.m;
        sh_l[wave] = st.l;
    }
#pragma unroll
    for (int g = 0; g < kMaxLatentPerLane; ++g) {
        if ((unsigned int)g < groups) {
            sh_acc[wave][g * 64 + lane] = st.acc[g];
        }
    }
    __syncthreads();
    const float top = fmaxf(fmaxf(sh_m[0], sh_m[1]), fmaxf(sh_m[2], sh_m[3]));
    float weight[4], total = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        weight[w] = sh_l[w] > 0.0f ? __builtin_amdgcn_exp2f(sh_m[w] - top) : 0.0f;
        total += sh_l[w] * weight[w];
    }
    if (threadIdx.x == 0u) {
        p.stats[rec * 2] = total > 0.0f ? top : kNegInf;
        p.stats[rec * 2 + 1] = total;
    }
    float* out = p.partial + rec * p.latent_dim;
    for (unsigned int c = threadIdx.x; c < p.latent_dim; c += 256u) {
        out[c] = sh_acc[0][c] * weight[0] + sh_acc[1][c] * weight[1] + sh_acc[2][c] * weight[2] + sh_acc[3][c] * weight[3];
    }
}

// grid = (heads, query rows), 256 threads: a wave takes value columns wave, wave + 4, ...; its lanes share the latent
// columns of one weight row
__global__ __launch_bounds__(256) void mla_project_any(MlaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int wave = threadIdx.x >> 6;
    const float* merged = p.weighted + ((size_t)b * p.heads + head) * p.latent_dim;
    const unsigned int out_stride = p.out_compact ? p.value_dim : p.q_head_dim;
    const size_t out_base = ((size_t)b * p.heads + head) * out_stride;
    for (unsigned int v = wave; v < p.value_dim; v += 4u) {
        float sum = 0.0f;
        for (unsigned int c = lane; c < p.latent_dim; c += 64u) {
            sum = fmaf(merged[c], weight_at(p, head * p.kv_head_dim + p.nope_dim + v, c), sum);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            sum += __shfl_xor(sum, off);
        }
        if (lane == 0u) {
            if (p.out_dtype == 0) {
                ((float*)p.out)[out_base + v] = sum;
            } else {
                ((unsigned short*)p.out)[out_base + v] = f32_to_bf16_bits(sum);
            }
        }
    }
}

} // namespace

hipError_t launch_mla_absorb_any(const MlaDecodeParams& p, hipStream_t stream)
{
    mla_absorb_any<<<dim3(p.heads, p.batch), dim3(256), 0, stream>>>(p);
    return hipGetLastError();
}

hipError_t launch_mla_partial_any(const MlaDecodeParams& p, hipStream_t stream)
{
    const dim3 grid = p.record_rows != 0u ? dim3(p.record_rows, p.heads, 1) : dim3(p.max_chunks, p.heads, p.batch);
    mla_partial_any<<<grid, dim3(256), 0, stream>>>(p);
    return hipGetLastError();
}

hipError_t launch_mla_project_any(const MlaDecodeParams& p, hipStream_t stream)
{
    mla_project_any<<<dim3(p.heads, p.batch), dim3(256), 0, stream>>>(p);
    return hipGetLastError();
}

} // namespace zllm

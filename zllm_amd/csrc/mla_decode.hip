// Absorbed MLA decode over the paged Q8g64 latent cache — gfx950, bf16 MFMA.
//
// Stages (the reference's chain absorb -> partial -> merge -> project,
// src/kernel/rocm/hip/attention/paged_mla.rs:3042-3621):
//   1. mla_absorb:  qa[b, h, 0:512] = bf16(q_nope[b, h, :] . W_kv_b[h, 0:nope, :]),
//                   qa[b, h, 512:576] = bf16(q_rope[b, h, :])
//   2. mla_partial: split-KV attention of 128 heads against one shared latent row per token.
//                   A workgroup owns (split, sequence).  Per 32-token step it converts the latent
//                   codes ONCE into LDS as bf16 integers (exact) next to the bf16 rope columns and
//                   the f32 group scales; its four waves (32 heads each) then run
//                     S^T[token, head]  = sum_g scale[token, g] * (codes_g[token, :] . qa_g[head, :])
//                                         + rope[token, :] . q_rope[head, :]     (MFMA 16x16x32 bf16,
//                                         one accumulator per 64-column group: products are exact)
//                     online softmax (wave shuffles)
//                     O^T[dim, head]   += codes^T[dim, token] . P'_g[token, head], P'_g = bf16(p * scale_g)
//                   The same row-major tile feeds both products: QK^T reads it with ds_read_b128,
//                   P.V reads it transposed with ds_read_b64_tr_b16.  A 16-byte XOR swizzle keeps both
//                   access patterns free of bank conflicts.
//   3. split merge by log-sum-exp (shared with GQA decode)
//   4. mla_project: out[b, h, v] = weighted[b, h, :] . W_kv_b[h, nope + v, :]
#include <string.h>

#include "common.hpp"
#include "kernels.hpp"

namespace zllm {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kLatent = 512;
constexpr int kRope = 64;
constexpr int kRowElems = kLatent + kRope; // 576 bf16 per token in LDS
constexpr int kRowBytes = kRowElems * 2;   // 1152 = 72 chunks of 16 B
constexpr int kStepTokens = 32;
constexpr int kTileBytes = kStepTokens * kRowBytes; // 36,864

typedef short s16x4 __attribute__((ext_vector_type(4)));

union Frag {
    u32x4 u;
    bf16x8 b;
};

// chunk swizzle: eight consecutive rows land in eight different 16-byte columns, and four
// consecutive rows in four different 32-byte column pairs
__device__ __forceinline__ unsigned int swz(unsigned int row)
{
    const unsigned int x = row & 7u;
    return ((x & 3u) << 1) | (x >> 2);
}

__device__ __forceinline__ unsigned int tile_offset(unsigned int row, unsigned int chunk)
{
    return row * kRowBytes + ((chunk ^ swz(row)) << 4);
}

// ---------------------------------------------------------------------------------------------
// 1. absorb
// ---------------------------------------------------------------------------------------------
// grid = (heads, batch), 256 threads, thread c owns latent columns c and c + 256.
// The sum runs over k in ascending order with separately rounded multiply and add, the order of
// the reference's scalar matmul (src/kernel/cpu/mla.rs:712-728); the result is rounded to bf16
// (mla.rs:1037).
__global__ __launch_bounds__(256) void mla_absorb(MlaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    __shared__ float q_sh[1024];
    const size_t q_base = ((size_t)b * p.heads + head) * p.q_head_dim;
    for (unsigned int i = threadIdx.x; i < p.q_head_dim; i += 256) {
        float x = load_as_f32(p.q, q_base + i, p.q_dtype);
        // the oracle takes a bf16 query (src/kernel/cpu/mla.rs:958-961)
        q_sh[i] = bf16_bits_to_f32(f32_to_bf16_bits(x));
    }
    __syncthreads();
    unsigned short* qa = p.absorbed + ((size_t)b * p.heads + head) * (p.latent_dim + p.rope_dim);
    const unsigned short* w = p.kv_b + (size_t)head * p.kv_head_dim * p.latent_dim;
    for (unsigned int c = threadIdx.x; c < p.latent_dim; c += 256) {
        float acc = 0.0f;
        for (unsigned int k = 0; k < p.nope_dim; ++k) {
            acc = __fadd_rn(acc, __fmul_rn(q_sh[k], bf16_bits_to_f32(w[(size_t)k * p.latent_dim + c])));
        }
        qa[c] = f32_to_bf16_bits(acc);
    }
    for (unsigned int r = threadIdx.x; r < p.rope_dim; r += 256) {
        qa[p.latent_dim + r] = f32_to_bf16_bits(q_sh[p.nope_dim + r]);
    }
}

// ---------------------------------------------------------------------------------------------
// 2. split-KV partial
// ---------------------------------------------------------------------------------------------
struct StepRegs {
    u32x4 codes[4];          // 4 items x 16 int8 codes
    unsigned short scale[4]; // bf16 scale of each item's group
    u32x4 rope;              // 8 bf16 rope values
};

// TPW = head tiles (16 heads) per wave, 4 waves per workgroup.  DSPLIT = number of workgroups that
// share one (split, sequence, head block): each accumulates 512 / DSPLIT output columns (and repeats the
// score computation), which keeps accumulators + query fragments inside the register file.
template <int TPW, int DSPLIT>
__global__ __launch_bounds__(256) void mla_partial(MlaDecodeParams p)
{
    constexpr int MT = 32 / DSPLIT; // output M tiles (16 latent columns each) of this workgroup
    __shared__ __align__(16) unsigned char lds[2 * kTileBytes];
    __shared__ __align__(16) float lds_scale[2][8][kStepTokens]; // [buffer][group][token]
    const unsigned int tid = threadIdx.x;
    const unsigned int lane = tid & 63u;
    const unsigned int wave = tid >> 6;
    const unsigned int m = lane & 15u;
    const unsigned int j = lane >> 4;
    const unsigned int chunk = blockIdx.x;
    const unsigned int dsplit = blockIdx.y % DSPLIT;
    const unsigned int head_base = (blockIdx.y / DSPLIT) * (64u * TPW) + wave * (16u * TPW);
    const unsigned int b = blockIdx.z;
    const unsigned int len = p.ctx_lens[b];
    const unsigned long long c_start64 = (unsigned long long)chunk * p.chunk_tokens;

    // (max, sum) records for an empty split
    if (c_start64 >= len) {
#pragma unroll
        for (int h = 0; h < TPW; ++h) {
            const unsigned int head = head_base + 16u * h + m;
            if (head < p.heads && j == 0 && dsplit == 0) {
                const size_t si = (((size_t)b * p.max_chunks + chunk) * p.heads + head) * 2;
                p.stats[si] = kNegInf;
                p.stats[si + 1] = 0.0f;
            }
        }
        return;
    }
    const unsigned int c_start = (unsigned int)c_start64;
    const unsigned int c_end = (unsigned int)min((unsigned long long)len, c_start64 + p.chunk_tokens);
    const unsigned int steps = (c_end - c_start + kStepTokens - 1) / kStepTokens;

    // ---- Q fragments (B operand): lane = (head column m, k-slice j); k-step ks covers dims
    //      ks*32 + j*8 .. +8 of the 576-wide absorbed query ------------------------------------
    Frag qf[TPW][18];
#pragma unroll
    for (int h = 0; h < TPW; ++h) {
        const unsigned int head = head_base + 16u * h + m;
        const unsigned short* qa = p.absorbed + ((size_t)b * p.heads + min(head, p.heads - 1u)) * kRowElems;
#pragma unroll
        for (int ks = 0; ks < 18; ++ks) {
            u32x4 v = *(const u32x4*)(qa + ks * 32 + j * 8);
            if (head >= p.heads) {
                v = u32x4{0u, 0u, 0u, 0u};
            }
            qf[h][ks].u = v;
        }
    }

    const unsigned int* table = p.tables != nullptr ? p.tables + (size_t)b * p.table_stride : nullptr;
    const bool pow2 = (p.block_tokens & (p.block_tokens - 1u)) == 0;
    auto row_of = [&](unsigned int token) __attribute__((always_inline)) -> unsigned long long {
        token = min(token, len - 1u);
        if (table == nullptr) {
            return token;
        }
        if (pow2) {
            return ((unsigned long long)table[token >> p.block_shift] << p.block_shift) + (token & (p.block_tokens - 1u));
        }
        return (unsigned long long)table[token / p.block_tokens] * p.block_tokens + token % p.block_tokens;
    };

    // cooperative staging: item i of a thread = token (tid >> 5) + 8 i, 16-code chunk cc = tid & 31
    const unsigned int cc = tid & 31u;
    const unsigned int t_lo = tid >> 5;
    const unsigned int rope_t = tid >> 3;
    const unsigned int rope_c = tid & 7u;
    auto load_step = [&](StepRegs& r, unsigned int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const unsigned long long row = row_of(t0 + t_lo + 8u * i);
            r.codes[i] = *(const u32x4*)(p.latent_codes + row * kLatent + cc * 16u);
            r.scale[i] = p.latent_scales[row * (kLatent / 64) + (cc >> 2)];
        }
        const unsigned long long row = row_of(t0 + rope_t);
        r.rope = *(const u32x4*)(p.rope_cache + row * kRope + rope_c * 8u);
    };
    auto store_step = [&](const StepRegs& r, unsigned char* tile, float (*scale_tile)[kStepTokens]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const unsigned int row = t_lo + 8u * i;
            u32x4 out[2];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const unsigned int word = r.codes[i][w];
                const float c0 = (float)(int)(signed char)(word & 0xffu);
                const float c1 = (float)(int)(signed char)((word >> 8) & 0xffu);
                const float c2 = (float)(int)(signed char)((word >> 16) & 0xffu);
                const float c3 = (float)(int)(signed char)(word >> 24);
                out[w >> 1][(w & 1) * 2] = pack_bf16_trunc(c0, c1);
                out[w >> 1][(w & 1) * 2 + 1] = pack_bf16_trunc(c2, c3);
            }
            *(u32x4*)(tile + tile_offset(row, cc * 2u)) = out[0];
            *(u32x4*)(tile + tile_offset(row, cc * 2u + 1u)) = out[1];
            if ((cc & 3u) == 0) {
                scale_tile[cc >> 2][row] = bf16_bits_to_f32(r.scale[i]);
            }
        }
        *(u32x4*)(tile + tile_offset(rope_t, 64u + rope_c)) = r.rope;
    };

    f32x4 acc[TPW][MT];
#pragma unroll
    for (int h = 0; h < TPW; ++h) {
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            acc[h][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float run_max[TPW], run_sum[TPW];
#pragma unroll
    for (int h = 0; h < TPW; ++h) {
        run_max[h] = kNegInf;
        run_sum[h] = 0.0f;
    }
    const float scale_log2 = p.score_scale * kLog2e;
    constexpr float kRescaleSlack = 8.0f; // log2 units: keep a stale maximum while p stays below 2^8

    // LDS byte offsets of this lane's fragments, split into a lane part and a compile-time part so
    // that every read is `base + immediate`:  chunk = (hi << 3) | lo, and only `lo` meets the swizzle.
    const unsigned int qk_base[2] = {m * kRowBytes + ((j ^ swz(m)) << 4), m * kRowBytes + (((4u | j) ^ swz(m)) << 4)};
    const unsigned int tr_row = 4u * j + (m >> 2);
    unsigned int pv_base[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        pv_base[q] = tr_row * kRowBytes + ((((unsigned int)q << 1 | ((m & 3u) >> 1)) ^ swz(tr_row)) << 4) + (m & 1u) * 8u;
    }

    constexpr int GROUPS = 8 / DSPLIT; // scale groups among this workgroup's output columns
    auto compute_step = [&](const unsigned char* tile, const float (*scale_tile)[kStepTokens], unsigned int t0) __attribute__((always_inline)) {
        // ---- S^T = sum_g scale_g * (codes_g . qa_g) + rope . q_rope -----------------------------
        f32x4 s[2][TPW];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int h = 0; h < TPW; ++h) {
                s[i][h] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            // rope columns (k-steps 16, 17): unscaled
#pragma unroll
            for (int ks = 16; ks < 18; ++ks) {
                Frag kf;
                kf.u = *(const u32x4*)(tile + qk_base[ks & 1] + (i * 16 * kRowBytes + (ks >> 1) * 128));
#pragma unroll
                for (int h = 0; h < TPW; ++h) {
                    s[i][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.b, qf[h][ks].b, s[i][h], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                Frag k0, k1;
                k0.u = *(const u32x4*)(tile + qk_base[0] + (i * 16 * kRowBytes + g * 128));
                k1.u = *(const u32x4*)(tile + qk_base[1] + (i * 16 * kRowBytes + g * 128));
                // group scales of this lane's four token rows (one address per 16-lane group)
                const f32x4 gs = *(const f32x4*)(&scale_tile[g][i * 16 + 4 * j]);
#pragma unroll
                for (int h = 0; h < TPW; ++h) {
                    f32x4 d = {0.f, 0.f, 0.f, 0.f};
                    d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0.b, qf[h][2 * g].b, d, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1.b, qf[h][2 * g + 1].b, d, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        s[i][h][r] = fmaf(d[r], gs[r], s[i][h][r]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0); // bound the number of LDS fragments kept live
            }
        }
        // ---- online softmax per head column ---------------------------------------------------------
        float pr[TPW][8];
        bool rescale = false;
        float alpha[TPW];
#pragma unroll
        for (int h = 0; h < TPW; ++h) {
            float sc[8];
            float step_max = kNegInf;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const unsigned int token = t0 + 16u * (e >> 2) + 4u * j + (e & 3);
                sc[e] = token < len ? s[e >> 2][h][e & 3] * scale_log2 : kNegInf;
                step_max = fmaxf(step_max, sc[e]);
            }
            step_max = wave_max_16x4(step_max);
            // lazy rescaling: the stored maximum only moves when a score exceeds it by the slack
            float new_max = run_max[h];
            if (step_max > run_max[h] + kRescaleSlack || run_max[h] == kNegInf) {
                new_max = fmaxf(run_max[h], step_max);
            }
            const float safe_max = new_max == kNegInf ? 0.0f : new_max;
            alpha[h] = __builtin_amdgcn_exp2f(run_max[h] - safe_max);
            rescale = rescale || (alpha[h] != 1.0f && run_sum[h] != 0.0f);
            float step_sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                pr[h][e] = __builtin_amdgcn_exp2f(sc[e] - safe_max);
                step_sum += pr[h][e];
            }
            run_sum[h] = run_sum[h] * alpha[h] + step_sum;
            run_max[h] = new_max;
        }
        if (__any(rescale)) {
#pragma unroll
            for (int h = 0; h < TPW; ++h) {
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    acc[h][t] *= alpha[h];
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- O^T += codes^T . P'_g,  P'_g = bf16(p * scale_g) --------------------------------------
        const unsigned char* pv_tile = tile + dsplit * (MT / 4) * 128;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            const float* gs_row = scale_tile[dsplit * GROUPS + g];
            const f32x4 gs0 = *(const f32x4*)(gs_row + 4 * j);
            const f32x4 gs1 = *(const f32x4*)(gs_row + 16 + 4 * j);
            Frag pf[TPW];
#pragma unroll
            for (int h = 0; h < TPW; ++h) {
                pf[h].u[0] = pack_bf16_rne(pr[h][0] * gs0[0], pr[h][1] * gs0[1]);
                pf[h].u[1] = pack_bf16_rne(pr[h][2] * gs0[2], pr[h][3] * gs0[3]);
                pf[h].u[2] = pack_bf16_rne(pr[h][4] * gs1[0], pr[h][5] * gs1[1]);
                pf[h].u[3] = pack_bf16_rne(pr[h][6] * gs1[2], pr[h][7] * gs1[3]);
            }
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) {
                const int t = g * 4 + tt;
                const unsigned char* at = pv_tile + pv_base[tt] + g * 128;
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(at));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(at + 16 * kRowBytes));
                union {
                    s16x4 s[2];
                    bf16x8 b;
                } vf;
                vf.s[0] = lo;
                vf.s[1] = hi;
#pragma unroll
                for (int h = 0; h < TPW; ++h) {
                    acc[h][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pf[h].b, acc[h][t], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- pipeline: global loads of step n+1 overlap the MFMA work of step n; LDS double-buffered
    StepRegs regs;
    load_step(regs, c_start);
    store_step(regs, lds, lds_scale[0]);
    __syncthreads();
    for (unsigned int step = 0; step < steps; ++step) {
        unsigned char* cur = lds + (step & 1u) * kTileBytes;
        unsigned char* nxt = lds + ((step + 1u) & 1u) * kTileBytes;
        const bool more = step + 1 < steps;
        if (more) {
            load_step(regs, c_start + (step + 1u) * kStepTokens);
        }
        compute_step(cur, lds_scale[step & 1u], c_start + step * kStepTokens);
        if (more) {
            store_step(regs, nxt, lds_scale[(step + 1u) & 1u]);
        }
        __syncthreads();
    }

    // ---- write un-normalised partials and (max, sum) -------------------------------------------
#pragma unroll
    for (int h = 0; h < TPW; ++h) {
        const unsigned int head = head_base + 16u * h + m;
        const float total = wave_sum_16x4(run_sum[h]);
        if (head < p.heads) {
            const size_t rec = ((size_t)b * p.max_chunks + chunk) * p.heads + head;
            if (j == 0 && dsplit == 0) {
                p.stats[rec * 2] = run_max[h];
                p.stats[rec * 2 + 1] = total;
            }
            float* out = p.partial + rec * kLatent + dsplit * (MT * 16);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                *(f32x4*)(out + t * 16 + 4 * j) = acc[h][t];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// 4. project value
// ---------------------------------------------------------------------------------------------
// grid = (heads, batch), 256 threads = 4 waves; each wave produces value columns v = wave, wave+4, ...
// with a 64-lane dot over the 512 latent columns.
__global__ __launch_bounds__(256) void mla_project(MlaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int wave = threadIdx.x >> 6;
    const float* weighted = p.weighted + ((size_t)b * p.heads + head) * p.latent_dim;
    const unsigned short* w = p.kv_b + ((size_t)head * p.kv_head_dim + p.nope_dim) * p.latent_dim;
    const unsigned int out_stride = p.out_compact ? p.value_dim : p.q_head_dim;
    const size_t out_base = ((size_t)b * p.heads + head) * out_stride;
    for (unsigned int v = wave; v < p.value_dim; v += 4) {
        float sum = 0.0f;
        for (unsigned int c = lane; c < p.latent_dim; c += 64) {
            sum = fmaf(weighted[c], bf16_bits_to_f32(w[(size_t)v * p.latent_dim + c]), sum);
        }
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) {
            sum += __shfl_xor(sum, offset);
        }
        if (lane == 0) {
            if (p.out_dtype == 0) {
                ((float*)p.out)[out_base + v] = sum;
            } else {
                ((unsigned short*)p.out)[out_base + v] = f32_to_bf16_bits(sum);
            }
        }
    }
}

} // namespace

hipError_t launch_mla_decode(const MlaDecodeParams& p, unsigned int stage_mask, hipStream_t stream)
{
    const unsigned int stages = stage_mask == 0 ? 15u : stage_mask;
    hipError_t err = hipSuccess;
    if (stages & 1u) {
        mla_absorb<<<dim3(p.heads, p.batch), dim3(256), 0, stream>>>(p);
        err = hipGetLastError();
        if (err != hipSuccess) {
            return err;
        }
    }
    if (stages & 2u) {
        if (p.heads > 64) {
            mla_partial<2, 2><<<dim3(p.max_chunks, 2 * ((p.heads + 127) / 128), p.batch), dim3(256), 0, stream>>>(p);
        } else {
            mla_partial<1, 1><<<dim3(p.max_chunks, 1, p.batch), dim3(256), 0, stream>>>(p);
        }
        err = hipGetLastError();
        if (err != hipSuccess) {
            return err;
        }
    }
    if (stages & 4u) {
        // LSE combine into weighted[b, h, 0:512] (f32)
        GqaDecodeParams mp = {};
        mp.kv_lens = p.ctx_lens;
        mp.first_visible = nullptr;
        mp.out = p.weighted;
        mp.partial = p.partial;
        mp.stats = p.stats;
        mp.batch = p.batch;
        mp.num_heads = p.heads;
        mp.head_dim = p.latent_dim;
        mp.chunk_tokens = p.chunk_tokens;
        mp.max_chunks = p.max_chunks;
        err = launch_split_merge(mp, stream);
        if (err != hipSuccess) {
            return err;
        }
    }
    if (stages & 8u) {
        mla_project<<<dim3(p.heads, p.batch), dim3(256), 0, stream>>>(p);
        err = hipGetLastError();
    }
    return err;
}

} // namespace zllm

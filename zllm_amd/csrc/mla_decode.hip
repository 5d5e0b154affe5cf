// Absorbed MLA decode over the paged Q8g64 latent cache — gfx950, f16 / bf16 MFMA.
//
// Stages (the reference's chain absorb -> partial -> merge -> project,
// src/kernel/rocm/hip/attention/paged_mla.rs:3042-3621):
//   1. mla_absorb:  qa[b, h, 0:512] = bf16(q_nope[b, h, :] . W_kv_b[h, 0:nope, :]),
//                   qa[b, h, 512:576] = bf16(q_rope[b, h, :])
//   2. mla_partial_ws: split-KV attention of the heads against one shared latent row per token.
//                   A workgroup owns (split, block of 64 heads, sequence).  Per 32-token step it converts
//                   the latent codes ONCE into LDS as f16 integers (exact) next to the bf16 rope columns,
//                   the f32 group scales and an f16 copy of them divided by the value side's exponent window.
//                   Four score waves (16 heads each) compute
//                     S^T[token, head]  = sum_g scale[token, g] * (codes_g[token, :] . qa_g[head, :])
//                                         + rope[token, :] . q_rope[head, :]     (MFMA 16x16x32 f16 on the
//                                         latent part, bf16 on the rope part; one accumulator per 64-column
//                                         group: products are exact)
//                   and the online softmax; four value waves, one step behind, accumulate
//                     O^T[dim, head]   += codes^T[dim, token] . P'_g[token, head],
//                     P'_g = f16(p) * f16(scale_g / 2^window)   (one packed f16 multiply per two tokens)
//                   The same row-major tile feeds both products: QK^T reads it with ds_read_b128,
//                   P.V reads it transposed with ds_read_b64_tr_b16.  A 16-byte XOR swizzle keeps both
//                   access patterns free of bank conflicts.
//   3. split merge by log-sum-exp (shared with GQA decode)
//   4. mla_project: out[b, h, v] = weighted[b, h, :] . W_kv_b[h, nope + v, :]
#include <string.h>
#include <type_traits>

#include "common.hpp"
#include "kernels.hpp"
#include "mla_rows.hpp"

namespace zllm {

namespace {

// Fences for the instruction scheduler between phases of a step: without them LDS fragment loads of
// later phases are hoisted to the top and the kernel spills.
#define MLA_PHASE_FENCE() __builtin_amdgcn_sched_barrier(0)

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
    f16x8 h;
};

// Chunk swizzle for the 64-bank LDS (256 B per cycle).  A tile row is 72 chunks of 16 B, i.e. 8 chunks past a
// multiple of 256 B, so the row's parity already selects the upper or lower 128 B of a bank line; XOR-ing
// row bits 1 and 2 into chunk bits 1 and 2 spreads eight rows over all sixteen 16-byte slots.  Measured with
// the LDS bank-conflict counter: ds_read_b128 of the K operand (lanes = 16 rows x 4 k-slices) 4.0 cycles and
// ds_read_b64_tr_b16 of the V operand 2.0 cycles per instruction, both conflict-free (the earlier swizzle,
// laid out for 32 banks, took 8 and 4).
__device__ __forceinline__ unsigned int swz(unsigned int row)
{
    return row & 6u;
}

__device__ __forceinline__ unsigned int tile_offset(unsigned int row, unsigned int chunk)
{
    return row * kRowBytes + ((chunk ^ swz(row)) << 4);
}

// ---------------------------------------------------------------------------------------------
// 1. absorb
// ---------------------------------------------------------------------------------------------
// grid = (heads, batch, z), 256 / z threads, z = 1 or 4; a thread owns two adjacent latent columns, the z workgroups of a
// (row, head) take the runs of 256 / z column pairs in turn.  A decode call of one sequence has as many (row, head) pairs
// as heads: with z = 4 the weights of a head are fetched by four compute units, 128 load instructions each, instead of
// 512 on one (one sequence of 32 heads: 6.7 -> 4.7 us); from a few hundred pairs on the compute units are busy either
// way and one workgroup per pair is the shorter launch (config 4, 512 pairs: 7.7 against 8.3 us).
// The sum runs over k in ascending order with separately rounded multiply and add, the order of
// the reference's scalar matmul (src/kernel/cpu/mla.rs:712-728); the result is rounded to bf16
// (mla.rs:1037).
__global__ __launch_bounds__(256) void mla_absorb(MlaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    __shared__ float q_sh[1024];
    const size_t q_base = ((size_t)b * p.heads + head) * p.q_head_dim;
    for (unsigned int i = threadIdx.x; i < p.q_head_dim; i += blockDim.x) {
        float x = load_as_f32(p.q, q_base + i, p.q_dtype);
        // the oracle takes a bf16 query (src/kernel/cpu/mla.rs:958-961)
        q_sh[i] = bf16_bits_to_f32(f32_to_bf16_bits(x));
    }
    unsigned short* qa = p.absorbed + ((size_t)b * p.heads + head) * (p.latent_dim + p.rope_dim);
    // a thread owns two adjacent latent columns: one 4-byte weight load per k (the sums themselves stay strictly
    // sequential in k)
    const unsigned int pairs = p.latent_dim / 2u;
    const unsigned int* w = (const unsigned int*)(p.kv_b + (size_t)head * p.kv_head_dim * p.latent_dim);
    // the usual geometries (latent 512; nope 128, or 192 as in the reference's own decode test): all weight words of the
    // thread are requested at once, before the query has even arrived in LDS -- the kernel is one memory round trip long
    // instead of one per 32 query elements
    auto one_trip = [&](auto nope) __attribute__((always_inline)) {
        constexpr int NOPE = decltype(nope)::value;
        const unsigned int c2 = blockIdx.z * blockDim.x + threadIdx.x;
        unsigned int word[NOPE];
#pragma unroll
        for (int k = 0; k < NOPE; ++k) {
            word[k] = w[(size_t)k * 256u + c2];
        }
        __syncthreads();
        {
            // product and sum rounded separately, as in the CPU code
#pragma clang fp contract(off)
            float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
            for (int k = 0; k < NOPE; ++k) {
                acc0 = acc0 + q_sh[k] * __uint_as_float(word[k] << 16);
                acc1 = acc1 + q_sh[k] * __uint_as_float(word[k] & 0xffff0000u);
            }
            *(unsigned int*)(qa + 2u * c2) = (unsigned int)f32_to_bf16_bits(acc0) | ((unsigned int)f32_to_bf16_bits(acc1) << 16);
        }
    };
    if (pairs == 256u && p.nope_dim == 128u) {
        one_trip(std::integral_constant<int, 128>{});
    } else if (pairs == 256u && p.nope_dim == 192u) {
        one_trip(std::integral_constant<int, 192>{});
    } else {
        __syncthreads();
        for (unsigned int c2 = blockIdx.z * blockDim.x + threadIdx.x; c2 < pairs; c2 += 256) {
            // product and sum rounded separately, as in the CPU code (plain operators: the __fmul_rn / __fadd_rn intrinsics
            // are ordinary operators from a header compiled with fusing allowed)
#pragma clang fp contract(off)
            float acc0 = 0.0f, acc1 = 0.0f;
            for (unsigned int k0 = 0; k0 < p.nope_dim; k0 += 32u) {
                unsigned int word[32];
#pragma unroll
                for (int u = 0; u < 32; ++u) {
                    word[u] = w[(size_t)min(k0 + u, p.nope_dim - 1u) * pairs + c2];
                }
#pragma unroll
                for (int u = 0; u < 32; ++u) {
                    if (k0 + u < p.nope_dim) {
                        acc0 = acc0 + q_sh[k0 + u] * __uint_as_float(word[u] << 16);
                        acc1 = acc1 + q_sh[k0 + u] * __uint_as_float(word[u] & 0xffff0000u);
                    }
                }
            }
            *(unsigned int*)(qa + 2u * c2) = (unsigned int)f32_to_bf16_bits(acc0) | ((unsigned int)f32_to_bf16_bits(acc1) << 16);
        }
    }
    if (blockIdx.z == 0u) {
        for (unsigned int r = threadIdx.x; r < p.rope_dim; r += blockDim.x) {
            qa[p.latent_dim + r] = f32_to_bf16_bits(q_sh[p.nope_dim + r]);
        }
    }
}

// The same absorb for a prefill chunk: a workgroup takes R query rows of one head, so a weight word read from memory
// serves R rows (with one row per workgroup a 2,048-row chunk reads the 16 MiB of absorb weights 2,048 times).  Every
// row's sum still runs over k in ascending order with separately rounded products: the bits are those of mla_absorb.
template <int R> __global__ __launch_bounds__(256) void mla_absorb_rows(MlaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int row0 = blockIdx.y * R;
    __shared__ float q_sh[R][256]; // the nope part of a head's query (at most 256 columns on this path)
    for (unsigned int i = threadIdx.x; i < R * p.q_head_dim; i += 256) {
        const unsigned int r = i / p.q_head_dim, c = i % p.q_head_dim;
        const unsigned int row = min(row0 + r, p.batch - 1u);
        const float x = load_as_f32(p.q, ((size_t)row * p.heads + head) * p.q_head_dim + c, p.q_dtype);
        const float rounded = bf16_bits_to_f32(f32_to_bf16_bits(x));
        if (c < p.nope_dim) {
            q_sh[r][c] = rounded;
        } else if (row0 + r < p.batch) {
            p.absorbed[((size_t)row * p.heads + head) * (p.latent_dim + p.rope_dim) + p.latent_dim + (c - p.nope_dim)] = f32_to_bf16_bits(rounded);
        }
    }
    __syncthreads();
    const unsigned int pairs = p.latent_dim / 2u;
    const unsigned int* w = (const unsigned int*)(p.kv_b + (size_t)head * p.kv_head_dim * p.latent_dim);
    for (unsigned int c2 = threadIdx.x; c2 < pairs; c2 += 256) {
#pragma clang fp contract(off)
        float acc0[R], acc1[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            acc0[r] = 0.0f;
            acc1[r] = 0.0f;
        }
        for (unsigned int k0 = 0; k0 < p.nope_dim; k0 += 16u) {
            unsigned int word[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                word[u] = w[(size_t)min(k0 + u, p.nope_dim - 1u) * pairs + c2];
            }
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                if (k0 + u < p.nope_dim) {
                    const float w0 = __uint_as_float(word[u] << 16), w1 = __uint_as_float(word[u] & 0xffff0000u);
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const float x = q_sh[r][k0 + u];
                        acc0[r] = acc0[r] + x * w0;
                        acc1[r] = acc1[r] + x * w1;
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (row0 + r < p.batch) {
                unsigned short* qa = p.absorbed + ((size_t)(row0 + r) * p.heads + head) * (p.latent_dim + p.rope_dim);
                *(unsigned int*)(qa + 2u * c2) = (unsigned int)f32_to_bf16_bits(acc0[r]) | ((unsigned int)f32_to_bf16_bits(acc1[r]) << 16);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// absorb and projection on the matrix cores, for calls of sixteen rows and more
// ---------------------------------------------------------------------------------------------
// The per-row kernels keep the oracle's summation order and cost a multiply and an add per weight and row on the vector
// ALU: 28 us of absorb and 23 us of projection for 32 rows, more than the attention between them at short contexts.
// With sixteen rows a workgroup the two are small GEMMs, (16 x 128).(128 x 512) and (16 x 512).(512 x 128) per head.
// Products of bf16 values are exact in f32 and only the order of the f32 sum differs from the oracle's, so an absorbed
// query differs from the bit-exact one by a bf16 step in a few elements out of a million.

// W_k[head] (nope rows of bf16) lies in LDS as in memory, rows padded by 16 bytes: the sixteen rows a transposed read
// touches then start in different banks.  128 query columns x 512 latent columns are 133 KB; 192 query columns (the
// reference's decode test, src/kernel/rocm/hip/attention/paged_mla.rs:6226-6233) x 256, half the latent columns, 101 KB.

// absorbed^T[n, row] = sum_k W_k[k, n] q[row, k].  A operand: W_k^T fragments through ds_read_b64_tr_b16 (lane (m, j) gets
// column n = 16 nt + m at k = 4 j .. 4 j + 3 and 16 + 4 j .. 16 + 4 j + 3 of a 32-k step); B operand: the query row m at
// the same k.  grid = (heads, workgroups per head), 4 or 16 waves; a workgroup stages the head's weights once and its
// waves take blocks of sixteen rows in turn, a wave (or the 2 to 16 waves that share a block) all 512 latent columns.
// NOPE query columns and COLS latent columns a workgroup: 128 x 512, or 192 x 256 with the two column halves in
// workgroups of their own (blockIdx.z), which is what fits the LDS.
template <int WAVES, int NOPE, int COLS> __global__ __launch_bounds__(64 * WAVES) void mla_absorb_mfma(MlaDecodeParams p)
{
    constexpr int kRowBytes = COLS * 2 + 16; // LDS bytes of one weight row: sixteen rows start in different banks
    constexpr int kRowChunks = COLS / 8;     // its 16-byte chunks
    const unsigned int col0 = blockIdx.z * COLS;
    __shared__ __align__(16) unsigned char w_lds[NOPE * kRowBytes];
    const unsigned int head = blockIdx.x;
    const unsigned int tid = threadIdx.x;
    const unsigned int lane = tid & 63u;
    const unsigned int wave = tid >> 6;
    constexpr unsigned int waves = WAVES;
    const unsigned int m = lane & 15u;
    const unsigned int j = lane >> 4;
    {
        const unsigned char* w = (const unsigned char*)(p.kv_b + (size_t)head * p.kv_head_dim * kLatent + col0);
        // NOPE * COLS / 8 16-byte chunks (chunk c % kRowChunks of weight row c / kRowChunks), all of a thread's requested
        // before any is stored
        constexpr int kPerThread = NOPE * kRowChunks / (64 * WAVES);
        static_assert(NOPE * kRowChunks % (64 * WAVES) == 0, "whole chunks per thread");
        u32x4 staged[kPerThread];
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            const unsigned int c = tid + 64u * WAVES * i;
            staged[i] = *(const u32x4*)(w + (size_t)(c / kRowChunks) * (kLatent * 2) + (c % kRowChunks) * 16u);
        }
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            const unsigned int c = tid + 64u * WAVES * i;
            *(u32x4*)(w_lds + (c / kRowChunks) * kRowBytes + (c % kRowChunks) * 16u) = staged[i];
        }
    }
    __syncthreads();
    // The staged weights serve every block of sixteen rows the workgroup takes.  The weights leave room for one workgroup
    // per compute unit, so its waves are all the loads a compute unit has in flight: four waves walking the blocks one
    // after the other ran the stage at 1.9 TB/s.  Every wave takes blocks of its own, all 512 latent columns of them; when
    // the workgroup has fewer blocks than waves, 2, 4, 8 or 16 waves share a block and split its columns.
    const unsigned int share = p.column_split;           // waves per block
    const unsigned int slots = waves / share;            // blocks the workgroup has in flight
    const unsigned int tiles = (COLS / 16u) / share;     // 16-column tiles of a wave
    const unsigned int tile0 = (wave % share) * tiles;
    const unsigned char* frag_at = w_lds + (4u * j + (m >> 2)) * kRowBytes + (m & 3u) * 8u;
    for (unsigned int row0 = (blockIdx.y * slots + wave / share) * 16u; row0 < p.batch; row0 += gridDim.y * slots * 16u) {
        const unsigned int row = min(row0 + m, p.batch - 1u);
        const size_t q_base = ((size_t)row * p.heads + head) * p.q_head_dim;
        // four consecutive query elements per load, rounded to bf16: the oracle takes a bf16 query (src/kernel/cpu/mla.rs:958-961)
        auto four_as_bf16 = [&](size_t at) __attribute__((always_inline)) -> u32x2 {
            if (p.q_dtype == 1) {
                return *(const u32x2*)((const unsigned short*)p.q + at);
            }
            if (p.q_dtype == 0) {
                const f32x4 x = *(const f32x4*)((const float*)p.q + at);
                return u32x2{pack_bf16_rne(x[0], x[1]), pack_bf16_rne(x[2], x[3])};
            }
            const u32x2 h = *(const u32x2*)((const unsigned short*)p.q + at);
            return u32x2{pack_bf16_rne(f16_bits_to_f32((unsigned short)(h[0] & 0xffffu)), f16_bits_to_f32((unsigned short)(h[0] >> 16))),
                         pack_bf16_rne(f16_bits_to_f32((unsigned short)(h[1] & 0xffffu)), f16_bits_to_f32((unsigned short)(h[1] >> 16)))};
        };
        Frag qf[NOPE / 32];
#pragma unroll
        for (int ks = 0; ks < NOPE / 32; ++ks) {
            const u32x2 lo = four_as_bf16(q_base + ks * 32u + 4u * j), hi = four_as_bf16(q_base + ks * 32u + 16u + 4u * j);
            qf[ks].u = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
        // the rope part of the sixteen rows is a copy: lane = column, one row a pass, the rows dealt out to the block's waves
        {
            const unsigned int part = wave % share + share * blockIdx.z; // of share * gridDim.z waves on this block
            float rope_in[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const unsigned int r = min(row0 + i, p.batch - 1u);
                if ((i & (share * gridDim.z - 1u)) == part) {
                    rope_in[i] = load_as_f32(p.q, ((size_t)r * p.heads + head) * p.q_head_dim + NOPE + lane, p.q_dtype);
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                if ((i & (share * gridDim.z - 1u)) == part && row0 + i < p.batch) {
                    p.absorbed[((size_t)(row0 + i) * p.heads + head) * (kLatent + kRope) + kLatent + lane] = f32_to_bf16_bits(rope_in[i]);
                }
            }
        }
        unsigned short* qa = p.absorbed + ((size_t)(row0 + m) * p.heads + head) * (kLatent + kRope) + col0 + 4u * j;
        for (unsigned int nt = tile0; nt < tile0 + tiles; ++nt) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < NOPE / 32; ++ks) {
                union {
                    s16x4 s[2];
                    bf16x8 b;
                } wf;
                const unsigned char* at = frag_at + ks * 32 * kRowBytes + nt * 32u;
                wf.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(at));
                wf.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(at + 16 * kRowBytes));
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf.b, qf[ks].b, acc, 0, 0, 0);
            }
            if (row0 + m < p.batch) { // lane (m, j) holds latent columns 16 nt + 4 j .. + 4 of row m
                *(u32x2*)(qa + nt * 16u) = u32x2{pack_bf16_rne(acc[0], acc[1]), pack_bf16_rne(acc[2], acc[3])};
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// 2. split-KV partial
// ---------------------------------------------------------------------------------------------
// Workgroup barrier for LDS traffic only.  __syncthreads() also waits for the global loads in flight
// (s_waitcnt vmcnt(0)), which would drain the prefetch of the next step at every barrier; what those loads
// bring is consumed by the issuing thread alone, one iteration later.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

constexpr int kItemsMax = 4;

// Block-table entries of a thread's staging items: fetched one step before the loads that use them, so
// nothing waits on a table -> data chain.  Slot ITEMS belongs to the rope role (threads 0..255) or the
// scale role (threads 256..511).
struct StepRows {
    unsigned int entry[kItemsMax + 1];
    // selected-token mode only: the token positions behind `entry`, and those of the step after (fetched one
    // step earlier still, so that neither the selection list nor the block table is waited for)
    unsigned int token[kItemsMax + 1];
    unsigned int next_token[kItemsMax + 1];
};


// Workgroup = (split, block of 64 heads, sequence), eight waves in two roles that run one step apart:
//   score waves (0..3, 16 heads each): S^T = K.Q^T for all 32 tokens of tile i, online softmax, and hand
//       the step's probabilities p[32 tokens] and the rescale factor alpha to their value wave through LDS.
//       The C layout of S^T is the B layout the value wave needs, so the hand-over is lane to lane.
//   value waves (4..7): O^T += V^T.P' for tile i - 1; each owns two head tiles x 256 output columns, so that
//       every V^T fragment read from LDS feeds two MFMAs.
// The score work is LDS reads + vector ALU (exp, max), the value work LDS reads + MFMA; with one wave of each
// role per SIMD the two overlap instead of every wave running the same phase at the same time, and the
// score exchange between waves of a head tile (a second barrier per step) disappears.  Three tile buffers
// rotate: tile i (scores), tile i - 1 (values), tile i + 1 (being converted from the bytes the threads loaded
// an iteration ago).  One LDS-only barrier per step.
constexpr int kWsTiles = 3;
// The probabilities travel from the score to the value waves as f16 of p * 2^kPShift (p <= 2^8 by the lazy rescaling, so
// the product stays below 2^13 and p down to 2^-18 keeps f16's full precision); the f16 copy of the scale table carries
// the inverse, so that P' = p16 * scale16 is one packed multiply per two tokens.
constexpr int kPShift = 4;

// ALIGNED: pages hold a multiple of 32 tokens (splits always start at one), so the 32 rows of a step are
// contiguous in one page: one block-table entry per step, and every staging load takes a scalar base
// plus a constant per-lane offset -- no vector address arithmetic in the loop.  Rows past the end of the
// sequence are then whatever the page holds; their scales are zeroed during conversion and their scores
// masked, so they contribute exact zeros.
// SELECTED: the `selection` arm (src/kernel/rocm/hip/attention/paged_mla/source.hip:4738-4764): a sequence longer than
// top_k attends to the listed token positions only.  The kernel then walks list slots instead of positions -- splits,
// masks and softmax are over slots -- and only the address of a row goes through the list.
// POW2: the page size is a power of two and the sequences have block tables, known at compile time: the address
// arithmetic of a step is then shifts and masks without the run-time choice (and the division code behind it).
template <bool ALIGNED, bool SELECTED, bool POW2 = false, bool NARROW = false> __global__ __launch_bounds__(512) void mla_partial_ws(MlaDecodeParams p)
{
    static_assert(!(ALIGNED && SELECTED), "selected rows are not contiguous");
    // Staging items (token row, 16 codes) per thread: the 32 rows of a step are split 24 : 8 between the score and the
    // value waves, because the value waves' step is the longer one.  A score thread takes rows r, r + 8 and r + 16,
    // a value thread row 24 + r, with r = (thread % 256) / 32.
    constexpr int ITEMS = 3;
    __shared__ __align__(16) unsigned char lds[kWsTiles * kTileBytes];
    __shared__ __align__(16) float lds_scale[kWsTiles][8][kStepTokens]; // [buffer][group][token]
    __shared__ __align__(16) u32x4 lds_p16[2][4][64]; // [parity][head tile][lane]: the step's probabilities times 2^kPShift as
                                                      // f16, tokens (4j, 4j+1) (4j+2, 4j+3) (16+4j, ..) (16+4j+2, ..): 16-byte slots
                                                      // of consecutive lanes are contiguous (conflict-free 16-byte reads)
    __shared__ __align__(16) _Float16 lds_scale16[kWsTiles][8][kStepTokens]; // [buffer][group][token]: scale / 2^(window + kPShift)
    __shared__ int lds_win[kWsTiles];                    // the window lds_scale16[buffer] was written for
    __shared__ __align__(16) float lds_alpha[2][4][64];  // [parity][head tile][lane]; narrow: [parity][2 head tile + token half][lane],
                                                         // the running maximum the half's probabilities are relative to
    __shared__ float2 lds_final[2][16];                  // narrow: [head tile][head]: (maximum, sum) of the second token half
    __shared__ __align__(16) float lds_top[kWsTiles][4]; // [buffer][value wave]: largest group scale the wave converted
    const unsigned int tid = threadIdx.x;
    const unsigned int lane = tid & 63u;
    const unsigned int wave = tid >> 6;
    const bool value_role = wave >= 4u;
    const unsigned int hw = wave & 3u;
    const unsigned int m = lane & 15u;
    const unsigned int j = lane >> 4;
    // the split and the query row this workgroup works on: grid coordinates, or looked up from the dense item number.
    // Query rows run the last first: the rows of a chunk see more keys the later they come, and workgroups are handed
    // out in the order of their index
    unsigned int chunk = blockIdx.x;
    unsigned int b = gridDim.z - 1u - blockIdx.z;
    if (p.record_rows != 0u && !mla_locate_split(p, blockIdx.x, lane, b, chunk)) {
        return;
    }
    // NARROW (a call of at most 32 heads: head tiles 2 and 3 would be empty): the four score waves are two head tiles x
    // two halves of a step's tokens, each half with its own running maximum and sum, and every value wave takes both
    // head tiles and a quarter of the columns.
    const unsigned int score_tile = NARROW ? (hw & 1u) : hw; // head tile of a score wave
    const unsigned int stream = NARROW ? (hw >> 1) : 0u;     // narrow: which sixteen tokens of a step it scores
    const unsigned int head = blockIdx.y * 64u + score_tile * 16u + m; // this lane's head column
    unsigned int seq;
    unsigned int len = visible_tokens(p.ctx_lens, p.query_rows, b, seq); // keys of this row: positions, or list slots when a selection applies
    const unsigned int* selected = nullptr;
    if constexpr (SELECTED) {
        if (p.selection != nullptr && p.top_k < len) {
            selected = p.selection + (size_t)b * p.top_k;
            len = p.selection_counts != nullptr ? min(p.selection_counts[b], p.top_k) : p.top_k;
        }
    }
    // the planned split size is an upper bound: the sequence cuts its keys into equal 32-aligned parts, so a ragged
    // batch has no full-length splits next to short remainders
    const unsigned int n_splits = min(p.max_chunks, (len + p.chunk_tokens - 1u) / p.chunk_tokens);
    const unsigned int span = n_splits > 0u ? min(p.chunk_tokens, (((len + n_splits - 1u) / n_splits) + 31u) & ~31u) : p.chunk_tokens;
    const unsigned long long c_start64 = (unsigned long long)chunk * span;
    const size_t row = p.record_rows != 0u ? (size_t)blockIdx.x : (size_t)b * p.max_chunks + chunk;
    const size_t rec = row * p.heads + head;
    if (c_start64 >= len) { // empty split: (max, sum) = (-inf, 0), merge skips it
        if (head < p.heads && j == 0 && !value_role) {
            p.stats[rec * 2] = kNegInf;
            p.stats[rec * 2 + 1] = 0.0f;
        }
        return;
    }
    const unsigned int c_start = (unsigned int)c_start64;
    const unsigned int c_end = (unsigned int)min((unsigned long long)len, c_start64 + span);
    const unsigned int steps = (c_end - c_start + kStepTokens - 1) / kStepTokens;
    const unsigned int* table = (POW2 || p.tables != nullptr) ? p.tables + (size_t)seq * p.table_stride : nullptr;
    const bool pow2 = POW2 || (p.block_tokens & (p.block_tokens - 1u)) == 0;

    // ---- staging: loads of a later tile's bytes, converted by the thread that loaded them
    const unsigned int cc = tid & 31u;
    const unsigned int t_lo = (tid & 255u) >> 5;
    const int n_items = value_role ? 1 : 3;
    const unsigned int row_first = value_role ? 24u + t_lo : t_lo;      // row of item 0; item i is 8 i further on
    const unsigned int rope_t = (tid >> 3) & 31u;
    const unsigned int rope_c = tid & 7u;
    const bool has_rope = tid < 256u;
    const bool has_scales = tid >= 256u; // value-role threads: one (token, group) scale each
    const unsigned int scale_t = (tid - 256u) & 31u; // consecutive lanes write consecutive floats of a group's row
    const unsigned int scale_g = (tid - 256u) >> 5;
    const unsigned int extra_t = has_rope ? rope_t : scale_t;
    // selected-token mode: positions of the thread's items for the step that starts at slot t0
    auto fetch_tokens = [&](StepRows& r, unsigned int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i <= ITEMS; ++i) {
            if (i < n_items || i == ITEMS) {
                const unsigned int slot = min(t0 + (i < ITEMS ? row_first + 8u * i : extra_t), len - 1u);
                r.next_token[i] = selected != nullptr ? selected[slot] : slot;
            }
        }
    };
    auto lookup_step = [&](StepRows& r, unsigned int t0) __attribute__((always_inline)) {
        if constexpr (ALIGNED) {
            const unsigned int page = pow2 ? t0 >> p.block_shift : t0 / p.block_tokens;
            r.entry[0] = (POW2 || table != nullptr) ? table[page] : page;
        } else {
#pragma unroll
            for (int i = 0; i <= ITEMS; ++i) {
                if (i < n_items || i == ITEMS) {
                    unsigned int token = min(t0 + (i < ITEMS ? row_first + 8u * i : extra_t), len - 1u);
                    if constexpr (SELECTED) {
                        token = r.next_token[i]; // fetched a step ago for this t0
                        r.token[i] = token;
                    }
                    const unsigned int page = pow2 ? token >> p.block_shift : token / p.block_tokens;
                    r.entry[i] = table != nullptr ? table[page] : page;
                }
            }
            if constexpr (SELECTED) {
                fetch_tokens(r, t0 + kStepTokens);
            }
        }
    };
    auto row_of = [&](const StepRows& r, int i, unsigned int t0) __attribute__((always_inline)) -> unsigned long long {
        unsigned int token = min(t0 + (i < ITEMS ? row_first + 8u * i : extra_t), len - 1u);
        if constexpr (SELECTED) {
            token = r.token[i];
        }
        if (pow2) {
            return ((unsigned long long)r.entry[i] << p.block_shift) + (token & (p.block_tokens - 1u));
        }
        return (unsigned long long)r.entry[i] * p.block_tokens + token % p.block_tokens;
    };
    // The raw bytes of a step travel through registers: a thread loads its items (two runs of eight codes each), its rope piece
    // or one scale with plain loads and converts them itself one iteration later, so nothing is waited for
    // (a load has a whole iteration to land) and the conversion makes no LDS round trip before its writes.
    struct StageRegs {
        u32x4 codes[ITEMS];
        u32x4 extra; // rope piece (threads 0..255); threads 256..511 keep one scale (16 bits) in extra[0]
    };
    auto load_step = [&](StageRegs& regs, const StepRows& rows, unsigned int t0) __attribute__((always_inline)) {
        if constexpr (ALIGNED) {
            const unsigned int entry = __builtin_amdgcn_readfirstlane(rows.entry[0]);
            const unsigned long long row0 = pow2 ? ((unsigned long long)entry << p.block_shift) + (t0 & (p.block_tokens - 1u))
                                                 : (unsigned long long)entry * p.block_tokens + t0 % p.block_tokens;
            const unsigned char* codes = (const unsigned char*)p.latent_codes + row0 * kLatent;
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                if (i < n_items) { // codes 8 cc .. + 8 and 256 + 8 cc .. + 8 of the row
                    const unsigned char* at = codes + (row_first + 8u * i) * kLatent + cc * 8u;
                    const u32x2 lo = *(const u32x2*)(at), hi = *(const u32x2*)(at + 256);
                    regs.codes[i] = u32x4{lo[0], lo[1], hi[0], hi[1]};
                }
            }
            if (has_rope) {
                regs.extra = *(const u32x4*)((const unsigned char*)p.rope_cache + row0 * (kRope * 2) + tid * 16u);
            }
            if (has_scales) {
                regs.extra[0] = *(const unsigned short*)((const unsigned char*)p.latent_scales + (row0 + scale_t) * (kLatent / 64 * 2) + scale_g * 2u);
            }
        } else {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                if (i < n_items) {
                    const signed char* at = p.latent_codes + row_of(rows, i, t0) * kLatent + cc * 8u;
                    const u32x2 lo = *(const u32x2*)(at), hi = *(const u32x2*)(at + 256);
                    regs.codes[i] = u32x4{lo[0], lo[1], hi[0], hi[1]};
                }
            }
            if (has_rope) {
                regs.extra = *(const u32x4*)(p.rope_cache + row_of(rows, ITEMS, t0) * kRope + rope_c * 8u);
            }
            if (has_scales) {
                regs.extra[0] = p.latent_scales[row_of(rows, ITEMS, t0) * (kLatent / 64) + scale_g];
            }
        }
    };
    int window = 0; // value waves: exponent window of P' (see below); the f16 scale table is written for the window of the moment
    auto convert_step = [&](const StageRegs& regs, unsigned char* tile, float (*scale_tile)[kStepTokens], _Float16 (*scale16_tile)[kStepTokens],
                            int* table_window, float* step_top, unsigned int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            if (i >= n_items) {
                break;
            }
            // codes 8 cc .. + 8 and 256 + 8 cc .. + 8 -> chunks cc and cc + 32 of the row: 32 consecutive lanes write 512
            // contiguous bytes per instruction, which the LDS takes without conflicts (chunks 2 cc and 2 cc + 1, the
            // natural output of one 16-byte load, measured a two-way conflict on every write: sixteen lanes go per cycle)
            const unsigned int row = row_first + 8u * i;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                u32x4 out;
#pragma unroll
                for (int w = 0; w < 2; ++w) {
                    unsigned int pair_lo, pair_hi;
                    codes4_to_f16(regs.codes[i][h * 2 + w], pair_lo, pair_hi);
                    out[w * 2] = pair_lo;
                    out[w * 2 + 1] = pair_hi;
                }
                *(u32x4*)(tile + tile_offset(row, cc + 32u * h)) = out;
            }
        }
        if (has_rope) {
            *(u32x4*)(tile + tile_offset(rope_t, 64u + rope_c)) = regs.extra;
        }
        if (has_scales) {
            float sg = bf16_bits_to_f32((unsigned short)regs.extra[0]);
            if (t0 + scale_t >= len) {
                sg = 0.0f; // a row past the end: its codes may be anything, its weight is an exact zero
            }
            scale_tile[scale_g][scale_t] = sg;
            // out of the window's range the product overflows to infinity: such a step moves the window, and a table whose
            // window is not the reader's is not used
            scale16_tile[scale_g][scale_t] = (_Float16)(sg * __uint_as_float((unsigned int)(127 - kPShift - window) << 23));
            if (tid == 256u) {
                *table_window = window;
            }
            // largest scale the wave holds, for the value waves' exponent window: rotate-and-max inside the four
            // 16-lane rows, then one lane of each row
            float top = sg;
            top = fmaxf(top, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(top), 0x128, 0xf, 0xf, false))); // row_ror:8
            top = fmaxf(top, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(top), 0x124, 0xf, 0xf, false))); // row_ror:4
            top = fmaxf(top, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(top), 0x122, 0xf, 0xf, false))); // row_ror:2
            top = fmaxf(top, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(top), 0x121, 0xf, 0xf, false))); // row_ror:1
            const float rows01 = fmaxf(__uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 0)),
                                       __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 16)));
            const float rows23 = fmaxf(__uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 32)),
                                       __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 48)));
            if (lane == 0u) {
                step_top[hw] = fmaxf(rows01, rows23);
            }
        }
    };

    // LDS byte offsets of this lane's fragments (lane part; the rest is compile-time)
    const unsigned int qk_base[2] = {m * kRowBytes + ((j ^ swz(m)) << 4), m * kRowBytes + (((4u | j) ^ swz(m)) << 4)};
    const unsigned int tr_row = 4u * j + (m >> 2);
    unsigned int pv_base[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        pv_base[q] = tr_row * kRowBytes + ((((unsigned int)q << 1 | ((m & 3u) >> 1)) ^ swz(tr_row)) << 4) + (m & 1u) * 8u;
    }

    StepRows rows = {};
    if constexpr (SELECTED) {
        fetch_tokens(rows, c_start);
    }
    lookup_step(rows, c_start);
    StageRegs staged;
    load_step(staged, rows, c_start);
    if (steps > 1) {
        lookup_step(rows, c_start + kStepTokens);
    }
    convert_step(staged, lds, lds_scale[0], lds_scale16[0], &lds_win[0], lds_top[0], c_start);
    lds_barrier();

    // Both roles run the same number of iterations and barriers: iteration i scores tile i and accumulates tile
    // i - 1.  The roles are half a step out of phase: a score wave requests step i + 1 first, scores tile i (matrix
    // work) and converts step i + 1 last; a value wave converts step i + 1 first (requested an iteration ago),
    // requests step i + 2, and accumulates tile i - 1 (matrix work) last.  So the conversion and load-issue work of
    // one role runs under the matrix work of the other instead of all eight waves queueing at the load unit and
    // the LDS write port together.
    auto stage_step = [&](unsigned int n) __attribute__((always_inline)) { // request the raw bytes of step n
        if (n < steps) {
            // The entries were fetched an iteration ago.  Naming them here places the compiler's wait for them
            // before the first load of this iteration; left to itself it waits again before every address it
            // forms from them, i.e. for the load it has just issued.
            if constexpr (ALIGNED) {
                asm volatile("" : "+v"(rows.entry[0]));
            } else {
                asm volatile("" : "+v"(rows.entry[0]), "+v"(rows.entry[1]), "+v"(rows.entry[2]), "+v"(rows.entry[3]));
                if constexpr (SELECTED) {
                    asm volatile("" : "+v"(rows.token[0]), "+v"(rows.token[1]), "+v"(rows.token[2]), "+v"(rows.token[3]),
                                      "+v"(rows.next_token[0]), "+v"(rows.next_token[1]), "+v"(rows.next_token[2]), "+v"(rows.next_token[3]));
                }
            }
            load_step(staged, rows, c_start + n * kStepTokens);
            if (n + 1 < steps) {
                lookup_step(rows, c_start + (n + 1u) * kStepTokens);
            }
        }
    };
    auto convert_to = [&](unsigned int n) __attribute__((always_inline)) { // raw bytes of step n -> tile buffer n % 3
        if (n < steps) {
            const unsigned int nb = n % kWsTiles;
            convert_step(staged, lds + nb * kTileBytes, lds_scale[nb], lds_scale16[nb], &lds_win[nb], lds_top[nb], c_start + n * kStepTokens);
        }
    };

    if (!value_role) {
        // ================================ score waves ================================
        // B operand: lane = (head column m, k-slice j); k-step ks covers dims ks*32 + j*8 .. +8.  The latent part
        // multiplies f16 codes, so the absorbed query (bf16) is carried as f16 after dividing the head's row by the
        // power of two of its largest magnitude: exact for every element within 2^-14 of that magnitude, and free
        // of f16's range limit.  The rope part stays bf16 on both sides.
        Frag qf[18];
        float head_pow2 = 1.0f; // the power of two taken out of this head's latent query
        {
            const unsigned short* qa = p.absorbed + ((size_t)b * p.heads + min(head, p.heads - 1u)) * kRowElems;
#pragma unroll
            for (int ks = 0; ks < 18; ++ks) {
                u32x4 v = *(const u32x4*)(qa + ks * 32 + j * 8);
                if (head >= p.heads) {
                    v = u32x4{0u, 0u, 0u, 0u};
                }
                qf[ks].u = v;
            }
            float top = 0.0f;
#pragma unroll
            for (int ks = 0; ks < 16; ++ks) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    top = fmaxf(top, fmaxf(fabsf(__uint_as_float(qf[ks].u[w] << 16)), fabsf(__uint_as_float(qf[ks].u[w] & 0xffff0000u))));
                }
            }
            top = wave_max_16x4(top);
            const unsigned int top_exp = min(max((__float_as_uint(top) >> 23) & 0xffu, 1u), 253u);
            head_pow2 = __uint_as_float(top_exp << 23);
            const float down = __uint_as_float((254u - top_exp) << 23);
#pragma unroll
            for (int ks = 0; ks < 16; ++ks) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const unsigned int word = qf[ks].u[w];
                    qf[ks].u[w] = pack_f16_hw(__uint_as_float(word << 16) * down, __uint_as_float(word & 0xffff0000u) * down);
                }
            }
        }
        // narrow: a head tile past the last head stages and converts like the others and scores nothing
        const bool tile_live = !NARROW || (unsigned int)__builtin_amdgcn_readfirstlane((int)(score_tile * 16u)) < p.heads;
        float run_max = kNegInf, run_sum = 0.0f;
        float neg_ref = 0.0f; // minus the reference the scores are taken against: the running maximum, 0 before the first score
        float neg_ref_shifted = (float)kPShift; // the same plus the hand-over shift: the scores below are log2(p * 2^kPShift)
        const float scale_log2 = p.score_scale * kLog2e;
        const float latent_log2 = scale_log2 * head_pow2;
        stage_step(1u);
        for (unsigned int i = 0; i <= steps; ++i) {
            if constexpr (NARROW) {
                if (i < steps && tile_live) {
                    // sixteen tokens of the step: four batches of four k-steps (latent groups {0..3} first k-step, {0..3} second,
                    // {4..7} first, {4..7} second; the rope k-steps ride along with batch 0), fragments requested two batches ahead
                    const unsigned int tb = i % kWsTiles;
                    const unsigned char* tile = lds + tb * kTileBytes + stream * (16u * kRowBytes);
                    const float (*scale_tile)[kStepTokens] = lds_scale[tb];
                    const unsigned int t0 = c_start + i * kStepTokens + 16u * stream;
                    constexpr int kRing = 3, kAhead = kRing - 1;
                    Frag kf[kRing][4], kr[2];
                    f32x4 gsv[2][4];
                    auto load_batch = [&](int q) __attribute__((always_inline)) {
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            kf[q % kRing][u].u = *(const u32x4*)(tile + qk_base[q & 1] + ((q >> 1) * 4 + u) * 128);
                        }
                        if (q == 0) {
                            kr[0].u = *(const u32x4*)(tile + qk_base[0] + 8 * 128);
                            kr[1].u = *(const u32x4*)(tile + qk_base[1] + 8 * 128);
                        }
                        if (q & 1) {
#pragma unroll
                            for (int u = 0; u < 4; ++u) {
                                gsv[q >> 1][u] = *(const f32x4*)(&scale_tile[(q >> 1) * 4 + u][16u * stream + 4 * j]);
                            }
                        }
                    };
#pragma unroll
                    for (int q = 0; q < kAhead; ++q) {
                        load_batch(q);
                    }
                    f32x4 s = {0.f, 0.f, 0.f, 0.f};
                    f32x4 s_rope = {0.f, 0.f, 0.f, 0.f};
                    f32x4 d[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (q + kAhead < 4) {
                            load_batch(q + kAhead);
                        }
                        asm volatile("" ::: "memory"); // the requests above stay above the MFMAs below
                        if (q == 0) {
                            s_rope = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kr[0].b, qf[16].b, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                            s_rope = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kr[1].b, qf[17].b, s_rope, 0, 0, 0);
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int g = (q >> 1) * 4 + u;
                            if ((q & 1) == 0) {
                                d[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[q % kRing][u].h, qf[2 * g].h, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                            } else {
                                d[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[q % kRing][u].h, qf[2 * g + 1].h, d[u], 0, 0, 0);
                            }
                        }
                        if (q & 1) {
#pragma unroll
                            for (int u = 0; u < 4; ++u) {
                                const f32x4 gs = gsv[q >> 1][u];
#pragma unroll
                                for (int r = 0; r < 4; ++r) {
                                    s[r] = fmaf(d[u][r], gs[r], s[r]);
                                }
                            }
                        }
                    }
                    float sc[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        sc[r] = fmaf(s[r], latent_log2, fmaf(s_rope[r], scale_log2, neg_ref_shifted)); // relative to the reference
                    }
                    if (t0 + 16u > len) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            sc[r] = t0 + 4u * j + r < len ? sc[r] : kNegInf;
                        }
                    }
                    // the lazy online softmax of the wide layout: the reference is the largest score seen when it last moved, so
                    // the largest probability of a short or peaked row is exactly 1
                    const float lane_max = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
                    if (__any(lane_max > 8.0f + (float)kPShift || run_max == kNegInf)) {
                        const float step_max = wave_max_16x4(lane_max) - (float)kPShift;
                        const float ref = -neg_ref;
                        float new_max = run_max;
                        if (step_max > 8.0f || run_max == kNegInf) {
                            new_max = fmaxf(run_max, ref + step_max);
                        }
                        const float safe_max = new_max == kNegInf ? 0.0f : new_max;
                        const float delta = safe_max - ref;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            sc[r] -= delta;
                        }
                        run_sum *= __builtin_amdgcn_exp2f(run_max - safe_max); // 0 on the first step: nothing accumulated yet
                        run_max = new_max;
                        neg_ref = -safe_max;
                        neg_ref_shifted = neg_ref + (float)kPShift;
                    }
                    float pr[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        pr[r] = __builtin_amdgcn_exp2f(sc[r]);
                    }
                    // The sum takes the probabilities as the value waves will multiply them, rounded to f16: numerator and
                    // denominator of a row then carry the same weights.
                    typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
                    const unsigned int p01 = pack_f16_hw(pr[0], pr[1]), p23 = pack_f16_hw(pr[2], pr[3]);
                    const f16x2_t h01 = __builtin_bit_cast(f16x2_t, p01), h23 = __builtin_bit_cast(f16x2_t, p23);
                    run_sum += ((float)h01[0] + (float)h01[1]) + ((float)h23[0] + (float)h23[1]); // in units of 2^-kPShift
                    ((u32x2*)&lds_p16[i & 1u][score_tile][lane])[stream] = u32x2{p01, p23};
                    lds_alpha[i & 1u][2u * score_tile + stream][lane] = run_max; // -inf: nothing seen yet, the probabilities are zeros
                }
            } else if (i < steps) {
                const unsigned int tb = i % kWsTiles;
                const unsigned char* tile = lds + tb * kTileBytes;
                const float (*scale_tile)[kStepTokens] = lds_scale[tb];
                const unsigned int t0 = c_start + i * kStepTokens;
                float sc[8];
                // K fragments are requested kAhead batches (of four k-steps) ahead of the MFMAs that use them: an LDS
                // round trip under load is several batches of matrix work long, and nothing else hides it with two
                // waves per SIMD.  Batch b of a step: token tile b / 4; q = b % 4 -> latent groups {0..3} first
                // k-step, {0..3} second k-step, {4..7} first, {4..7} second; the two rope k-steps of a token tile
                // ride along with its batch 0.
                constexpr int kRing = 3, kAhead = kRing - 1;
                Frag kf[kRing][4], kr[2][2];
                f32x4 gsv[2][4]; // group scales of the odd batches (LDS returns in order: a late scale read would wait
                                 // for every fragment requested before it)
                auto load_batch = [&](int bt) __attribute__((always_inline)) {
                    const unsigned char* kt = tile + (bt >> 2) * 16 * kRowBytes;
                    const int q = bt & 3;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        kf[bt % kRing][u].u = *(const u32x4*)(kt + qk_base[q & 1] + ((q >> 1) * 4 + u) * 128);
                    }
                    if (q == 0) {
                        kr[bt >> 2][0].u = *(const u32x4*)(kt + qk_base[0] + 8 * 128);
                        kr[bt >> 2][1].u = *(const u32x4*)(kt + qk_base[1] + 8 * 128);
                    }
                    if (q & 1) {
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            gsv[(bt >> 1) & 1][u] = *(const f32x4*)(&scale_tile[(q >> 1) * 4 + u][(bt >> 2) * 16 + 4 * j]);
                        }
                    }
                };
#pragma unroll
                for (int bt = 0; bt < kAhead; ++bt) {
                    load_batch(bt);
                }
                f32x4 s = {0.f, 0.f, 0.f, 0.f};      // latent part, in units of head_pow2
                f32x4 s_rope = {0.f, 0.f, 0.f, 0.f}; // rope part
                f32x4 d[4];
#pragma unroll
                for (int bt = 0; bt < 8; ++bt) {
                    const int t2 = bt >> 2, q = bt & 3;
                    if (bt + kAhead < 8) {
                        load_batch(bt + kAhead);
                    }
                    asm volatile("" ::: "memory"); // the requests above stay above the MFMAs below
                    if (q == 0) {
                        s = f32x4{0.f, 0.f, 0.f, 0.f};
                        s_rope = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kr[t2][0].b, qf[16].b, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                        s_rope = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kr[t2][1].b, qf[17].b, s_rope, 0, 0, 0);
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int g = (q >> 1) * 4 + u;
                        if ((q & 1) == 0) {
                            d[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[bt % kRing][u].h, qf[2 * g].h, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                        } else {
                            d[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[bt % kRing][u].h, qf[2 * g + 1].h, d[u], 0, 0, 0);
                        }
                    }
                    if ((q & 1) == 1) {
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const f32x4 gs = gsv[(bt >> 1) & 1][u];
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                s[r] = fmaf(d[u][r], gs[r], s[r]);
                            }
                        }
                    }
                    if (q == 3) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            sc[t2 * 4 + r] = fmaf(s[r], latent_log2, fmaf(s_rope[r], scale_log2, neg_ref_shifted)); // relative to the reference
                        }
                    }
                }
                if (t0 + kStepTokens > len) { // only the last step of a sequence has tokens to mask
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const unsigned int token = t0 + 16u * (e >> 2) + 4u * j + (e & 3);
                        sc[e] = token < len ? sc[e] : kNegInf;
                    }
                }
                // Online softmax for this head column with lazy rescaling: the stored maximum (the reference the scores
                // above are already relative to) only moves when a score exceeds it by 2^8 (p stays <= 256).  On most
                // steps no lane sees such a score, and the reduction across the wave's rows, the new reference and the
                // rescaling factor are skipped altogether.
                float lane_max = sc[0];
#pragma unroll
                for (int e = 1; e < 8; ++e) {
                    lane_max = fmaxf(lane_max, sc[e]);
                }
                float alpha = 1.0f;
                if (__any(lane_max > 8.0f + (float)kPShift || run_max == kNegInf)) {
                    const float step_max = wave_max_16x4(lane_max) - (float)kPShift; // relative as well, without the shift
                    const float ref = -neg_ref;
                    float new_max = run_max;
                    if (step_max > 8.0f || run_max == kNegInf) {
                        new_max = fmaxf(run_max, ref + step_max);
                    }
                    const float safe_max = new_max == kNegInf ? 0.0f : new_max;
                    alpha = __builtin_amdgcn_exp2f(run_max - safe_max); // 0 on the first step: nothing accumulated yet
                    const float delta = safe_max - ref;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        sc[e] -= delta;
                    }
                    run_max = new_max;
                    neg_ref = -safe_max;
                    neg_ref_shifted = neg_ref + (float)kPShift;
                    run_sum *= alpha;
                }
                f32x4 p_lo, p_hi;
                float step_sum = 0.0f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    p_lo[e] = __builtin_amdgcn_exp2f(sc[e]);
                    p_hi[e] = __builtin_amdgcn_exp2f(sc[4 + e]);
                    step_sum += p_lo[e] + p_hi[e];
                }
                run_sum += step_sum; // in units of 2^-kPShift, like the probabilities
                lds_p16[i & 1u][hw][lane] = u32x4{pack_f16_hw(p_lo[0], p_lo[1]), pack_f16_hw(p_lo[2], p_lo[3]),
                                                 pack_f16_hw(p_hi[0], p_hi[1]), pack_f16_hw(p_hi[2], p_hi[3])};
                lds_alpha[i & 1u][hw][lane] = alpha;
            }
            convert_to(i + 1u);
            stage_step(i + 2u);
            lds_barrier();
        }
        const float total = wave_sum_16x4(run_sum) * (1.0f / (float)(1 << kPShift));
        if constexpr (NARROW) {
            // the two token halves of a head become one record: the larger reference (the one the value waves ended on) and
            // both sums brought to it
            if (stream == 1u && j == 0u) {
                lds_final[score_tile][m] = float2{run_max, total};
            }
            lds_barrier();
            if (stream == 0u && head < p.heads && j == 0u) {
                const float2 other = lds_final[score_tile][m];
                const float common = fmaxf(run_max, other.x);
                float sum = 0.0f;
                if (run_max != kNegInf) {
                    sum += total * __builtin_amdgcn_exp2f(run_max - common);
                }
                if (other.x != kNegInf) {
                    sum += other.y * __builtin_amdgcn_exp2f(other.x - common);
                }
                p.stats[rec * 2] = common;
                p.stats[rec * 2 + 1] = sum;
            }
        } else if (head < p.heads && j == 0) {
            p.stats[rec * 2] = run_max;
            p.stats[rec * 2 + 1] = total;
        }
    } else {
        // ================================ value waves ================================
        // Value wave v = 2 hp + dh owns head tiles 2 hp and 2 hp + 1 and output columns [256 dh, 256 dh + 256):
        // every V^T fragment it reads from LDS feeds two MFMAs (one per head tile), which halves the LDS traffic
        // of this stage and doubles the matrix work behind each LDS round trip.
        // NARROW: every value wave takes head tiles 0 and 1 and a quarter of the columns, [128 v, 128 v + 128).
        constexpr int GROUPS = NARROW ? 2 : 4; // 64-column scale groups of this wave
        const unsigned int hp = NARROW ? 0u : hw >> 1;
        const unsigned int part = NARROW ? hw : hw & 1u; // the wave's run of 64 * GROUPS columns
        // narrow: sixteen heads or fewer leave the second head tile empty; it is neither rescaled nor multiplied
        const bool second_tile = !NARROW || __builtin_amdgcn_readfirstlane((int)(p.heads > 16u)) != 0;
        f32x4 acc[2][GROUPS * 4];
#pragma unroll
        for (int ht = 0; ht < 2; ++ht) {
#pragma unroll
            for (int t = 0; t < GROUPS * 4; ++t) {
                acc[ht][t] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
        // exponent window of P': the accumulators hold sum(P' c) / 2^window with 2^window above the largest scale
        // seen / 2^7, so p (<= 2^8) * scale / 2^window stays below 2^15; the window only grows, and the accumulators
        // are rescaled by the power of two it grows by.  It starts at what tile 0 needs, so that the f16 scale table of
        // every later tile is written for a window its reader still has, unless the scales grew in between.
        auto window_for = [](unsigned int top_bits) __attribute__((always_inline)) -> int {
            return min(max((int)((top_bits >> 23) & 0xffu) - 133, -96), 112);
        };
        {
            const f32x4 tops = *(const f32x4*)lds_top[0];
            window = window_for(__builtin_amdgcn_readfirstlane(__float_as_uint(fmaxf(fmaxf(tops[0], tops[1]), fmaxf(tops[2], tops[3])))));
        }
        typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
        auto pk_mul = [](unsigned int x, unsigned int y) __attribute__((always_inline)) -> unsigned int {
            return __builtin_bit_cast(unsigned int, __builtin_bit_cast(f16x2_t, x) * __builtin_bit_cast(f16x2_t, y));
        };
        float common[2] = {kNegInf, kNegInf}; // narrow: the reference a head's accumulators are relative to
        unsigned int value_tile = 0; // buffer of tile i - 1
        stage_step(1u);
        const unsigned int lds_base = (unsigned int)(unsigned long long)(__attribute__((address_space(3))) const unsigned char*)lds;
        for (unsigned int i = 0; i <= steps; ++i) {
            // the hand-over records are requested first: their LDS round trip hides behind the staging work
            u32x4 p16[2];
            float alpha[2];
            float half_ref[2][2];
#pragma unroll
            for (int ht = 0; ht < 2; ++ht) {
                p16[ht] = lds_p16[(i + 1u) & 1u][2u * hp + ht][lane];
                if constexpr (NARROW) {
                    half_ref[ht][0] = lds_alpha[(i + 1u) & 1u][2 * ht][lane];
                    half_ref[ht][1] = lds_alpha[(i + 1u) & 1u][2 * ht + 1][lane];
                    alpha[ht] = 1.0f;
                } else {
                    alpha[ht] = lds_alpha[(i + 1u) & 1u][2u * hp + ht][lane];
                }
            }
            const f32x4 tops = *(const f32x4*)lds_top[value_tile]; // tile i - 1
            const unsigned int top_bits = __builtin_amdgcn_readfirstlane(__float_as_uint(fmaxf(fmaxf(tops[0], tops[1]), fmaxf(tops[2], tops[3]))));
            const int table_window = __builtin_amdgcn_readfirstlane(lds_win[value_tile]);
            asm volatile("" ::: "memory");
            if constexpr (NARROW) {
                if (i > 0) {
                    // The two token halves of a head were scored against references of their own (-inf while a half has
                    // seen nothing).  The accumulators follow the larger one: they are rescaled when it moves, and each
                    // half's probabilities are brought to it by a factor of at most 1 (exactly 1 for the half that holds
                    // the larger reference, 0 for -inf).
#pragma unroll
                    for (int ht = 0; ht < 2; ++ht) {
                        const float ra = half_ref[ht][0], rb = half_ref[ht][1];
                        const float to = fmaxf(common[ht], fmaxf(ra, rb));
                        alpha[ht] = to == common[ht] ? 1.0f : __builtin_amdgcn_exp2f(common[ht] - to);
                        common[ht] = to;
                        const float fa = ra == kNegInf ? 0.0f : __builtin_amdgcn_exp2f(ra - to);
                        const float fb = rb == kNegInf ? 0.0f : __builtin_amdgcn_exp2f(rb - to);
                        const unsigned int fa2 = pack_f16_hw(fa, fa), fb2 = pack_f16_hw(fb, fb);
                        p16[ht][0] = pk_mul(p16[ht][0], fa2);
                        p16[ht][1] = pk_mul(p16[ht][1], fa2);
                        p16[ht][2] = pk_mul(p16[ht][2], fb2);
                        p16[ht][3] = pk_mul(p16[ht][3], fb2);
                    }
                }
            }
            if (i > 0) {
                // the window moves before this iteration's conversion, so that the table written now is written for it
                const int need = window_for(top_bits);
                if (need > window) {
                    const float shrink = __uint_as_float((unsigned int)(127 - min(need - window, 126)) << 23);
                    alpha[0] *= shrink;
                    alpha[1] *= shrink;
                    window = need;
                }
            }
            const bool table_fits = table_window == window;
            __builtin_amdgcn_s_setprio(3);
            convert_to(i + 1u);
            stage_step(i + 2u);
            __builtin_amdgcn_s_setprio(0);
            // O^T += V^T . P' of tile i - 1 for the first HT head tiles of the pair
            auto accumulate = [&](auto tiles) __attribute__((always_inline)) {
                constexpr int HT = decltype(tiles)::value;
                // LDS byte addresses of this step: one register per fragment row, everything else is an immediate
                const unsigned int tile_lds = lds_base + value_tile * kTileBytes + part * (GROUPS * 128u); // this wave's scale groups
#pragma unroll
                for (int ht = 0; ht < HT; ++ht) {
                    if (__any(alpha[ht] != 1.0f)) {
#pragma unroll
                        for (int t = 0; t < GROUPS * 4; ++t) {
                            acc[ht][t] *= alpha[ht];
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                // V^T fragments of scale group g + 1 are requested before group g's MFMAs are issued: with the
                // reads in program order behind each MFMA the wave pays one LDS round trip per tile.
                union VFrag {
                    s16x4 s[2];
                    f16x8 h;
                };
                // The transposed reads are written as inline assembly with immediate offsets: one address register per
                // fragment row serves all of the wave's groups, and the waits are placed by hand (lgkmcnt, LDS operations
                // complete in issue order) exactly one group behind the requests.  The scale reads are assembly as
                // well: the compiler does not count the transposed reads, so a wait it places for a scale read of its
                // own would also wait for every fragment requested since.
                const unsigned int at[4] = {tile_lds + pv_base[0], tile_lds + pv_base[1], tile_lds + pv_base[2], tile_lds + pv_base[3]};
                auto load_group = [&](VFrag (&vf)[4], int g) __attribute__((always_inline)) {
#pragma unroll
                    for (int tt = 0; tt < 4; ++tt) {
                        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(vf[tt].s[0]) : "v"(at[tt]), "i"(g * 128));
                        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(vf[tt].s[1]) : "v"(at[tt]), "i"(g * 128 + 16 * kRowBytes));
                    }
                };
                VFrag vf[2][4];
                if (!table_fits) {
                    // The f16 table of this tile was written for another window (the first tile of a split, or the scales
                    // grew since): the wave rewrites the GROUPS x 32 entries it is about to read from the f32 table.  Another
                    // value wave with the same columns writes the same values; LDS operations of a wave complete in order.
                    const float into_window = __uint_as_float((unsigned int)(127 - kPShift - window) << 23);
#pragma unroll
                    for (int e = 0; e < GROUPS / 2; ++e) {
                        const unsigned int idx = lane + 64u * e;
                        const unsigned int g = GROUPS * part + (idx >> 5), t = idx & 31u;
                        lds_scale16[value_tile][g][t] = (_Float16)(lds_scale[value_tile][g][t] * into_window);
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                }
                // P'_g = p16 * scale16_g: both factors are f16 already (the probabilities from the score wave, the scales
                // from the conversion, divided by the window there), one packed multiply per two tokens
                const unsigned int gs16_lds = (unsigned int)(unsigned long long)(__attribute__((address_space(3))) const _Float16*)&lds_scale16[0][0][0] +
                                              (value_tile * (8 * kStepTokens) + part * (GROUPS * kStepTokens) + 4 * j) * 2u;
                auto scales16_of = [&](int g, u32x2& lo, u32x2& hi) __attribute__((always_inline)) {
                    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(lo) : "v"(gs16_lds), "i"(g * kStepTokens * 2));
                    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(hi) : "v"(gs16_lds), "i"(g * kStepTokens * 2 + 32));
                };
                u32x2 gs_lo[2], gs_hi[2];
                load_group(vf[0], 0);
                scales16_of(0, gs_lo[0], gs_hi[0]);
#pragma unroll
                for (int g = 0; g < GROUPS; ++g) {
                    const int cur = g & 1;
                    if (g + 1 < GROUPS) {
                        load_group(vf[cur ^ 1], g + 1);
                        scales16_of(g + 1, gs_lo[cur ^ 1], gs_hi[cur ^ 1]);
                        // group g's ten reads are older than the ten just issued
                        asm volatile("s_waitcnt lgkmcnt(10)" : "+v"(vf[cur][0].s[0]), "+v"(vf[cur][0].s[1]), "+v"(vf[cur][1].s[0]), "+v"(vf[cur][1].s[1]),
                                     "+v"(vf[cur][2].s[0]), "+v"(vf[cur][2].s[1]), "+v"(vf[cur][3].s[0]), "+v"(vf[cur][3].s[1]),
                                     "+v"(gs_lo[cur]), "+v"(gs_hi[cur])
                                     :
                                     : "memory");
                    } else {
                        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vf[cur][0].s[0]), "+v"(vf[cur][0].s[1]), "+v"(vf[cur][1].s[0]), "+v"(vf[cur][1].s[1]),
                                     "+v"(vf[cur][2].s[0]), "+v"(vf[cur][2].s[1]), "+v"(vf[cur][3].s[0]), "+v"(vf[cur][3].s[1]),
                                     "+v"(gs_lo[cur]), "+v"(gs_hi[cur])
                                     :
                                     : "memory");
                    }
#pragma unroll
                    for (int ht = 0; ht < HT; ++ht) {
                        Frag pf;
                        pf.u[0] = pk_mul(p16[ht][0], gs_lo[cur][0]);
                        pf.u[1] = pk_mul(p16[ht][1], gs_lo[cur][1]);
                        pf.u[2] = pk_mul(p16[ht][2], gs_hi[cur][0]);
                        pf.u[3] = pk_mul(p16[ht][3], gs_hi[cur][1]);
#pragma unroll
                        for (int tt = 0; tt < 4; ++tt) {
                            acc[ht][g * 4 + tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[cur][tt].h, pf.h, acc[ht][g * 4 + tt], 0, 0, 0);
                        }
                    }
                }
            };
            if (i > 0) {
                // (the one-tile form exists in the narrow layout only: with the wide layout's 32 accumulators a second form
                // of the block in the same kernel costs 150 spilled registers, and its empty tiles are multiplied and dropped)
                if (second_tile) {
                    accumulate(std::integral_constant<int, 2>{});
                } else {
                    accumulate(std::integral_constant<int, 1>{});
                }
                value_tile = value_tile == kWsTiles - 1u ? 0u : value_tile + 1u;
            }
            lds_barrier();
        }
        if constexpr (NARROW) {
            lds_barrier(); // the score waves exchange their token halves' sums behind this one
        }
#pragma unroll
        for (int ht = 0; ht < 2; ++ht) {
            const unsigned int out_head = blockIdx.y * 64u + (2u * hp + ht) * 16u + m;
            if (out_head < p.heads) {
                float* out = p.partial + (row * p.heads + out_head) * kLatent + part * (GROUPS * 64u);
                const float out_of_window = __uint_as_float((unsigned int)(127 + window) << 23);
#pragma unroll
                for (int t = 0; t < GROUPS * 4; ++t) {
                    *(f32x4*)(out + t * 16 + 4 * j) = acc[ht][t] * out_of_window;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// 4. project value
// ---------------------------------------------------------------------------------------------
// 256 threads = 4 waves.  A wave works on eight value columns at a time: lane = (column v0 + lane / 8, slice
// lane % 8); slice s owns the latent columns 64 i + 8 s .. + 8 for i = 0..7, so that the eight slices of a column
// fetch one whole 128-byte line of its weight row per load instruction (with 64 consecutive columns per slice every
// instruction touched 64 different lines: measured, the projection took 12 us of a 16 us kernel).  The lane keeps its
// 64 weighted values in registers and the eight slices are summed with DPP row shifts.
__device__ __forceinline__ void project_head(const MlaDecodeParams& p, unsigned int head, unsigned int b, const float (&x)[64],
                                             unsigned int v_begin, unsigned int v_end)
{
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int wave = threadIdx.x >> 6;
    const unsigned int slice = lane & 7u;
    const unsigned int sub = lane >> 3;
    const unsigned short* w = p.kv_b + ((size_t)head * p.kv_head_dim + p.nope_dim) * kLatent + slice * 8u;
    const unsigned int out_stride = p.out_compact ? p.value_dim : p.q_head_dim;
    const size_t out_base = ((size_t)b * p.heads + head) * out_stride;
    for (unsigned int v0 = v_begin + wave * 8u; v0 < v_end; v0 += 32u) {
        const unsigned int v = v0 + sub;
        const unsigned int vr = min(v, p.value_dim - 1u);
        u32x4 raw[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            raw[i] = *(const u32x4*)(w + (size_t)vr * kLatent + 64 * i);
        }
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                sum = fmaf(x[8 * i + 2 * e], __uint_as_float(raw[i][e] << 16), sum);
                sum = fmaf(x[8 * i + 2 * e + 1], __uint_as_float(raw[i][e] & 0xffff0000u), sum);
            }
        }
        // sum the eight slices of a column: lanes 8 sub .. 8 sub + 7 sit in one 16-lane row
        sum += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(sum), 0x114, 0xf, 0xf, true)); // row_shr:4
        sum += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(sum), 0x112, 0xf, 0xf, true)); // row_shr:2
        sum += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(sum), 0x111, 0xf, 0xf, true)); // row_shr:1
        if (slice == 7u && v < p.value_dim) {
            if (p.out_dtype == 0) {
                ((float*)p.out)[out_base + v] = sum;
            } else {
                ((unsigned short*)p.out)[out_base + v] = f32_to_bf16_bits(sum);
            }
        }
    }
}

// grid = (heads, batch, value_dim / 32 rounded up): projection of the merged rows in the workspace, 32 value columns a
// workgroup -- one pass of project_head, so the kernel is one round trip to memory long (merged row and weights together)
__global__ __launch_bounds__(256) void mla_project(MlaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    const float* weighted = p.weighted + ((size_t)b * p.heads + head) * kLatent + (threadIdx.x & 7u) * 8u;
    float x[64]; // x[8 i + e] = column 64 i + 8 slice + e
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const f32x4 t = *(const f32x4*)(weighted + 64 * (i >> 1) + 4 * (i & 1));
        x[4 * i] = t[0];
        x[4 * i + 1] = t[1];
        x[4 * i + 2] = t[2];
        x[4 * i + 3] = t[3];
    }
    project_head(p, head, b, x, blockIdx.z * 32u, min(p.value_dim, blockIdx.z * 32u + 32u));
}

// grid = (heads, batch): split merge and projection in one kernel when both stages run.  The merge is the
// log-sum-exp combine of the split records (same algebra as the stand-alone merge, base 2): threads =
// (128 column quads) x (2 split lanes), all loads of a lane issued before any is used; the merged row goes
// through LDS to the projection's register layout instead of through the workspace.  With the usual value width
// (128 columns) a thread's weight vectors for all four passes of the projection are requested first of all, so that
// the kernel is two memory round trips long (sequence length, then records and weights together) instead of seven.
__global__ __launch_bounds__(256) void mla_merge_project(MlaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    const unsigned int quad = threadIdx.x & 127u;
    const unsigned int sl = threadIdx.x >> 7;
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int wave = threadIdx.x >> 6;
    const unsigned int slice = lane & 7u;
    const unsigned int sub = lane >> 3;
    const bool wide = p.value_dim == 128u;
    u32x4 raw[4][8];
    const unsigned short* w_head = p.kv_b + ((size_t)head * p.kv_head_dim + p.nope_dim) * kLatent + slice * 8u;
    if (wide) {
        const unsigned short* w = w_head;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const unsigned int v = wave * 8u + 32u * pass + sub;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                raw[pass][i] = *(const u32x4*)(w + (size_t)v * kLatent + 64 * i);
            }
        }
    }
    unsigned int seq;
    const unsigned int len = visible_tokens(p.ctx_lens, p.query_rows, b, seq);
    unsigned int chunks = (unsigned int)min((unsigned long long)p.max_chunks, ((unsigned long long)len + p.chunk_tokens - 1u) / p.chunk_tokens);
    const size_t base = mla_merge_base(p, b, chunks);
    const float* stats = p.stats + (base * p.heads + head) * 2;
    const size_t stat_stride = (size_t)p.heads * 2;
    const float* partial = p.partial + (base * p.heads + head) * kLatent + quad * 4u;
    const size_t partial_stride = (size_t)p.heads * kLatent;
    float m = kNegInf, l = 0.0f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    // sixteen records per trip and lane: a sequence of up to 32 splits is one round trip
    for (unsigned int c0 = sl; c0 < chunks; c0 += 32u) {
        float cm[16], cl[16];
        f32x4 part[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const unsigned int c = min(c0 + 2u * u, chunks - 1u);
            const bool live = c0 + 2u * u < chunks;
            const float2 st = *(const float2*)(stats + c * stat_stride);
            cm[u] = live ? st.x : kNegInf;
            cl[u] = live ? st.y : 0.0f;
            part[u] = *(const f32x4*)(partial + c * partial_stride);
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            if (cl[u] > 0.0f) {
                const float nm = fmaxf(m, cm[u]);
                const float a = __builtin_amdgcn_exp2f(m - nm); // m = -inf -> 0
                const float w = __builtin_amdgcn_exp2f(cm[u] - nm);
                acc = acc * a + part[u] * w;
                l = l * a + cl[u] * w;
                m = nm;
            }
        }
    }
    __shared__ float other_m[128], other_l[128];
    __shared__ f32x4 other_acc[128];
    __shared__ __align__(16) float merged[kLatent];
    if (sl == 1u) {
        other_m[quad] = m;
        other_l[quad] = l;
        other_acc[quad] = acc;
    }
    __syncthreads();
    if (sl == 0u) {
        const float om = other_m[quad], ol = other_l[quad];
        const float gm = fmaxf(m, om);
        const float safe_g = gm == kNegInf ? 0.0f : gm;
        float denom = 0.0f;
        f32x4 total = {0.f, 0.f, 0.f, 0.f};
        if (l > 0.0f) {
            const float w = __builtin_amdgcn_exp2f(m - safe_g);
            denom += l * w;
            total += acc * w;
        }
        if (ol > 0.0f) {
            const float w = __builtin_amdgcn_exp2f(om - safe_g);
            denom += ol * w;
            total += other_acc[quad] * w;
        }
        f32x4 result = {0.f, 0.f, 0.f, 0.f};
        if (denom > 0.0f && denom < __builtin_inff()) {
            result = total * (1.0f / denom);
        }
        *(f32x4*)(merged + quad * 4u) = result;
    }
    __syncthreads();
    if (wide) { // the other two passes' weights travel while the merged row is read back
#pragma unroll
        for (int pass = 2; pass < 4; ++pass) {
            const unsigned int v = wave * 8u + 32u * pass + sub;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                raw[pass][i] = *(const u32x4*)(w_head + (size_t)v * kLatent + 64 * i);
            }
        }
    }
    float x[64]; // x[8 i + e] = column 64 i + 8 slice + e: the eight slices read 256 contiguous bytes at a time
    const float* row = merged + slice * 8u;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const f32x4 t = *(const f32x4*)(row + 64 * (i >> 1) + 4 * (i & 1));
        x[4 * i] = t[0];
        x[4 * i + 1] = t[1];
        x[4 * i + 2] = t[2];
        x[4 * i + 3] = t[3];
    }
    if (!wide) {
        project_head(p, head, b, x, 0u, p.value_dim);
        return;
    }
    // same arithmetic and order as project_head, on the weights fetched at the start
    const unsigned int out_stride = p.out_compact ? p.value_dim : p.q_head_dim;
    const size_t out_base = ((size_t)b * p.heads + head) * out_stride;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const unsigned int v = wave * 8u + 32u * pass + sub;
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                sum = fmaf(x[8 * i + 2 * e], __uint_as_float(raw[pass][i][e] << 16), sum);
                sum = fmaf(x[8 * i + 2 * e + 1], __uint_as_float(raw[pass][i][e] & 0xffff0000u), sum);
            }
        }
        sum += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(sum), 0x114, 0xf, 0xf, true)); // row_shr:4
        sum += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(sum), 0x112, 0xf, 0xf, true)); // row_shr:2
        sum += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(sum), 0x111, 0xf, 0xf, true)); // row_shr:1
        if (slice == 7u) {
            if (p.out_dtype == 0) {
                ((float*)p.out)[out_base + v] = sum;
            } else {
                ((unsigned short*)p.out)[out_base + v] = f32_to_bf16_bits(sum);
            }
        }
    }
}

// The split merge on its own for a call of few rows with many splits each (one sequence of 32 K tokens is cut into 256
// splits, one per compute unit): a workgroup per (row, head) folds them in eight dependent round trips, on as many
// compute units as the call has heads.  Here eight workgroups share a (row, head), each taking a run of 64 latent columns:
// 256 threads = 16 split lanes x 16 column quads fold sixteen records per lane and trip (256 splits: one round trip, and
// no wait for the sequence length first: every split of the plan has a record, whose sum says whether it holds
// anything); the lanes of a quad meet through lane exchanges and LDS.  The merged row goes to the workspace and
// mla_project reads it from there.  (One kernel for both, the eight runs' products summed by the workgroup that arrives
// last, was built: the release fence before the arrival counter writes back a level-two cache full of split records, and
// the kernel took 23 us where the two launches take 10.)  grid = (heads, rows, 8).
constexpr int kWideParts = 8;
__global__ __launch_bounds__(256) void mla_merge_wide(MlaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    const unsigned int tid = threadIdx.x;
    const unsigned int quad = tid & 15u;
    const unsigned int sl = tid >> 4;
    const unsigned int column = blockIdx.z * 64u + quad * 4u;
    // every planned split has a record (an empty one says so) when the rows are [query row][max_chunks]; densely numbered
    // rows hold live splits only, so there the row's own count bounds the walk
    unsigned int limit = p.max_chunks;
    if (p.record_rows != 0u) {
        unsigned int seq;
        const unsigned int len = visible_tokens(p.ctx_lens, p.query_rows, b, seq);
        limit = (unsigned int)min((unsigned long long)p.max_chunks, ((unsigned long long)len + p.chunk_tokens - 1u) / p.chunk_tokens);
    }
    const size_t base = mla_merge_base(p, b, limit);
    const float* stats = p.stats + (base * p.heads + head) * 2;
    const size_t stat_stride = (size_t)p.heads * 2;
    const float* partial = p.partial + (base * p.heads + head) * kLatent + column;
    const size_t partial_stride = (size_t)p.heads * kLatent;
    float m = kNegInf, l = 0.0f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (unsigned int c0 = sl; c0 < limit; c0 += 256u) {
        float cm[16], cl[16];
        f32x4 part[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const unsigned int c = c0 + 16u * u;
            cm[u] = kNegInf;
            cl[u] = 0.0f;
            part[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (c < limit) { // a plan of few splits leaves most of a lane's sixteen requests unmade
                const float2 st = *(const float2*)(stats + c * stat_stride);
                cm[u] = st.x;
                cl[u] = st.y;
                part[u] = *(const f32x4*)(partial + c * partial_stride);
            }
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            if (cl[u] > 0.0f) {
                const float nm = fmaxf(m, cm[u]);
                const float a = __builtin_amdgcn_exp2f(m - nm); // m = -inf -> 0
                const float w = __builtin_amdgcn_exp2f(cm[u] - nm);
                acc = acc * a + part[u] * w;
                l = l * a + cl[u] * w;
                m = nm;
            }
        }
    }
    // two partial merges into one; a side that holds nothing has l = 0
    auto fold = [](float& m, float& l, f32x4& acc, float om, float ol, const f32x4& oacc) __attribute__((always_inline)) {
        const float nm = fmaxf(l > 0.0f ? m : kNegInf, ol > 0.0f ? om : kNegInf);
        const float a = l > 0.0f ? __builtin_amdgcn_exp2f(m - nm) : 0.0f;
        const float w = ol > 0.0f ? __builtin_amdgcn_exp2f(om - nm) : 0.0f;
        acc = acc * a + oacc * w;
        l = l * a + ol * w;
        m = nm;
    };
    // the four split lanes of a wave (lanes 16 and 32 apart), then the four waves
#pragma unroll
    for (int step = 16; step <= 32; step *= 2) {
        const float om = __shfl_xor(m, step), ol = __shfl_xor(l, step);
        const f32x4 oacc = {__shfl_xor(acc[0], step), __shfl_xor(acc[1], step), __shfl_xor(acc[2], step), __shfl_xor(acc[3], step)};
        fold(m, l, acc, om, ol, oacc);
    }
    __shared__ float wave_m[4][16], wave_l[4][16];
    __shared__ f32x4 wave_acc[4][16];
    if ((tid & 63u) < 16u) {
        wave_m[tid >> 6][quad] = m;
        wave_l[tid >> 6][quad] = l;
        wave_acc[tid >> 6][quad] = acc;
    }
    __syncthreads();
    if (tid < 16u) {
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            fold(m, l, acc, wave_m[w][quad], wave_l[w][quad], wave_acc[w][quad]);
        }
        f32x4 result = {0.f, 0.f, 0.f, 0.f};
        if (l > 0.0f && l < __builtin_inff()) {
            result = acc * (1.0f / l);
        }
        *(f32x4*)(p.weighted + ((size_t)b * p.heads + head) * kLatent + column) = result;
    }
}

// Split merge and projection for a prefill chunk: a workgroup takes R query rows of one head.  A chunk row usually has
// one or two splits, so each thread folds all splits of its (row, column quad) itself -- two rows at a time over the
// 256 threads, no exchange between threads -- and writes the merged row to LDS; the projection then reads every weight
// vector once and applies it to the R merged rows, instead of once per row.
template <int R> __global__ __launch_bounds__(256) void mla_merge_project_rows(MlaDecodeParams p)
{
    static_assert(R % 2 == 0, "two rows are merged at a time");
    const unsigned int head = blockIdx.x;
    const unsigned int row0 = blockIdx.y * R;
    const unsigned int quad = threadIdx.x & 127u;
    __shared__ __align__(16) float merged[R][kLatent];
    for (int r = (int)(threadIdx.x >> 7); r < R; r += 2) {
        const unsigned int b = min(row0 + r, p.batch - 1u);
        unsigned int seq;
        const unsigned int len = visible_tokens(p.ctx_lens, p.query_rows, b, seq);
        unsigned int chunks = (unsigned int)min((unsigned long long)p.max_chunks, ((unsigned long long)len + p.chunk_tokens - 1u) / p.chunk_tokens);
        const size_t base = mla_merge_base(p, b, chunks);
        const float* stats = p.stats + (base * p.heads + head) * 2;
        const size_t stat_stride = (size_t)p.heads * 2;
        const float* partial = p.partial + (base * p.heads + head) * kLatent + quad * 4u;
        const size_t partial_stride = (size_t)p.heads * kLatent;
        float m = kNegInf, l = 0.0f;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (unsigned int c0 = 0; c0 < chunks; c0 += 4u) {
            float cm[4], cl[4];
            f32x4 part[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const unsigned int c = min(c0 + u, chunks - 1u);
                const bool live = c0 + u < chunks;
                const float2 st = *(const float2*)(stats + c * stat_stride);
                cm[u] = live ? st.x : kNegInf;
                cl[u] = live ? st.y : 0.0f;
                part[u] = *(const f32x4*)(partial + c * partial_stride);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (cl[u] > 0.0f) {
                    const float nm = fmaxf(m, cm[u]);
                    const float a = __builtin_amdgcn_exp2f(m - nm);
                    const float w = __builtin_amdgcn_exp2f(cm[u] - nm);
                    acc = acc * a + part[u] * w;
                    l = l * a + cl[u] * w;
                    m = nm;
                }
            }
        }
        f32x4 result = {0.f, 0.f, 0.f, 0.f};
        if (l > 0.0f && l < __builtin_inff()) {
            result = acc * (1.0f / l);
        }
        *(f32x4*)(&merged[r][quad * 4u]) = result;
    }
    __syncthreads();
    // projection: lane = (value column v0 + lane / 8, slice lane % 8 of 64 latent columns), as in project_head
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int wave = threadIdx.x >> 6;
    const unsigned int slice = lane & 7u;
    const unsigned int sub = lane >> 3;
    const unsigned short* w = p.kv_b + ((size_t)head * p.kv_head_dim + p.nope_dim) * kLatent + slice * 8u;
    const unsigned int out_stride = p.out_compact ? p.value_dim : p.q_head_dim;
    for (unsigned int v0 = wave * 8u; v0 < p.value_dim; v0 += 32u) {
        const unsigned int v = v0 + sub;
        const unsigned int vr = min(v, p.value_dim - 1u);
        u32x4 raw[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            raw[i] = *(const u32x4*)(w + (size_t)vr * kLatent + 64 * i);
        }
        for (int r = 0; r < R; ++r) {
            const float* x = &merged[r][slice * 8u]; // columns 64 i + 8 slice .. + 8, as the weights
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const f32x4 x0 = *(const f32x4*)(x + 64 * i), x1 = *(const f32x4*)(x + 64 * i + 4);
                sum = fmaf(x0[0], __uint_as_float(raw[i][0] << 16), sum);
                sum = fmaf(x0[1], __uint_as_float(raw[i][0] & 0xffff0000u), sum);
                sum = fmaf(x0[2], __uint_as_float(raw[i][1] << 16), sum);
                sum = fmaf(x0[3], __uint_as_float(raw[i][1] & 0xffff0000u), sum);
                sum = fmaf(x1[0], __uint_as_float(raw[i][2] << 16), sum);
                sum = fmaf(x1[1], __uint_as_float(raw[i][2] & 0xffff0000u), sum);
                sum = fmaf(x1[2], __uint_as_float(raw[i][3] << 16), sum);
                sum = fmaf(x1[3], __uint_as_float(raw[i][3] & 0xffff0000u), sum);
            }
            sum += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(sum), 0x114, 0xf, 0xf, true)); // row_shr:4
            sum += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(sum), 0x112, 0xf, 0xf, true)); // row_shr:2
            sum += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(sum), 0x111, 0xf, 0xf, true)); // row_shr:1
            if (slice == 7u && v < p.value_dim && row0 + r < p.batch) {
                const size_t at = ((size_t)(row0 + r) * p.heads + head) * out_stride + v;
                if (p.out_dtype == 0) {
                    ((float*)p.out)[at] = sum;
                } else {
                    ((unsigned short*)p.out)[at] = f32_to_bf16_bits(sum);
                }
            }
        }
    }
}

// The split merge of sixteen rows of one head, then out^T[v, row] = sum_c W_v[v, c] merged[row, c] on the matrix cores:
// A operand: W_v rows straight from memory (a lane's eight consecutive latent columns are 16 bytes); B operand: the merged
// rows from LDS as bf16 hi + lo (the merged values are f32: two terms keep 16 bits of them).  value_dim <= 128.
// grid = (heads, workgroups per head), 512 threads; a workgroup takes blocks of sixteen rows in turn.  The merge is a chain of round trips to memory, so it is spread as wide
// as the workgroup goes: a thread folds the splits of four latent columns of four rows, the four rows' records requested
// together, four splits a trip.  Wave w then owns value columns [16 w, 16 w + 16).
// MODE 0: the workgroup folds its rows' split records.  MODE 1: the rows were merged by the split-merge kernel and lie in
// the workspace (p.weighted).  MODE 2: the plan has one record a row (a long chunk without KV splits), which only wants
// its sum divided out.  Modes 1 and 2 leave the registers for two workgroups per compute unit.
constexpr int kMergedStride = kLatent + 8; // bf16 elements: sixteen rows' 16-byte fragments start in different banks
// WAVES: 8 (value widths up to 128) or 16 (up to 256; modes 1 and 2, whose registers allow 1,024 threads).
template <int MODE, int WAVES = 8> __global__ __launch_bounds__(64 * WAVES) void mla_merge_project_mfma(MlaDecodeParams p)
{
    static_assert(WAVES == 8 || MODE != 0, "the record-folding form needs the registers of 512 threads");
    constexpr unsigned int RG = WAVES / 2;  // groups of 128 threads: thread group rb takes rows rb, rb + RG, ...
    constexpr int RPT = 16 / RG;            // rows of a block per thread
    // the merged rows as two bf16 terms (value = hi + lo keeps 16 bits of the f32), split once by the thread that merged them
    __shared__ __align__(16) unsigned short merged_hi[16][kMergedStride], merged_lo[16][kMergedStride];
    const unsigned int head = blockIdx.x;
    const unsigned int tid = threadIdx.x;
    const unsigned int quad = tid & 127u;
    const unsigned int lane = tid & 63u;
    const unsigned int wave = tid >> 6;
    const unsigned int m = lane & 15u;
    const unsigned int j = lane >> 4;
    // the projection's weights travel under the first merge and serve every block of sixteen rows the workgroup takes
    const unsigned short* w_head = p.kv_b + ((size_t)head * p.kv_head_dim + p.nope_dim) * kLatent;
    Frag wf[16];
    {
        const unsigned int v = min(wave * 16u + m, p.value_dim - 1u);
#pragma unroll
        for (int ks = 0; ks < 16; ++ks) {
            wf[ks].u = *(const u32x4*)(w_head + (size_t)v * kLatent + ks * 32 + 8u * j);
        }
    }
    // the merged values of this thread's four rows (rb, rb + 4, rb + 8, rb + 12 of the block at row0) and four columns
    auto fetch_rows = [&](unsigned int row0, f32x4 (&out)[RPT]) __attribute__((always_inline)) {
        if constexpr (MODE == 1) {
            const unsigned int rb = tid >> 7;
            f32x4 row[RPT];
#pragma unroll
            for (int u = 0; u < RPT; ++u) {
                const unsigned int b = min(row0 + rb + RG * u, p.batch - 1u);
                row[u] = *(const f32x4*)(p.weighted + ((size_t)b * p.heads + head) * kLatent + quad * 4u);
            }
#pragma unroll
            for (int u = 0; u < RPT; ++u) {
                out[u] = row[u];
            }
        } else if constexpr (MODE == 2) {
            const unsigned int rb = tid >> 7;
            float2 st[RPT];
            f32x4 part[RPT];
            unsigned int len[RPT];
#pragma unroll
            for (int u = 0; u < RPT; ++u) {
                const unsigned int b = min(row0 + rb + RG * u, p.batch - 1u);
                unsigned int seq;
                len[u] = visible_tokens(p.ctx_lens, p.query_rows, b, seq);
                st[u] = *(const float2*)(p.stats + ((size_t)b * p.heads + head) * 2);
                part[u] = *(const f32x4*)(p.partial + ((size_t)b * p.heads + head) * kLatent + quad * 4u);
            }
#pragma unroll
            for (int u = 0; u < RPT; ++u) {
                f32x4 result = {0.f, 0.f, 0.f, 0.f};
                if (len[u] > 0u && st[u].y > 0.0f && st[u].y < __builtin_inff()) {
                    result = part[u] * (1.0f / st[u].y);
                }
                out[u] = result;
            }
        } else {
            const unsigned int rb = tid >> 7; // rows rb, rb + 4, rb + 8, rb + 12
            const float* stats[4];
            const float* partial[4];
            unsigned int chunks[4];
            float mx[4], l[4];
            f32x4 acc[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const unsigned int b = min(row0 + rb + 4u * u, p.batch - 1u);
                unsigned int seq;
                const unsigned int len = visible_tokens(p.ctx_lens, p.query_rows, b, seq);
                chunks[u] = (unsigned int)min((unsigned long long)p.max_chunks, ((unsigned long long)len + p.chunk_tokens - 1u) / p.chunk_tokens);
                const size_t base = mla_merge_base(p, b, chunks[u]);
                stats[u] = p.stats + (base * p.heads + head) * 2;
                partial[u] = p.partial + (base * p.heads + head) * kLatent + quad * 4u;
                mx[u] = kNegInf;
                l[u] = 0.0f;
                acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            const size_t stat_stride = (size_t)p.heads * 2;
            const size_t partial_stride = (size_t)p.heads * kLatent;
            const unsigned int most = max(max(chunks[0], chunks[1]), max(chunks[2], chunks[3]));
            for (unsigned int c0 = 0; c0 < most; c0 += 4u) {
                float2 st[4][4];
                f32x4 part[4][4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const unsigned int c = min(c0 + v, max(chunks[u], 1u) - 1u);
                        st[u][v] = *(const float2*)(stats[u] + c * stat_stride);
                        part[u][v] = *(const f32x4*)(partial[u] + c * partial_stride);
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const bool live = c0 + v < chunks[u];
                        const float cl = live ? st[u][v].y : 0.0f;
                        if (cl > 0.0f) {
                            const float cm = st[u][v].x;
                            const float nm = fmaxf(mx[u], cm);
                            const float a = __builtin_amdgcn_exp2f(mx[u] - nm);
                            const float w = __builtin_amdgcn_exp2f(cm - nm);
                            acc[u] = acc[u] * a + part[u][v] * w;
                            l[u] = l[u] * a + cl * w;
                            mx[u] = nm;
                        }
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                f32x4 result = {0.f, 0.f, 0.f, 0.f};
                if (l[u] > 0.0f && l[u] < __builtin_inff()) {
                    result = acc[u] * (1.0f / l[u]);
                }
                out[u] = result;
            }
        }
    };
    // The next block's rows are requested before the projection of this one, so that the round trips to memory (one for
    // merged rows, several for split records) run under the matrix work instead of between two barriers: a 2,048-row
    // chunk of one record a row spent 3 us a block waiting, 408 us in all.
    f32x4 next_rows[RPT];
    fetch_rows(blockIdx.y * 16u, next_rows);
    for (unsigned int row0 = blockIdx.y * 16u; row0 < p.batch; row0 += gridDim.y * 16u) {
    {
        const unsigned int rb = tid >> 7;
#pragma unroll
        for (int u = 0; u < RPT; ++u) {
            const f32x4 x = next_rows[u];
            const u32x2 hi = {pack_bf16_rne(x[0], x[1]), pack_bf16_rne(x[2], x[3])};
            const u32x2 lo = {pack_bf16_rne(x[0] - __uint_as_float(hi[0] << 16), x[1] - __uint_as_float(hi[0] & 0xffff0000u)),
                              pack_bf16_rne(x[2] - __uint_as_float(hi[1] << 16), x[3] - __uint_as_float(hi[1] & 0xffff0000u))};
            *(u32x2*)(&merged_hi[rb + RG * u][quad * 4u]) = hi;
            *(u32x2*)(&merged_lo[rb + RG * u][quad * 4u]) = lo;
        }
    }
    __syncthreads();
    if (row0 + gridDim.y * 16u < p.batch) {
        fetch_rows(row0 + gridDim.y * 16u, next_rows);
    }
    // ---- projection
    const unsigned int out_stride = p.out_compact ? p.value_dim : p.q_head_dim;
    f32x4 out_acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 16; ++ks) {
        Frag hi, lo;
        hi.u = *(const u32x4*)(&merged_hi[m][ks * 32 + 8u * j]);
        lo.u = *(const u32x4*)(&merged_lo[m][ks * 32 + 8u * j]);
        out_acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[ks].b, hi.b, out_acc, 0, 0, 0);
        out_acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[ks].b, lo.b, out_acc, 0, 0, 0);
    }
    if (row0 + m < p.batch) { // lane (m, j) holds value columns 16 wave + 4 j .. + 4 of row m
        const size_t base = ((size_t)(row0 + m) * p.heads + head) * out_stride;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const unsigned int v = wave * 16u + 4u * j + r;
            if (v < p.value_dim) {
                if (p.out_dtype == 0) {
                    ((float*)p.out)[base + v] = out_acc[r];
                } else {
                    ((unsigned short*)p.out)[base + v] = f32_to_bf16_bits(out_acc[r]);
                }
            }
        }
    }
    __syncthreads(); // the next block's merge overwrites the rows just read
    }
}

} // namespace

// Workgroups per head of the matrix-core absorb and projection: every workgroup loads its head's weights once, so a long
// chunk is covered by one round of workgroups (about 256 in all), each taking several blocks of sixteen rows (four rounds
// measured 15 to 25 % slower on 64 rows and on a 512-row chunk: the weights are read four times as often).
static unsigned int row_block_groups(const MlaDecodeParams& p)
{
    const unsigned int blocks = (p.batch + 15u) / 16u;
    const unsigned int per_head = (256u + p.heads - 1u) / p.heads;
    return blocks < per_head ? blocks : per_head;
}

// One workgroup per (row, head) folds 32 split records a round trip; the wide merge and the separate projection cost a
// launch more and read any number of splits in one.  Measured (merge and projection together): one row of 32 heads with 256
// splits 19.4 -> 8.1 us, of 64 heads 21.1 -> 11.3; two rows of 32 heads with 128 splits 11.8 -> 8.1; one row of 128 heads
// with 128 splits 13.5 -> 14.7 (no gain: 1,024 workgroups for the merge).
static bool wide_merge_pays(const MlaDecodeParams& p)
{
    if (p.latent_dim != (unsigned int)kLatent) {
        return false;
    }
    return p.max_chunks > 128u || (p.max_chunks > 64u && p.heads * p.batch <= 64u);
}

// LSE combine of the split records into weighted[b, h, 0:512] (f32) with the split-merge kernels of GQA decode
static hipError_t merge_into_workspace(const MlaDecodeParams& p, hipStream_t stream)
{
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
    mp.query_rows = p.query_rows;
    mp.record_rows = p.record_rows;
    mp.first_rows = p.first_rows;
    return launch_split_merge(mp, stream);
}

hipError_t launch_mla_decode(const MlaDecodeParams& p, unsigned int stage_mask, hipStream_t stream)
{
    const unsigned int stages = (stage_mask & 15u) == 0 ? 15u : (stage_mask & 15u);
    hipError_t err = hipSuccess;
    // what the matrix-core kernels are built for; anything else runs the vector-ALU kernels of mla_generic.hip -- all
    // stages for other widths, absorb and projection (the stages that read kv_b) for other weight forms
    const bool usual_widths = p.latent_dim == (unsigned int)kLatent && p.rope_dim == 64u;
    const bool bf16_weights = p.kv_b_bits == 16u;
    if ((stages & 1u) && !(usual_widths && bf16_weights)) {
        err = launch_mla_absorb_any(p, stream);
        if (err != hipSuccess) {
            return err;
        }
    } else if (stages & 1u) {
        // Eight rows per workgroup share every weight load, and the workgroup then runs eight rows' sums: measured 28 us from
        // 16 rows up to a few hundred, against 13 us (15 rows) to 27 us (32 rows) for one workgroup per row
        if (p.batch >= 16u && (p.nope_dim == 128u || p.nope_dim == 192u) && (p.q_head_dim & 3u) == 0) { // sixteen rows a workgroup, on the matrix cores
            // four waves for a decode batch, sixteen for a chunk (33 against 61 us on 512 rows of 128 heads; on 16 to 64 rows
            // the larger workgroup costs 4 us); as many waves share a block of sixteen rows as keeps every wave busy
            MlaDecodeParams q = p;
            const unsigned int groups = row_block_groups(p);
            const unsigned int blocks_here = ((p.batch + 15u) / 16u + groups - 1u) / groups;
            const unsigned int waves = p.batch >= 128u ? 16u : 4u;
            q.column_split = 1u;
            while (q.column_split < waves && blocks_here * q.column_split < waves) {
                q.column_split *= 2u;
            }
            if (p.nope_dim == 128u) {
                waves == 16u ? mla_absorb_mfma<16, 128, 512><<<dim3(p.heads, groups), dim3(1024), 0, stream>>>(q)
                             : mla_absorb_mfma<4, 128, 512><<<dim3(p.heads, groups), dim3(256), 0, stream>>>(q);
            } else {
                waves == 16u ? mla_absorb_mfma<16, 192, 256><<<dim3(p.heads, groups, 2), dim3(1024), 0, stream>>>(q)
                             : mla_absorb_mfma<4, 192, 256><<<dim3(p.heads, groups, 2), dim3(256), 0, stream>>>(q);
            }
        } else if (p.batch >= 32u && p.nope_dim <= 256u) {
            mla_absorb_rows<8><<<dim3(p.heads, (p.batch + 7u) / 8u), dim3(256), 0, stream>>>(p);
        } else {
            const unsigned int z = p.heads * p.batch <= 128u ? 4u : 1u;
            mla_absorb<<<dim3(p.heads, p.batch, z), dim3(256u / z), 0, stream>>>(p);
        }
        err = hipGetLastError();
        if (err != hipSuccess) {
            return err;
        }
    }
    if ((stages & 2u) && !usual_widths) {
        err = launch_mla_partial_any(p, stream);
        if (err != hipSuccess) {
            return err;
        }
    } else if (stages & 2u) {
        // eight waves per workgroup measured 1.7x faster than four (261 vs 446 us on the 64K-context case)
        // densely numbered records are sized for the live splits: one workgroup per item and head block
        const dim3 grid = p.record_rows != 0u ? dim3(p.record_rows, (p.heads + 63) / 64, 1) : dim3(p.max_chunks, (p.heads + 63) / 64, p.batch);
        const bool narrow = p.heads <= 32u; // two head tiles at most: the score waves split a step's tokens, the value waves the columns four ways
        const bool aligned = p.block_tokens % kStepTokens == 0 && p.chunk_tokens % kStepTokens == 0;
        const bool pow2_tables = (p.block_tokens & (p.block_tokens - 1u)) == 0 && p.tables != nullptr;
        if ((stage_mask & 16u) != 0 && mla_partial_x32_takes(p)) { // ZLLM_MLA_WIDE_TILES: the caller asks for the 32x32x16-tile kernel
            err = launch_mla_partial_x32(p, stream);
            if (err != hipSuccess) {
                return err;
            }
        } else if (p.selection != nullptr) {
            (narrow ? mla_partial_ws<false, true, false, true> : mla_partial_ws<false, true>)<<<grid, dim3(512), 0, stream>>>(p);
        } else if (aligned && pow2_tables) {
            (narrow ? mla_partial_ws<true, false, true, true> : mla_partial_ws<true, false, true>)<<<grid, dim3(512), 0, stream>>>(p);
        } else if (aligned) {
            (narrow ? mla_partial_ws<true, false, false, true> : mla_partial_ws<true, false>)<<<grid, dim3(512), 0, stream>>>(p);
        } else {
            (narrow ? mla_partial_ws<false, false, false, true> : mla_partial_ws<false, false>)<<<grid, dim3(512), 0, stream>>>(p);
        }
        err = hipGetLastError();
        if (err != hipSuccess) {
            return err;
        }
    }
    if (!(usual_widths && bf16_weights)) {
        if (stages & 4u) {
            err = merge_into_workspace(p, stream);
            if (err != hipSuccess) {
                return err;
            }
        }
        return (stages & 8u) ? launch_mla_project_any(p, stream) : hipSuccess;
    }
    if ((stages & 12u) == 12u) {
        // value widths up to 128 run eight waves, up to 256 sixteen (not the record-folding form, whose registers stop at 512 threads)
        const bool wide_values = p.value_dim > 128u;
        const bool two_step = p.max_chunks > 1u && p.batch <= 64u;
        if (p.batch >= 16u && (p.value_dim <= 128u || (p.value_dim <= 256u && (two_step || p.max_chunks == 1u)))) {
            // sixteen rows a workgroup, the projection on the matrix cores.
            // Up to 64 rows the fused kernel is at most 256 workgroups, each a chain of round trips (lengths, records four
            // splits at a time, projection); the split-merge kernel reads the same records with a thread per (row, head,
            // column quad), and the projection then starts from merged rows: 22.9 -> 18.4 us for 16 rows of 128 heads in 8
            // splits, 29.6 -> 25.7 us for 64 rows.  A long chunk keeps the fused kernel: its merged rows would cross the
            // workspace twice (134 MB each way for 512 rows).
            const dim3 grid(p.heads, row_block_groups(p));
            if (two_step) {
                err = merge_into_workspace(p, stream);
                if (err != hipSuccess) {
                    return err;
                }
                wide_values ? mla_merge_project_mfma<1, 16><<<grid, dim3(1024), 0, stream>>>(p) : mla_merge_project_mfma<1, 8><<<grid, dim3(512), 0, stream>>>(p);
            } else if (p.max_chunks == 1u && wide_values) {
                mla_merge_project_mfma<2, 16><<<grid, dim3(1024), 0, stream>>>(p);
            } else if (p.max_chunks == 1u) {
                // one record a row: two workgroups of eight waves fit a compute unit, so twice the workgroups of the usual round
                const unsigned int blocks = (p.batch + 15u) / 16u;
                const unsigned int groups = 2u * row_block_groups(p);
                mla_merge_project_mfma<2, 8><<<dim3(p.heads, groups < blocks ? groups : blocks), dim3(512), 0, stream>>>(p);
            } else {
                mla_merge_project_mfma<0, 8><<<grid, dim3(512), 0, stream>>>(p);
            }
        } else if (p.batch >= 16u) { // eight rows share every weight load of the projection
            mla_merge_project_rows<8><<<dim3(p.heads, (p.batch + 7u) / 8u), dim3(256), 0, stream>>>(p);
        } else if (wide_merge_pays(p)) {
            // few rows, each cut into many splits: the merge by eight workgroups per (row, head), then the projection
            mla_merge_wide<<<dim3(p.heads, p.batch, kWideParts), dim3(256), 0, stream>>>(p);
            err = hipGetLastError();
            if (err != hipSuccess) {
                return err;
            }
            mla_project<<<dim3(p.heads, p.batch, (p.value_dim + 31u) / 32u), dim3(256), 0, stream>>>(p);
        } else {
            mla_merge_project<<<dim3(p.heads, p.batch), dim3(256), 0, stream>>>(p);
        }
        return hipGetLastError();
    }
    if (stages & 4u) {
        err = merge_into_workspace(p, stream);
        if (err != hipSuccess) {
            return err;
        }
    }
    if (stages & 8u) {
        mla_project<<<dim3(p.heads, p.batch, (p.value_dim + 31u) / 32u), dim3(256), 0, stream>>>(p);
        err = hipGetLastError();
    }
    return err;
}

} // namespace zllm

// Split-KV partial of absorbed MLA decode on 32x32x16 matrix tiles — gfx950.
//
// Same contract as mla_partial_ws (mla_decode.hip): workgroup = (split, block of 64 heads, query row), records
// (sum p v, max, sum p) for the split merge; it replaces the reference's mla_paged_decode_partial_f32
// (src/kernel/rocm/hip/attention/paged_mla/source.hip:4731-5249) for dense calls of more than 32 heads over pages of a
// multiple of 32 tokens.  What differs from mla_partial_ws is how a 32-token step is laid on the matrix cores:
//
//   * The tile a step's rows are converted into holds  f16(code * scale_g / 2^W)  (W = exponent of the largest group
//     scale the split has met so far), not integer codes beside a scale table.  Scores then need one accumulator for the
//     whole latent part and the value side multiplies plain probabilities: the per-(token, group) multiply-adds of the
//     score side and the P' = p * scale_g products of the value side are gone.  What it costs is one f16 rounding
//     (2^-12 relative, random sign) of every code * scale product.
//   * Scores and P.V run on v_mfma_f32_32x32x16: a K fragment read from LDS (1 KiB) feeds 32 cycles of matrix work
//     instead of 16, which is what lets the LDS keep four SIMDs' matrix cores fed.
//   * Roles.  Two score waves (32 heads each, the whole absorbed query row of a head in registers: 144 VGPRs), four
//     value waves (128 output columns x 64 heads each) and two staging waves that load and convert the next step's
//     rows.  A score wave and a staging wave share a SIMD: matrix work beside vector work.
//
// W only grows.  The staging waves agree on a step's W one iteration before they convert it (a maximum over the
// step's scale exponents through LDS, behind the step barrier that is there anyway); the score waves follow the
// same sequence of W and fold every growth into the rescaling factor they hand to the value waves.
#include <type_traits>

#include "common.hpp"
#include "kernels.hpp"
#include "mla_rows.hpp"

namespace zllm {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kLatent = 512;
constexpr int kRope = 64;
constexpr int kRowBytes = (kLatent + kRope) * 2; // 1152: 72 chunks of 16 bytes
constexpr int kStepTokens = 32;
constexpr int kTileBytes = kStepTokens * kRowBytes; // 36,864
constexpr int kTiles = 3;
// probabilities travel as f16 of p * 2^kPShift: p <= 2^8 by the lazy rescaling, so the product stays below 2^13 and
// p down to 2^-18 keeps f16's full precision
constexpr int kPShift = 4;

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

union Frag {
    u32x4 u;
    bf16x8 b;
    f16x8 h;
};

// 16-byte chunk swizzle of a tile row.  A row is 4.5 bank lines (256 B) long, so a row's parity already picks the upper or
// lower half of a line; row bits 1 and 2 go into chunk bits 2 and 1.  Measured rules of this LDS (one lane per 256-byte line,
// SQ_LDS_BANK_CONFLICT): a 16-byte read serves sixteen lanes a cycle -- lane bits 0-2 free, bits 3 and 4 both flipped
// between the two halves of such a group -- so a score wave's fragment read (lane = (row, 16-byte slice of the k-step)) meets
// rows that differ in bits 0-3, the two halves in the slice's low bit as well; an 8-byte (transposed) read serves lanes
// 0-31, then 32-63: four rows x 64 contiguous bytes for the value waves, whose rows 0 / 2 and 1 / 3 need chunk bit 2 to
// differ; a 16-byte write serves eight consecutive lanes.  All three patterns come out conflict-free.
__device__ __forceinline__ unsigned int swz(unsigned int row)
{
    return ((row & 2u) << 1) | ((row & 4u) >> 1);
}

__device__ __forceinline__ unsigned int tile_offset(unsigned int row, unsigned int chunk)
{
    return row * kRowBytes + ((chunk ^ swz(row)) << 4);
}

__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// max / sum of a value with the one in lane ^ 32 (a head's tokens are split between the two lane halves)
__device__ __forceinline__ float pair_max(float v)
{
    const unsigned int bits = __float_as_uint(v);
    const u32x2_swap s = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    return fmaxf(__uint_as_float(s.x), __uint_as_float(s.y));
}

__device__ __forceinline__ float pair_sum(float v)
{
    const unsigned int bits = __float_as_uint(v);
    const u32x2_swap s = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    return __uint_as_float(s.x) + __uint_as_float(s.y);
}


// Sixteen codes of one scale group -> sixteen f16 values code * factor: the 16-byte chunks 2 k and 2 k + 1 of a tile row.
__device__ __forceinline__ void convert_run(const u32x4& codes, _Float16 f, unsigned char* tile, unsigned int row, unsigned int k)
{
    const f16x2 factor = {f, f};
    u32x4 out[2];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        unsigned int lo, hi;
        codes4_to_f16(codes[w], lo, hi);
        out[w >> 1][(w & 1) * 2] = __builtin_bit_cast(unsigned int, __builtin_bit_cast(f16x2, lo) * factor);
        out[w >> 1][(w & 1) * 2 + 1] = __builtin_bit_cast(unsigned int, __builtin_bit_cast(f16x2, hi) * factor);
    }
    *(u32x4*)(tile + tile_offset(row, 2u * k)) = out[0];
    *(u32x4*)(tile + tile_offset(row, 2u * k + 1u)) = out[1];
}

constexpr int kMaxSteps = 1024; // block-table entries of a split kept in LDS: one per 32-token step

// 2^-(W) for the tile's values, W = e_window - 127
__device__ __forceinline__ float window_down(int e_window)
{
    return __uint_as_float((unsigned int)(254 - min(max(e_window, 1), 253)) << 23);
}

__global__ __launch_bounds__(512) void mla_partial_x32(MlaDecodeParams p)
{
    __shared__ __align__(1024) unsigned char lds[kTiles * kTileBytes];
    __shared__ __align__(16) u32x4 lds_p[2][2][2][64]; // [parity][head tile][k-step][lane]: the lane's sixteen probabilities as f16 pairs
    __shared__ __align__(16) float lds_alpha[2][2][64]; // [parity][head tile][lane]: factor for the accumulators before this step's products
    __shared__ __align__(16) u32x4 lds_qrope[2][4][64]; // [score wave][k-step of the rope columns][lane]: the query's rope fragments
    __shared__ unsigned int lds_entry[kMaxSteps];       // block-table entry of every step of the split
    __shared__ int lds_tmax[4];                         // [step % 4]: largest biased scale exponent of the step's visible rows
    __shared__ unsigned int lds_flag[2];                // [head tile]: 1 + the last step whose probabilities the score wave has written
    __shared__ int lds_window[2];                       // [head tile]: the W the score wave ended on

    const unsigned int tid = threadIdx.x;
    const unsigned int lane = tid & 63u;
    const unsigned int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned int n32 = lane & 31u;
    const unsigned int half = lane >> 5;
    // grid coordinates, or looked up from the dense item number when the records are numbered that way
    unsigned int chunk = blockIdx.x;
    unsigned int b = gridDim.z - 1u - blockIdx.z; // rows of a chunk see more keys the later they come: longest first
    if (p.record_rows != 0u && !mla_locate_split(p, blockIdx.x, lane, b, chunk)) {
        return;
    }
    const size_t row = p.record_rows != 0u ? (size_t)blockIdx.x : (size_t)b * p.max_chunks + chunk;
    unsigned int seq;
    const unsigned int len = visible_tokens(p.ctx_lens, p.query_rows, b, seq);
    const unsigned int n_splits = min(p.max_chunks, (len + p.chunk_tokens - 1u) / p.chunk_tokens);
    const unsigned int span = n_splits > 0u ? min(p.chunk_tokens, (((len + n_splits - 1u) / n_splits) + 31u) & ~31u) : p.chunk_tokens;
    const unsigned long long c_start64 = (unsigned long long)chunk * span;
    const bool score_role = wave < 2u;
    const bool staging_role = wave == 4u || wave == 5u;
    if (c_start64 >= len) { // empty split: (max, sum) = (-inf, 0), the merge skips it
        if (score_role && half == 0u) {
            const unsigned int head = blockIdx.y * 64u + wave * 32u + n32;
            if (head < p.heads) {
                const size_t rec = row * p.heads + head;
                p.stats[rec * 2] = kNegInf;
                p.stats[rec * 2 + 1] = 0.0f;
            }
        }
        return;
    }
    const unsigned int c_start = (unsigned int)c_start64;
    const unsigned int c_end = (unsigned int)min((unsigned long long)len, c_start64 + span);
    const unsigned int steps = (c_end - c_start + kStepTokens - 1) / kStepTokens;
    if (tid < 4u) {
        lds_tmax[tid] = 0;
    }
    if (tid < 2u) {
        lds_flag[tid] = 0u;
    }
    {
        const unsigned int* table = p.tables != nullptr ? p.tables + (size_t)seq * p.table_stride : nullptr;
        for (unsigned int n = tid; n < steps; n += 512u) {
            const unsigned int t0 = c_start + n * kStepTokens;
            const unsigned int page = (p.block_tokens & (p.block_tokens - 1u)) == 0 ? t0 >> p.block_shift : t0 / p.block_tokens;
            lds_entry[n] = table != nullptr ? table[page] : page;
        }
    }
    __syncthreads();

    // first physical row of step n (pages hold a multiple of 32 tokens: the 32 rows of a step lie in one page)
    const bool pow2 = (p.block_tokens & (p.block_tokens - 1u)) == 0;
    const unsigned int last_step = steps - 1u;
    auto first_row = [&](unsigned int n) __attribute__((always_inline)) -> unsigned long long {
        const unsigned int step = min(n, last_step);
        const unsigned int t0 = c_start + step * kStepTokens;
        const unsigned int e = __builtin_amdgcn_readfirstlane(lds_entry[step]);
        return pow2 ? ((unsigned long long)e << p.block_shift) + (t0 & (p.block_tokens - 1u)) : (unsigned long long)e * p.block_tokens + t0 % p.block_tokens;
    };

    if (staging_role) {
        // ============================== staging waves ==============================
        // Thread = (row, quarter q of the row's first 256 columns): runs of 16 codes q, q + 4, q + 8, q + 12 (run i lies in
        // scale group i), a quarter of the row's rope columns and the row's eight scales, whose largest exponent one thread
        // of the row hands to the step's maximum.  The rows of step n are requested in iteration n - 4, their scale
        // exponents reduced in iteration n - 2, and they are converted in iteration n - 1: three steps' rows are in
        // registers at any time (a load has three iterations to land).
        const unsigned int st = (wave - 4u) * 64u + lane;
        const unsigned int row = st >> 2;
        const unsigned int part = st & 3u;
        struct Raw {
            u32x4 codes[4];
            u32x4 rope[2];
            u32x4 scales;
        };
        // The loads are written by hand and so are their waits: the load counter is in order, every batch is seven loads, the
        // scales first, and a batch is issued in every iteration (past the last step it re-reads the last one), so "rows of
        // three iterations ago" is vmcnt(14) and "scales of two iterations ago" vmcnt(13).  (Left to the compiler the waits
        // of this ring come out as vmcnt(0): every iteration then waits for the loads it has just issued.)
        auto load_rows = [&](Raw& raw, unsigned int n) __attribute__((always_inline)) {
            const unsigned long long r = first_row(n) + row;
            const unsigned char* scales = (const unsigned char*)p.latent_scales + r * (kLatent / 64 * 2);
            const unsigned char* codes = (const unsigned char*)p.latent_codes + r * kLatent + part * 16u;
            const unsigned char* rope = (const unsigned char*)p.rope_cache + r * (kRope * 2) + part * 32u;
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(raw.scales) : "v"(scales));
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(raw.codes[0]) : "v"(codes));
            asm volatile("global_load_dwordx4 %0, %1, off offset:64" : "=v"(raw.codes[1]) : "v"(codes));
            asm volatile("global_load_dwordx4 %0, %1, off offset:128" : "=v"(raw.codes[2]) : "v"(codes));
            asm volatile("global_load_dwordx4 %0, %1, off offset:192" : "=v"(raw.codes[3]) : "v"(codes));
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(raw.rope[0]) : "v"(rope));
            asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(raw.rope[1]) : "v"(rope));
        };
        auto wait_rows = [&](Raw& raw) __attribute__((always_inline)) {
            asm volatile("s_waitcnt vmcnt(14)" : "+v"(raw.scales), "+v"(raw.codes[0]), "+v"(raw.codes[1]), "+v"(raw.codes[2]), "+v"(raw.codes[3]),
                         "+v"(raw.rope[0]), "+v"(raw.rope[1])::"memory");
        };
        auto wait_scales = [&](Raw& raw) __attribute__((always_inline)) {
            asm volatile("s_waitcnt vmcnt(13)" : "+v"(raw.scales)::"memory");
        };
        // largest biased exponent among the row's eight bf16 scales (0 for a row past the end of the sequence)
        auto reduce_scales = [&](const u32x4& sc, unsigned int n) __attribute__((always_inline)) {
            if (n < steps && part == 0u) {
                unsigned int top = 0;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    top = max(top, max(sc[w] & 0x7fffu, (sc[w] >> 16) & 0x7fffu));
                }
                const unsigned int token = c_start + n * kStepTokens + row;
                const int e = token < len ? (int)(top >> 7) : 0;
                const unsigned int at = (unsigned int)(unsigned long long)(__attribute__((address_space(3))) int*)&lds_tmax[n & 3u];
                asm volatile("ds_max_i32 %0, %1" ::"v"(at), "v"(e) : "memory");
            }
        };
        auto convert = [&](const Raw& raw, unsigned int n, int e_window) __attribute__((always_inline)) {
            unsigned char* tile = lds + (n % kTiles) * kTileBytes;
            const unsigned int token = c_start + n * kStepTokens + row;
            // a row past the end gets factor 0: whatever its codes and scales are (NaN included), its tile row is zeros
            const bool visible = token < len;
            const float down = window_down(e_window);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const unsigned int bits = (i & 1) ? (raw.scales[i >> 1] & 0xffff0000u) : (raw.scales[i >> 1] << 16);
                convert_run(raw.codes[i], visible ? (_Float16)(__uint_as_float(bits) * down) : (_Float16)0.0f, tile, row, part + 4u * i);
            }
            *(u32x4*)(tile + tile_offset(row, 64u + 2u * part)) = raw.rope[0];
            *(u32x4*)(tile + tile_offset(row, 65u + 2u * part)) = raw.rope[1];
        };
        Raw r0, r1, r2; // the rows of step n wait in r(n % 3)
        load_rows(r0, 0u);
        load_rows(r1, 1u);
        load_rows(r2, 2u);
        wait_scales(r1); // and with it the scales of step 0
        asm volatile("" : "+v"(r0.scales));
        reduce_scales(r0.scales, 0u);
        reduce_scales(r1.scales, 1u);
        lds_barrier();
        int window = lds_tmax[0];
        wait_rows(r0);
        convert(r0, 0u, window);
        load_rows(r0, 3u);
        lds_barrier();
        // iteration i: convert step i + 1, request the rows of step i + 4 into the registers that frees, reduce the scale
        // exponents of step i + 2, look up the table entry of step i + 5
        auto iteration = [&](unsigned int i, Raw& convert_now, Raw& reduce_now) __attribute__((always_inline)) {
            wait_rows(convert_now);
            if (i + 1u < steps) {
                window = max(window, lds_tmax[(i + 1u) & 3u]);
                convert(convert_now, i + 1u, window);
            }
            wait_scales(reduce_now);
            reduce_scales(reduce_now.scales, i + 2u);
            load_rows(convert_now, i + 4u);
            if (tid == 256u) {
                lds_tmax[(i + 3u) & 3u] = 0; // read last in iteration i - 1, accumulated next in iteration i + 1
            }
            lds_barrier();
        };
        for (unsigned int i = 0;; i += 3u) {
            iteration(i, r1, r2);
            if (i + 1u > steps) {
                break;
            }
            iteration(i + 1u, r2, r0);
            if (i + 2u > steps) {
                break;
            }
            iteration(i + 2u, r0, r1);
            if (i + 3u > steps) {
                break;
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the loads past the last step land before the wave ends
        lds_barrier(); // the score waves publish their window behind this one
        return;
    }
    if (score_role) {
        lds_barrier(); // the converting waves reduce the first steps' scale exponents ...
        lds_barrier(); // ... and convert step 0
        // ============================== score waves ==============================
        // S^T[token, head] = K . Q^T for 32 tokens x 32 heads as 2 x 2 tiles of v_mfma_f32_16x16x32: A = K fragment from LDS
        // (lane = (token row m of the tile, 8-column slice j of the k-step)), B = query fragment in registers (lane = (head
        // column m, slice j)); every fragment feeds two MFMAs and the four accumulators are four independent chains (a
        // 32x32x16 MFMA that adds to the result of an earlier one was measured to wait some 160 cycles for it: one wave
        // with two such chains ran at 83 cycles an instruction).  C of tile (T, H): lane (m, j) holds head 16 H + m, tokens
        // 16 T + 4 j + r.
        const unsigned int m16 = lane & 15u;
        const unsigned int j4 = lane >> 4;
        const unsigned int head0 = blockIdx.y * 64u + wave * 32u + m16; // the lane's head of tile H is head0 + 16 H
        Frag qf[2][16]; // [head tile][k-step]: the latent part of the absorbed query; the rope part waits in LDS
        int lat_exp[2]; // exponent of the power of two a head's latent query was divided by
#pragma unroll
        for (int H = 0; H < 2; ++H) {
            const unsigned int head = head0 + 16u * H;
            const bool head_live = head < p.heads;
            const unsigned short* qa = p.absorbed + ((size_t)b * p.heads + min(head, p.heads - 1u)) * (kLatent + kRope) + j4 * 8u;
            // the latent part goes to f16 after the head's row is divided by the power of two of its largest magnitude: one
            // pass over the row for that magnitude, a second one that keeps the row
            float top = 0.0f;
#pragma unroll
            for (int ks = 0; ks < 16; ++ks) {
                const u32x4 v = *(const u32x4*)(qa + ks * 32);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    top = fmaxf(top, fmaxf(fabsf(__uint_as_float(v[w] << 16)), fabsf(__uint_as_float(v[w] & 0xffff0000u))));
                }
            }
            asm volatile("" : "+v"(top)::"memory");
            top = wave_max_16x4(head_live ? top : 0.0f);
            const unsigned int top_exp = min(max((__float_as_uint(top) >> 23) & 0xffu, 87u), 253u); // a zero or vanishing row counts as 2^-40
            lat_exp[H] = (int)top_exp - 127;
            const float down = head_live ? __uint_as_float((254u - top_exp) << 23) : 0.0f;
#pragma unroll
            for (int ks = 0; ks < 16; ++ks) {
                const u32x4 v = *(const u32x4*)(qa + ks * 32);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    qf[H][ks].u[w] = pack_f16_hw(__uint_as_float(v[w] << 16) * down, __uint_as_float(v[w] & 0xffff0000u) * down);
                }
            }
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                u32x4 v = *(const u32x4*)(qa + (16 + ks) * 32);
                if (!head_live) {
                    v = u32x4{0u, 0u, 0u, 0u};
                }
                lds_qrope[wave][2 * H + ks][lane] = v; // read back by this wave only
            }
        }
        const bool tile_live = (unsigned int)__builtin_amdgcn_readfirstlane((int)(blockIdx.y * 64u + wave * 32u)) < p.heads;
        // K fragment of token tile T, k-step ks: row 16 T + m, chunk 4 ks + j; the chunk's low three bits go through the swizzle,
        // (ks >> 1) * 128 bytes are an immediate
        unsigned int kbase[2][2];
#pragma unroll
        for (int T = 0; T < 2; ++T) {
#pragma unroll
            for (int par = 0; par < 2; ++par) {
                const unsigned int row = 16u * T + m16;
                kbase[T][par] = row * kRowBytes + (((4u * par + j4) ^ swz(row)) << 4);
            }
        }
        const unsigned int lds_base = (unsigned int)(unsigned long long)(__attribute__((address_space(3))) const unsigned char*)lds;
        const unsigned int qrope_lds = (unsigned int)(unsigned long long)(__attribute__((address_space(3))) const u32x4*)&lds_qrope[wave][0][lane];
        float run_max[2] = {kNegInf, kNegInf}, run_sum[2] = {0.0f, 0.0f};
        float neg_ref_shifted[2] = {(float)kPShift, (float)kPShift}; // minus the reference the scores are taken against, plus the hand-over shift
        float neg_ref[2] = {0.0f, 0.0f};
        const float scale_log2 = p.score_scale * kLog2e;
        int window = 0; // biased exponent of W; 0 = nothing seen yet
        // A step is scored in two iterations: iteration i multiplies tile i, iteration i + 1 opens with the fragment requests
        // of tile i + 1 and runs the softmax of step i while they are on their way (the matrix pipeline would otherwise sit
        // through an LDS round trip at the start of every step).  The value waves accumulate step i in iteration i + 1
        // either way; they find its probabilities by a flag in LDS instead of behind the iteration's barrier.
        constexpr int kRing = 3;
        Frag kf[kRing][4], qr[4]; // a group = two k-steps: [slot][2 (ks & 1) + T]
        f32x4 s_prev[2][2]; // [T][H]: q . k of the step before, all 576 columns, exact units
        float grow_prev = 1.0f;
        int e_tile = __builtin_amdgcn_readfirstlane(lds_tmax[0]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the hand-counted waits below start from zero
        unsigned int at[2][2];
#define X32_LOAD_GROUP(SLOT, G)                                                                                                      \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(kf[SLOT][0].u) : "v"(at[0][0]), "i"((G) * 128));                              \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(kf[SLOT][1].u) : "v"(at[1][0]), "i"((G) * 128));                              \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(kf[SLOT][2].u) : "v"(at[0][1]), "i"((G) * 128));                              \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(kf[SLOT][3].u) : "v"(at[1][1]), "i"((G) * 128))
#define X32_WAIT_GROUP(N, SLOT)                                                                                                      \
    asm volatile("s_waitcnt lgkmcnt(" #N ")" : "+v"(kf[SLOT][0].u), "+v"(kf[SLOT][1].u), "+v"(kf[SLOT][2].u), "+v"(kf[SLOT][3].u)::"memory")
        // Fragments are requested by hand, two groups (of two k-steps, eight MFMAs) ahead of the MFMAs that use them, and
        // waited for by count (LDS operations of a wave complete in order).  Group g = 0..7 holds latent columns 64 g .. in
        // ring slot g % 3; group 8 is the rope columns, with this wave's LDS copy of the query's rope part.
        auto open_step = [&](unsigned int n) __attribute__((always_inline)) { // the first two groups' requests
            const unsigned int tile_lds = lds_base + (n % kTiles) * kTileBytes;
#pragma unroll
            for (int T = 0; T < 2; ++T) {
                at[T][0] = tile_lds + kbase[T][0];
                at[T][1] = tile_lds + kbase[T][1];
            }
            X32_LOAD_GROUP(0, 0);
            X32_LOAD_GROUP(1, 1);
        };
        auto multiply_step = [&]() __attribute__((always_inline)) { // the step opened last: S^T into s_prev
            X32_LOAD_GROUP(2, 2);
            // window of this step: the accumulators of the value waves follow it through alpha
            grow_prev = 1.0f;
            if (e_tile > window) {
                if (window != 0) {
                    grow_prev = __uint_as_float((unsigned int)(127 - min(e_tile - window, 126)) << 23);
                }
                window = e_tile;
            }
            f32x4 acc[2][2];
#pragma unroll
            for (int T = 0; T < 2; ++T) {
                acc[T][0] = f32x4{0.f, 0.f, 0.f, 0.f};
                acc[T][1] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            // The waits count what may still be outstanding behind a group; up to four writes of the step before's
            // probabilities stand between the opening requests and the rest, which the first two counts allow for.
#define X32_LATENT_GROUP(G, N)                                                                                                       \
    X32_WAIT_GROUP(N, (G) % 3);                                                                                                       \
    _Pragma("unroll") for (int par = 0; par < 2; ++par)                                                                               \
    {                                                                                                                                 \
        _Pragma("unroll") for (int T = 0; T < 2; ++T)                                                                                 \
        {                                                                                                                             \
            _Pragma("unroll") for (int H = 0; H < 2; ++H)                                                                             \
            {                                                                                                                         \
                                acc[T][H] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[(G) % 3][2 * par + T].h, qf[H][2 * (G) + par].h, acc[T][H], 0, 0, 0); \
            }                                                                                                                         \
        }                                                                                                                             \
    }
            X32_LATENT_GROUP(0, 8)
            X32_LOAD_GROUP(0, 3);
            X32_LATENT_GROUP(1, 8)
            X32_LOAD_GROUP(1, 4);
            X32_LATENT_GROUP(2, 8)
            X32_LOAD_GROUP(2, 5);
            X32_LATENT_GROUP(3, 8)
            X32_LOAD_GROUP(0, 6);
            X32_LATENT_GROUP(4, 8)
            X32_LOAD_GROUP(1, 7);
            X32_LATENT_GROUP(5, 8)
            X32_LOAD_GROUP(2, 8);
#pragma unroll
            for (int f = 0; f < 4; ++f) {
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(qr[f].u) : "v"(qrope_lds), "i"(f * 1024));
            }
            X32_LATENT_GROUP(6, 12)
            X32_LATENT_GROUP(7, 8)
#undef X32_LATENT_GROUP
            // tile values are code * scale / 2^(window - 127) and a head's latent query was divided by 2^lat_exp: the latent
            // sums are brought to exact units by that power of two before the rope products are added on top
            const int w_exp = min(max(window, 1), 253);
#pragma unroll
            for (int H = 0; H < 2; ++H) {
                const float lat_to_exact = __uint_as_float((unsigned int)min(max(w_exp + lat_exp[H], 7), 247) << 23);
                acc[0][H] *= lat_to_exact;
                acc[1][H] *= lat_to_exact;
            }
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(kf[2][0].u), "+v"(kf[2][1].u), "+v"(kf[2][2].u), "+v"(kf[2][3].u), "+v"(qr[0].u), "+v"(qr[1].u),
                         "+v"(qr[2].u), "+v"(qr[3].u)::"memory");
#pragma unroll
            for (int par = 0; par < 2; ++par) {
#pragma unroll
                for (int T = 0; T < 2; ++T) {
#pragma unroll
                    for (int H = 0; H < 2; ++H) {
                        acc[T][H] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[2][2 * par + T].b, qr[2 * H + par].b, acc[T][H], 0, 0, 0);
                    }
                }
            }
#pragma unroll
            for (int T = 0; T < 2; ++T) {
                s_prev[T][0] = acc[T][0];
                s_prev[T][1] = acc[T][1];
            }
        };
        auto softmax_step = [&](unsigned int n) __attribute__((always_inline)) { // step n from s_prev: probabilities and alpha to the value waves
            const unsigned int t0 = c_start + n * kStepTokens;
#pragma unroll
            for (int H = 0; H < 2; ++H) {
                float sc[8]; // tokens 16 T + 4 j + r at index 4 T + r
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    sc[e] = fmaf(s_prev[e >> 2][H][e & 3], scale_log2, neg_ref_shifted[H]);
                }
                if (t0 + kStepTokens > len) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const unsigned int token = t0 + 16u * (e >> 2) + 4u * j4 + (e & 3);
                        sc[e] = token < len ? sc[e] : kNegInf;
                    }
                }
                float lane_max = sc[0];
#pragma unroll
                for (int e = 1; e < 8; ++e) {
                    lane_max = fmaxf(lane_max, sc[e]);
                }
                // Online softmax with lazy rescaling: the stored maximum (the reference the scores are already relative to)
                // only moves when a score exceeds it by 2^8 (p stays <= 256)
                float alpha = grow_prev;
                if (__any(lane_max > 8.0f + (float)kPShift || run_max[H] == kNegInf)) {
                    const float step_max = wave_max_16x4(lane_max) - (float)kPShift;
                    const float ref = -neg_ref[H];
                    float new_max = run_max[H];
                    if (step_max > 8.0f || run_max[H] == kNegInf) {
                        new_max = fmaxf(run_max[H], ref + step_max);
                    }
                    const float safe_max = new_max == kNegInf ? 0.0f : new_max;
                    const float shrink = __builtin_amdgcn_exp2f(run_max[H] - safe_max); // 0 on the first step: nothing accumulated yet
                    alpha *= shrink;
                    const float delta = safe_max - ref;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        sc[e] -= delta;
                    }
                    run_max[H] = new_max;
                    neg_ref[H] = -safe_max;
                    neg_ref_shifted[H] = neg_ref[H] + (float)kPShift;
                    run_sum[H] *= shrink;
                }
                float pr[8];
                float step_sum = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    pr[e] = __builtin_amdgcn_exp2f(sc[e]);
                    step_sum += pr[e];
                }
                run_sum[H] += step_sum;
                // value lane (half, head column) takes the tokens 16 s + 8 half + 0..7 of k-step s as one 16-byte fragment: this
                // lane's four tokens of token tile T are the 8 bytes (j % 2) of the fragment (s = T, half = j / 2)
#pragma unroll
                for (int T = 0; T < 2; ++T) {
                    const u32x2 piece = {pack_f16_hw(pr[4 * T], pr[4 * T + 1]), pack_f16_hw(pr[4 * T + 2], pr[4 * T + 3])};
                    *(u32x2*)((unsigned char*)&lds_p[n & 1u][wave][T][32u * (j4 >> 1) + 16u * H + m16] + 8u * (j4 & 1u)) = piece;
                }
                if (j4 == 0u) {
                    lds_alpha[n & 1u][wave][16u * H + m16] = alpha;
                }
            }
            // LDS operations of a wave complete in order: whoever reads n + 1 here finds the writes above done
            if (lane == 0u) {
                lds_flag[wave] = n + 1u;
            }
        };
        if (tile_live) {
            open_step(0u);
        }
        for (unsigned int i = 0; i <= steps; ++i) {
            if (tile_live) {
                if (i > 0) {
                    if (i < steps) {
                        open_step(i);
                    }
                    softmax_step(i - 1u);
                }
                if (i < steps) {
                    multiply_step();
                }
            }
            // the next step's window is final since the barrier before this iteration
            e_tile = __builtin_amdgcn_readfirstlane(lds_tmax[(i + 1u) & 3u]);
            lds_barrier();
        }
#undef X32_WAIT_GROUP
#undef X32_LOAD_GROUP
        if (lane == 0u) {
            lds_window[wave] = window;
        }
#pragma unroll
        for (int H = 0; H < 2; ++H) {
            const float total = wave_sum_16x4(run_sum[H]) * (1.0f / (float)(1 << kPShift));
            const unsigned int head = head0 + 16u * H;
            if (head < p.heads && j4 == 0u) {
                const size_t rec = row * p.heads + head;
                p.stats[rec * 2] = run_max[H];
                p.stats[rec * 2 + 1] = total;
            }
        }
        lds_barrier();
        return;
    }

    // ============================== value waves ==============================
    // O^T[column, head] += V^T . P on v_mfma_f32_32x32x16: A = V^T fragment read transposed from the row-major tile (lane =
    // column, the 8 tokens 16 s + 8 (lane / 32) + 0..7 of k-step s), B = the probabilities of the lane's head column for
    // the same tokens, one 16-byte read of what the score wave left.
    const unsigned int v = (wave & 1u) | ((wave >> 2) << 1); // waves 2, 3, 6, 7 -> 0..3: output columns [128 v, 128 v + 128)
    f32x16 acc[2][4];
#pragma unroll
    for (int ht = 0; ht < 2; ++ht) {
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                acc[ht][ct][r] = 0.0f;
            }
        }
    }
    const bool second_tile = (unsigned int)__builtin_amdgcn_readfirstlane((int)(blockIdx.y * 64u + 32u)) < p.heads;
    const unsigned int i16 = lane & 15u;
    const unsigned int cb = (lane >> 4) & 1u;
    const unsigned int lds_base = (unsigned int)(unsigned long long)(__attribute__((address_space(3))) const unsigned char*)lds;
    // the lane's 8-byte piece inside a 4-token x 16-column block of the tile: token row 8 (lane / 32) + 4 dq + (lane % 16) / 4
    // (row bit 2 = dq enters the swizzle; k-step s adds sixteen rows, an immediate)
    unsigned int vbase[2][4];
#pragma unroll
    for (int dq = 0; dq < 2; ++dq) {
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            const unsigned int row = 8u * half + 4u * dq + (i16 >> 2);
            const unsigned int chunk16 = 16u * v + 4u * ct + 2u * cb + ((i16 & 3u) >> 1);
            vbase[dq][ct] = row * kRowBytes + ((chunk16 ^ swz(row)) << 4) + (i16 & 1u) * 8u;
        }
    }
    // The value waves also convert the second 256 columns of a step's rows: thread = (row, eighth e of that half), runs
    // 16 + e and 24 + e of 16 codes, scale groups 4 + e / 4 and 6 + e / 4; same timing as the staging waves.
    const unsigned int vt = v * 64u + lane;
    // eight consecutive lanes = two rows x four runs: their 16-byte writes land in eight different slots of a bank line
    const unsigned int crow = ((vt >> 4) << 1) | (vt & 1u);
    const unsigned int part8 = (vt >> 1) & 7u;
    struct Raw {
        u32x4 codes[2];
        unsigned int scale[2]; // bf16 bits
    };
    // hand-written loads and waits, as in the staging waves: four loads a batch, one batch an iteration
    auto load_rows = [&](Raw& raw, unsigned int n) __attribute__((always_inline)) {
        const unsigned long long r = first_row(n) + crow;
        const unsigned char* codes = (const unsigned char*)p.latent_codes + r * kLatent + 256u + part8 * 16u;
        const unsigned short* sc = p.latent_scales + r * (kLatent / 64) + 4u + (part8 >> 2);
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(raw.codes[0]) : "v"(codes));
        asm volatile("global_load_dwordx4 %0, %1, off offset:128" : "=v"(raw.codes[1]) : "v"(codes));
        asm volatile("global_load_ushort %0, %1, off" : "=v"(raw.scale[0]) : "v"(sc));
        asm volatile("global_load_ushort %0, %1, off offset:4" : "=v"(raw.scale[1]) : "v"(sc));
    };
    auto wait_rows = [&](Raw& raw) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(8)" : "+v"(raw.codes[0]), "+v"(raw.codes[1]), "+v"(raw.scale[0]), "+v"(raw.scale[1])::"memory");
    };
    auto convert = [&](const Raw& raw, unsigned int n, int e_window) __attribute__((always_inline)) {
        unsigned char* tile = lds + (n % kTiles) * kTileBytes;
        const unsigned int token = c_start + n * kStepTokens + crow;
        const bool visible = token < len;
        const float down = window_down(e_window);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            convert_run(raw.codes[i], visible ? (_Float16)(__uint_as_float(raw.scale[i] << 16) * down) : (_Float16)0.0f, tile, crow, 16u + part8 + 8u * i);
        }
    };
    Raw r0, r1, r2; // the rows of step n wait in r(n % 3)
    load_rows(r0, 0u);
    load_rows(r1, 1u);
    load_rows(r2, 2u);
    lds_barrier();
    int cwindow = lds_tmax[0];
    wait_rows(r0);
    convert(r0, 0u, cwindow);
    load_rows(r0, 3u);
    lds_barrier();
    unsigned int value_tile = 0;
    auto iteration = [&](unsigned int i, Raw& convert_now) __attribute__((always_inline)) {
        wait_rows(convert_now);
        if (i + 1u < steps) {
            cwindow = max(cwindow, lds_tmax[(i + 1u) & 3u]);
            convert(convert_now, i + 1u, cwindow);
        }
        load_rows(convert_now, i + 4u);
        if (i > 0) {
            const unsigned int parity = (i - 1u) & 1u;
            union VFrag {
                s16x4 s[2];
                f16x8 h;
            };
            const unsigned int tile_lds = lds_base + value_tile * kTileBytes;
            // The sixteen MFMAs of a step visit the eight accumulators twice, k-step 0 of all of them first.  All eight
            // fragments (sixteen transposed reads) are requested here: they land while this wave looks for the step's probabilities.
            VFrag vf[8]; // [4 s + ct]
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int s = u >> 2, ct = u & 3;
                const unsigned int at0 = tile_lds + vbase[0][ct], at1 = tile_lds + vbase[1][ct];
                if (s == 0) {
                    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(vf[u].s[0]) : "v"(at0));
                    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(vf[u].s[1]) : "v"(at1));
                } else {
                    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(vf[u].s[0]) : "v"(at0), "i"(16 * kRowBytes));
                    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(vf[u].s[1]) : "v"(at1), "i"(16 * kRowBytes));
                }
            }
            // the probabilities of step i - 1 are written early in this iteration: wait for the score waves' flags
            while (true) {
                const unsigned int f0 = __builtin_amdgcn_readfirstlane(((volatile unsigned int*)lds_flag)[0]);
                const unsigned int f1 = second_tile ? __builtin_amdgcn_readfirstlane(((volatile unsigned int*)lds_flag)[1]) : i;
                if (f0 >= i && f1 >= i) {
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
            Frag pf[2][2];
            float alpha[2];
#pragma unroll
            for (int ht = 0; ht < 2; ++ht) {
                pf[ht][0].u = lds_p[parity][ht][0][lane];
                pf[ht][1].u = lds_p[parity][ht][1][lane];
                alpha[ht] = lds_alpha[parity][ht][n32];
            }
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vf[0].s[0]), "+v"(vf[0].s[1]), "+v"(vf[1].s[0]), "+v"(vf[1].s[1]), "+v"(vf[2].s[0]), "+v"(vf[2].s[1]),
                         "+v"(vf[3].s[0]), "+v"(vf[3].s[1]), "+v"(vf[4].s[0]), "+v"(vf[4].s[1]), "+v"(vf[5].s[0]), "+v"(vf[5].s[1]), "+v"(vf[6].s[0]),
                         "+v"(vf[6].s[1]), "+v"(vf[7].s[0]), "+v"(vf[7].s[1])::"memory");
#pragma unroll
            for (int ht = 0; ht < 2; ++ht) {
                if ((ht == 0 || second_tile) && __any(alpha[ht] != 1.0f)) {
#pragma unroll
                    for (int ct = 0; ct < 4; ++ct) {
                        acc[ht][ct] *= alpha[ht];
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(2);
#define X32_PV(U, N)                                                                                                                 \
    asm volatile("" : "+v"(vf[U].s[0]), "+v"(vf[U].s[1]));                                                                            \
    acc[0][(U)&3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[U].h, pf[0][(U) >> 2].h, acc[0][(U)&3], 0, 0, 0);       \
    if (second_tile) {                                                                                                  \
        acc[1][(U)&3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[U].h, pf[1][(U) >> 2].h, acc[1][(U)&3], 0, 0, 0);                   \
    }
            X32_PV(0, 14)
            X32_PV(1, 12)
            X32_PV(2, 10)
            X32_PV(3, 8)
            X32_PV(4, 6)
            X32_PV(5, 4)
            X32_PV(6, 2)
            X32_PV(7, 0)
#undef X32_PV
            __builtin_amdgcn_s_setprio(0);
            value_tile = value_tile == kTiles - 1u ? 0u : value_tile + 1u;
        }
        lds_barrier();
    };
    for (unsigned int i = 0;; i += 3u) {
        iteration(i, r1);
        if (i + 1u > steps) {
            break;
        }
        iteration(i + 1u, r2);
        if (i + 2u > steps) {
            break;
        }
        iteration(i + 2u, r0);
        if (i + 3u > steps) {
            break;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the loads past the last step land before their registers are reused
    lds_barrier(); // the score waves leave the window they ended on behind this one
#pragma unroll
    for (int ht = 0; ht < 2; ++ht) {
        const unsigned int out_head = blockIdx.y * 64u + 32u * ht + n32;
        if (out_head < p.heads) {
            const int window = lds_window[ht];
            // acc = sum p 2^kPShift v / 2^(window - 127)
            const float up = __uint_as_float((unsigned int)min(max(window - kPShift, 1), 253) << 23);
            float* out = p.partial + (row * p.heads + out_head) * kLatent + 128u * v + 4u * half;
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x4 o = {acc[ht][ct][4 * q] * up, acc[ht][ct][4 * q + 1] * up, acc[ht][ct][4 * q + 2] * up, acc[ht][ct][4 * q + 3] * up};
                    *(f32x4*)(out + 32 * ct + 8 * q) = o;
                }
            }
        }
    }
}

} // namespace

bool mla_partial_x32_takes(const MlaDecodeParams& p)
{
    return p.heads > 32u && p.selection == nullptr && p.latent_dim == 512u && p.rope_dim == 64u && p.block_tokens % kStepTokens == 0 &&
           p.chunk_tokens % kStepTokens == 0 && p.chunk_tokens <= (unsigned int)(kMaxSteps * kStepTokens);
}

hipError_t launch_mla_partial_x32(const MlaDecodeParams& p, hipStream_t stream)
{
    const dim3 grid = p.record_rows != 0u ? dim3(p.record_rows, (p.heads + 63) / 64, 1) : dim3(p.max_chunks, (p.heads + 63) / 64, p.batch);
    mla_partial_x32<<<grid, dim3(512), 0, stream>>>(p);
    return hipGetLastError();
}

} // namespace zllm

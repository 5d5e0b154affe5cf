// Chunked-prefill GQA attention over a paged KV cache — gfx950, f16 MFMA: gqa_prefill_q8 for Q8g64 caches (head_dim 128,
// described first), gqa_prefill_f16 for f16 caches (head_dim 128 and 256, further down).
//
// T query rows appended at `position` attend the cached prefix plus the chunk itself (causal,
// optional sliding window).  Replaces the per-(row, head) block attention the reference runs for this
// case (src/backend/rocm/attention.rs:2232-2242 -> tensor/attention/source.hip:618-686).
//
// A workgroup (8 waves) owns one KV head and a tile of query rows; its 256 MFMA columns enumerate
// (row, head-in-group) pairs, 32 per wave, so one K/V tile serves every query head of the group.
// Two waves share a SIMD, so the LDS and MFMA latencies of one are covered by the other.
// Per 32-token step the workgroup converts the K and V codes ONCE into LDS as f16 integers (exact)
// with their f32 group scales beside them; each wave then runs
//   S^T[token, col]  = sum_g k_scale[token, g] * (Kcodes_g[token, :] . Q'_g[col, :])   (f16 MFMA, exact products)
//   online softmax per column (wave shuffles)
//   O^T[dim, col]   += Vcodes^T[dim, token] . P'_g[token, col],  P'_g = p * v_scale_g as f16 hi (+ lo)
// The codes stay integers on purpose: a tile of code * scale products rounded to f16 moves single scores by
// up to 2^-11 of their largest term, which outlier channels turn into output errors above the 2e-3 bound.
// Q' is the wave's query tile times one power of two (largest magnitude in [2^8, 2^9)), undone in the fused
// multiply-add that feeds exp2.  P' must stay inside f16 range for any scale a cache can hold: the exponent of
// the largest V scale met so far (each V staging wave reduces the scales it converts) is subtracted from the softmax
// reference, so accumulators and running sum carry the same power of two and it cancels in the division.
// K is read from LDS with ds_read_b128, V transposed with ds_read_b64_tr_b16; a 16-byte XOR swizzle
// keeps both conflict-free.
// The kernel is bound by the vector-ALU instructions it issues, not by the matrix cores, so whatever does not depend on
// every (token, column) pair stays out of the common path of a step: the tile buffer is a literal (LDS addresses in
// immediates), edge masks and the low-order P' pass sit behind wave-uniform branches, and a column's reference
// (running maximum, V window) is only touched when some lane's score passes it.
#include <type_traits>

#include "common.hpp"
#include "kernels.hpp"

namespace zllm {

namespace {

// Fences for the instruction scheduler between the phases of a step (they keep the early LDS requests early).
#define PREFILL_PHASE_FENCE() __builtin_amdgcn_sched_barrier(0)

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kStep = 32;                 // tokens per step
constexpr int kD = 128;                   // head_dim handled by this kernel
constexpr int kRowBytes = kD * 2;         // one token of one KV head as f16
constexpr int kTileBytes = kStep * kRowBytes; // 8 KiB
constexpr float kPBias = 8.0f;            // probabilities are carried as p * 2^8: f16 stays normal down to p = 2^-22
constexpr float kLoThreshold = 8.0f;      // see the P.V stage
constexpr int kColTiles = 2;              // 16-column MFMA tiles per wave
constexpr int kWaves = 256 / (16 * kColTiles);
constexpr int kThreads = 64 * kWaves;
constexpr unsigned long long kComputeUnitsPrefill = 256; // compute units of the device the kernels are tuned for

typedef short s16x4 __attribute__((ext_vector_type(4)));

union Frag {
    u32x4 u;
    f16x8 h;
};

// Chunk swizzle for the 64-bank LDS (256 B per cycle = one tile row).  Row bits 1 and 2 are XOR-ed into chunk
// bits 1 and 2 and the row's parity into chunk bit 3 (the scale-group half of the row): the LDS serves a
// 16-byte read instruction sixteen lanes per cycle (eight rows of one k-slice with eight rows of the next),
// and this keeps those sixteen chunks on sixteen different bank groups; the transposed 8-byte reads of the V
// operand (thirty-two consecutive lanes per cycle) stay conflict-free as well.
__device__ __forceinline__ unsigned int swz(unsigned int row)
{
    return ((row & 1u) << 3) | (row & 6u);
}

__device__ __forceinline__ unsigned int tile_offset(unsigned int row, unsigned int chunk)
{
    return row * kRowBytes + ((chunk ^ swz(row)) << 4);
}

__device__ __forceinline__ float soft_tanh(float x)
{
    const float x2 = x * x;
    const float poly = x * (1.0f + x2 * (-1.0f / 3.0f + x2 * (2.0f / 15.0f + x2 * (-17.0f / 315.0f))));
    const float e = __builtin_amdgcn_exp2f(fminf(fabsf(x) * (2.0f * kLog2e), 80.0f));
    const float big = copysignf(1.0f - __fdividef(2.0f, e + 1.0f), x);
    return fabsf(x) < 0.1f ? poly : big;
}

struct StepRegs {
    u32x2 codes[2];        // codes 8 cc .. + 8 and 64 + 8 cc .. + 8 of the thread's plane (K: threads 0..255, V: 256..511)
    unsigned int scales;   // two 16-bit scales (groups 0, 1) of the token
};

// Biased exponent of a (positive) scale, clamped away from the ends of the f32 range.
__device__ __forceinline__ unsigned int window_exponent(float top)
{
    return min(max((__float_as_uint(top) >> 23) & 0xffu, 2u), 252u);
}

// ---- KV splits of a chunk -------------------------------------------------------------------------------------
// A chunk with few row tiles (a short chunk over a long prefix) leaves most CUs without a workgroup while each
// workgroup walks the whole prefix.  With p.max_chunks > 1 workgroup z of a row tile attends part z of the tile's
// visible range [t_begin, t_end) -- equal 32-aligned parts of at most p.chunk_tokens, as the decode kernels cut a
// sequence -- and writes un-normalised records (sum of p v, running maximum, sum of p) that gqa_decode_merge combines;
// parts beyond the tile's own count write empty records (maximum -inf, sum 0).
struct SplitRange {
    unsigned int begin, end;
    bool live;
};
__device__ __forceinline__ SplitRange split_range(const GqaPrefillParams& p, unsigned int t_begin, unsigned int t_end)
{
    SplitRange r = {t_begin, t_end, true};
    if (p.max_chunks > 1u) {
        const unsigned int parts = min(p.max_chunks, (t_end - t_begin + p.chunk_tokens - 1u) / p.chunk_tokens);
        const unsigned int span = (((t_end - t_begin + parts - 1u) / parts) + 31u) & ~31u;
        const unsigned long long begin = (unsigned long long)t_begin + (unsigned long long)blockIdx.z * span;
        r.live = blockIdx.z < parts && begin < t_end;
        r.begin = r.live ? (unsigned int)begin : t_begin;
        r.end = r.live ? (unsigned int)min((unsigned long long)t_end, begin + span) : t_begin;
    }
    return r;
}

__device__ __forceinline__ void store_empty_record(const GqaPrefillParams& p, unsigned int row, unsigned int head)
{
    const size_t rec = ((size_t)row * p.max_chunks + blockIdx.z) * p.num_heads + head;
    p.stats[rec * 2] = kNegInf;
    p.stats[rec * 2 + 1] = 0.0f;
}

// acc and total carry 2^v_shift (the bias that keeps f16 probabilities in range, less the V window): the records are
// in true units, so that splits with different windows combine
template <int DT>
__device__ __forceinline__ void store_split_record(const GqaPrefillParams& p, unsigned int row, unsigned int head, unsigned int j, float run_max,
                                                   float total, const f32x4 (&acc)[DT], float v_shift)
{
    const size_t rec = ((size_t)row * p.max_chunks + blockIdx.z) * p.num_heads + head;
    const int down = -(int)v_shift;
    const float fa = ldexpf(1.0f, down / 2), fb = ldexpf(1.0f, down - down / 2); // two factors: 2^down alone may leave f32's range
    const bool live = total > 0.0f && total < __builtin_inff();
    if (j == 0) {
        p.stats[rec * 2] = live ? run_max : kNegInf;
        p.stats[rec * 2 + 1] = live ? total * fa * fb : 0.0f;
    }
    float* out = p.partial + rec * (size_t)(DT * 16) + 4u * j;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        *(f32x4*)(out + t * 16) = acc[t] * fa * fb;
    }
}

// POW2: pages of a power-of-two size behind a block table, known at compile time (no run-time choice of the address
// arithmetic, no division code in the loop).
// CT: 16-column MFMA tiles per wave.  Two make a workgroup of 256 (row, head-in-group) pairs, in which every K and V^T
// fragment read from LDS feeds two MFMAs; one makes it 128 pairs, for chunks whose full-size row tiles would be one round
// of very unequal workgroups (a first chunk: the last tile walks the whole chunk, the first 64 keys) -- twice as many
// workgroups, handed out longest first, even that out.
template <int SDT, bool SOFTCAP, bool POW2, int CT = 2, bool QLO = false>
__global__ __launch_bounds__(kThreads) void gqa_prefill_q8(GqaPrefillParams p)
{
    constexpr int kColTiles = CT; // inside the kernel the name means this instantiation's count
    // Four tile buffers: a pass of the main loop attends two 32-token tiles (buffers 2 s and 2 s + 1) while the next two
    // are loaded, converted and stored into the other pair, with one barrier per 64 tokens.
    // One block, the small arrays first: every address a step forms is then a register (the lane's part) plus an
    // immediate below 64 KiB (the buffer's part), which is as far as an LDS instruction's offset field reaches.
    struct Lds {
        float ks[4][2][kStep]; // [buffer][group][token]
        float vs[4][2][kStep];
        float top[4][8];       // [buffer][staging wave]: largest scale the wave converted (4..7: V)
        unsigned char k[4][kTileBytes];
        unsigned char v[4][kTileBytes];
    };
    static_assert(offsetof(Lds, v) + 4 * kTileBytes <= 65536 + 2048 + 128, "tile buffers must stay within reach of LDS offsets");
    __shared__ __align__(16) Lds lds;
    auto& lds_k = lds.k;
    auto& lds_v = lds.v;
    auto& lds_ks = lds.ks;
    auto& lds_vs = lds.vs;
    auto& lds_top = lds.top;

    const unsigned int tid = threadIdx.x;
    const unsigned int lane = tid & 63u;
    const unsigned int wave = tid >> 6;
    const unsigned int m = lane & 15u;
    const unsigned int j = lane >> 4;
    // Workgroups are handed out in the order of their linear index: the row tile is the slow index and the one with the
    // longest range comes first (with the KV head as the slow index, the long tiles of the last KV heads would start when
    // the short tiles of the first ones had finished: a first chunk of 4,096 rows took 495 us instead of 300), and the
    // KV head is the fast index, so that with eight KV heads every XCD reads the cache of one.
    const unsigned int kvh = blockIdx.x % p.num_kv_heads;
    const unsigned int rows_per_wg = max(1u, (128u * CT) / p.group);
    const unsigned int row0 = (gridDim.x / p.num_kv_heads - 1u - blockIdx.x / p.num_kv_heads) * rows_per_wg;
    const unsigned int cols_used = rows_per_wg * p.group;

    // visible token range of the workgroup: union over its rows of key_range(position + row, kv_end), or of
    // key_range_with_visible_end when rows carry an explicit visible end (src/attention/gqa.rs:65-68)
    const unsigned int last_row = min(row0 + rows_per_wg, p.rows) - 1u;
    unsigned int t_end = p.position + last_row + 1u;
    unsigned int t_begin = 0;
    if (p.visible_starts != nullptr) { // explicit ranges (src/attention/block.rs:10-16): the union of the rows' own
        t_end = 0u;
        t_begin = 0xffffffffu;
        for (unsigned int r = row0; r <= last_row; ++r) { // uniform over the workgroup: scalar loads
            const unsigned int given_end = min(p.visible_ends[r], p.position + p.rows);
            t_end = max(t_end, given_end);
            t_begin = min(t_begin, min(p.visible_starts[r], given_end));
        }
    } else if (p.visible_ends != nullptr) {
        for (unsigned int r = row0; r <= last_row; ++r) { // uniform over the workgroup: scalar loads
            t_end = max(t_end, min(p.visible_ends[r], p.position + p.rows));
        }
    }
    if (p.window != 0 && p.visible_starts == nullptr) {
        const unsigned int first_pos = p.position + row0 + 1u;
        t_begin = first_pos > p.window ? first_pos - p.window : 0u;
    }
    t_begin &= ~31u;
    const SplitRange part = split_range(p, t_begin, t_end);
    if (!part.live) {
#pragma unroll
        for (int ct = 0; ct < kColTiles; ++ct) {
            const unsigned int col = wave * (16u * kColTiles) + ct * 16u + m;
            if (col < cols_used && row0 + col / p.group < p.rows && j == 0) {
                store_empty_record(p, row0 + col / p.group, kvh * p.group + col % p.group);
            }
        }
        return;
    }
    const unsigned int steps = (part.end - part.begin + kStep - 1) / kStep;

    // ---- this wave's columns and Q fragments -------------------------------------------------
    // The wave's queries are carried as f16 after a multiplication by one power of two that puts the largest
    // magnitude of its 32 columns into [2^8, 2^9); the inverse goes into the score factor.  bf16 and f16 queries are
    // exact in that form.  An f32 query keeps 11 of its 24 bits, which moves peaked rows by up to 2e-3 of the output
    // (a score scale of 0.3 over outlier channels), so QLO carries what the rounding dropped as a second f16 fragment
    // and multiplies every K fragment by both: products stay exact, the query is good to 22 bits.
    unsigned int col_row[kColTiles], col_head[kColTiles];
    bool col_valid[kColTiles];
    Frag qf[kColTiles][4];
    Frag ql[QLO ? kColTiles : 1][QLO ? 4 : 1];
    float q_fac;
    {
        float qx[kColTiles][4][8];
        float q_amax = 0.0f;
#pragma unroll
        for (int ct = 0; ct < kColTiles; ++ct) {
            const unsigned int col = wave * (16u * kColTiles) + ct * 16u + m;
            const unsigned int r = row0 + col / p.group;
            col_row[ct] = r;
            col_head[ct] = kvh * p.group + col % p.group;
            col_valid[ct] = col < cols_used && r < p.rows;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float x = col_valid[ct] ? load_as_f32(p.q, ((size_t)r * p.num_heads + col_head[ct]) * kD + ks * 32 + j * 8 + e, p.q_dtype) : 0.0f;
                    qx[ct][ks][e] = x;
                    q_amax = fmaxf(q_amax, fabsf(x));
                }
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            q_amax = fmaxf(q_amax, __shfl_xor(q_amax, off));
        }
        const unsigned int q_exp = min(max((__float_as_uint(q_amax) >> 23) & 0xffu, 16u), 240u);
        const float q_mul = __uint_as_float((262u - q_exp) << 23); // 2^(127 + 8 - q_exp)
#pragma unroll
        for (int ct = 0; ct < kColTiles; ++ct) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float x0 = qx[ct][ks][2 * e] * q_mul, x1 = qx[ct][ks][2 * e + 1] * q_mul;
                    const unsigned int word = pack_f16_hw(x0, x1);
                    qf[ct][ks].u[e] = word;
                    if constexpr (QLO) {
                        const f16x2 hi = __builtin_bit_cast(f16x2, word);
                        ql[ct][ks].u[e] = pack_f16_hw(x0 - (float)hi[0], x1 - (float)hi[1]);
                    }
                }
            }
        }
        q_fac = ldexpf(1.0f, (int)q_exp - 135);
    }

    // scores come out in base-2 units unless the soft cap needs them in natural ones first
    const float scale_log2 = SOFTCAP ? p.score_scale : p.score_scale * kLog2e;
    const float inv_cap = SOFTCAP ? 1.0f / p.softcap : 0.0f;
    const float cap_log2 = p.softcap * kLog2e;
    const bool small_cap = p.softcap < 256.0f;
    const float tanh_arg = SOFTCAP ? q_fac * inv_cap * (2.0f * kLog2e) : 0.0f; // scaled score -> 2 y log2(e), y = score / cap
    const unsigned int k_row = p.num_kv_heads * kD;
    const unsigned int s_row = p.num_kv_heads * 4u; // two 16-bit scales per KV head
    const bool pow2 = POW2 || (p.block_tokens & (p.block_tokens - 1u)) == 0;
    const unsigned int last_token = t_end - 1u;
    // The block-table entry of a staging thread's token is fetched one step before the data that needs
    // it, so no step waits on a table -> data load chain.
    auto entry_of = [&](unsigned int token) __attribute__((always_inline)) -> unsigned int {
        token = min(token, last_token);
        const unsigned int page = pow2 ? token >> p.block_shift : token / p.block_tokens;
        return (POW2 || p.table != nullptr) ? p.table[page] : page;
    };
    auto row_from = [&](unsigned int token, unsigned int entry) __attribute__((always_inline)) -> unsigned long long {
        token = min(token, last_token);
        if (pow2) {
            return ((unsigned long long)entry << p.block_shift) + (token & (p.block_tokens - 1u));
        }
        return (unsigned long long)entry * p.block_tokens + token % p.block_tokens;
    };
    const bool stage_v = tid >= 256u;          // threads 0..255 stage K, 256..511 stage V
    const unsigned int st_token = (tid & 255u) >> 3; // staging: token of the step, 16-code chunk cc
    const unsigned int cc = tid & 7u;
    const unsigned char* st_codes = (stage_v ? p.v_plane : p.k_plane) + kvh * kD + cc * 8u;
    const unsigned char* st_scales = (stage_v ? p.v_scales : p.k_scales) + kvh * 4u;
    auto load_step = [&](StepRegs& r, unsigned int t0, unsigned int entry) __attribute__((always_inline)) {
        const unsigned long long row = row_from(t0 + st_token, entry);
        r.codes[0] = *(const u32x2*)(st_codes + row * k_row);
        r.codes[1] = *(const u32x2*)(st_codes + row * k_row + 64u);
        r.scales = *(const unsigned int*)(st_scales + row * s_row);
    };
    auto convert8 = [&](const u32x2& codes) __attribute__((always_inline)) -> u32x4 {
        unsigned int a, b, c, d;
        codes4_to_f16(codes[0], a, b);
        codes4_to_f16(codes[1], c, d);
        return u32x4{a, b, c, d};
    };
    auto store_step = [&](const StepRegs& r, int buf) __attribute__((always_inline)) {
        // chunks cc and cc + 8: sixteen lanes (two rows x eight chunks) write sixteen different bank groups
        unsigned char* tile = stage_v ? lds_v[buf] : lds_k[buf];
        *(u32x4*)(tile + tile_offset(st_token, cc)) = convert8(r.codes[0]);
        *(u32x4*)(tile + tile_offset(st_token, cc + 8u)) = convert8(r.codes[1]);
        // the eight threads of a token all hold its two scales; K scales carry the score scale (and log2 e) so that
        // the hot loop does not multiply again
        const float s0 = scale_bits_to_f32<SDT>((unsigned short)(r.scales & 0xffffu));
        const float s1 = scale_bits_to_f32<SDT>((unsigned short)(r.scales >> 16));
        if (cc == 0) {
            float* dst = stage_v ? &lds_vs[buf][0][0] : &lds_ks[buf][0][0];
            const float fold = stage_v ? 1.0f : scale_log2;
            dst[st_token] = s0 * fold;
            dst[kStep + st_token] = s1 * fold;
        }
        if (!stage_v) {
            return;
        }
        // largest V scale of the wave's eight tokens (a row of sixteen lanes holds two)
        float top = fmaxf(s0, s1);
        top = fmaxf(top, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(top), 0x128, 0xf, 0xf, false))); // row_ror:8
        const float rows01 = fmaxf(__uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 0)),
                                   __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 16)));
        const float rows23 = fmaxf(__uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 32)),
                                   __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 48)));
        if (lane == 0) {
            lds_top[buf][wave] = fmaxf(rows01, rows23);
        }
    };
    // (biased) exponent of the largest V scale of the tile in `buf`, folded into the running one
    auto window_of = [&](int buf, unsigned int wv) __attribute__((always_inline)) -> unsigned int {
        const f32x4 tops = *(const f32x4*)&lds_top[buf][4];
        const float top = fmaxf(fmaxf(tops[0], tops[1]), fmaxf(tops[2], tops[3]));
        return max(wv, (unsigned int)__builtin_amdgcn_readfirstlane(window_exponent(top)));
    };

    f32x4 acc[kColTiles][8];
#pragma unroll
    for (int ct = 0; ct < kColTiles; ++ct) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            acc[ct][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float run_max[kColTiles], run_sum[kColTiles];
    float ref_shift[kColTiles]; // what is added to a scaled score before exp2: bias - V window - running maximum
    unsigned int vis_lo[kColTiles], vis_hi[kColTiles]; // visible tokens [lo, hi) of each column's row
#pragma unroll
    for (int ct = 0; ct < kColTiles; ++ct) {
        run_max[ct] = kNegInf;
        run_sum[ct] = 0.0f;
        ref_shift[ct] = kPBias;
        const unsigned int pos = p.position + col_row[ct];
        unsigned int hi = pos + 1u;
        unsigned int lo = (p.window != 0 && pos + 1u > p.window) ? pos + 1u - p.window : 0u;
        if (p.visible_starts != nullptr && col_valid[ct]) { // the row's range as given
            hi = min(p.visible_ends[col_row[ct]], p.position + p.rows);
            lo = min(p.visible_starts[col_row[ct]], hi);
        } else if (p.visible_ends != nullptr && col_valid[ct]) { // a row may read past itself, up to the end of the chunk
            hi = min(max(hi, p.visible_ends[col_row[ct]]), p.position + p.rows);
        }
        vis_hi[ct] = col_valid[ct] ? hi : 0u;
        vis_lo[ct] = lo;
    }

    // first token some column of the wave cannot see any more / last token some column does not see yet (wave-uniform)
    unsigned int wave_min_hi = vis_hi[0], wave_max_lo = vis_lo[0];
#pragma unroll
    for (int ct = 1; ct < kColTiles; ++ct) {
        wave_min_hi = min(wave_min_hi, vis_hi[ct]);
        wave_max_lo = max(wave_max_lo, vis_lo[ct]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        wave_min_hi = min(wave_min_hi, (unsigned int)__shfl_xor((int)wave_min_hi, off));
        wave_max_lo = max(wave_max_lo, (unsigned int)__shfl_xor((int)wave_max_lo, off));
    }
    wave_min_hi = __builtin_amdgcn_readfirstlane(wave_min_hi);
    wave_max_lo = __builtin_amdgcn_readfirstlane(wave_max_lo);

    // chunk = g * 8 + half * 4 + j: the low three bits meet row bits 1, 2; the group bit meets the row's parity
    // The byte offsets inside a tile are kept as finished sums, one register per (group, half) or (group, quarter):
    // formed from their parts inside the loop they cost an addition per LDS read.  The inline assembly hides the
    // parts from the optimizer, which would otherwise split the sums again to save the registers.
    unsigned int qk_at[2][2], pv_at[2][4];
    const unsigned int tr_row = 4u * j + (m >> 2);
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        const unsigned int qk_group = g == 0 ? (m & 1u) * 128u : 128u - (m & 1u) * 128u;
        const unsigned int pv_group = g == 0 ? (tr_row & 1u) * 128u : 128u - (tr_row & 1u) * 128u;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            qk_at[g][h] = m * kRowBytes + ((((unsigned int)h << 2 | j) ^ (m & 6u)) << 4) + qk_group;
            asm volatile("" : "+v"(qk_at[g][h]));
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            pv_at[g][q] = tr_row * kRowBytes + ((((unsigned int)q << 1 | ((m & 3u) >> 1)) ^ (tr_row & 6u)) << 4) + (m & 1u) * 8u + pv_group;
            asm volatile("" : "+v"(pv_at[g][q]));
        }
    }

    // `v_shift` = 8 - (V window exponent) is added to every score before exp2; `acc_fix` is 2^-(growth of that
    // window since the last step): 1 unless `window_moved`.
    auto compute_step = [&](int buf, unsigned int t0, float v_shift, float acc_fix, bool window_moved) __attribute__((always_inline)) {
        const unsigned char* kt = lds_k[buf];
        // ---- S^T = sum_g k_scale_g * (Kcodes_g . Q'_g) ------------------------------------------
        f32x4 s[2][kColTiles];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int ct = 0; ct < kColTiles; ++ct) {
                s[i][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                Frag k0, k1;
                k0.u = *(const u32x4*)(kt + qk_at[g][0] + i * 16 * kRowBytes);
                k1.u = *(const u32x4*)(kt + qk_at[g][1] + i * 16 * kRowBytes);
                const f32x4 gs = *(const f32x4*)(&lds_ks[buf][g][i * 16 + 4 * j]);
#pragma unroll
                for (int ct = 0; ct < kColTiles; ++ct) {
                    f32x4 d = {0.f, 0.f, 0.f, 0.f};
                    if constexpr (QLO) {
                        d = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0.h, ql[ct][2 * g].h, d, 0, 0, 0);
                        d = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1.h, ql[ct][2 * g + 1].h, d, 0, 0, 0);
                    }
                    d = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0.h, qf[ct][2 * g].h, d, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1.h, qf[ct][2 * g + 1].h, d, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        s[i][ct][r] = fmaf(d[r], gs[r], s[i][ct][r]);
                    }
                }
            }
        }
        // The P.V operands that do not depend on the softmax are requested now, so that their LDS round trips pass under
        // its vector-ALU work: the V^T fragments of scale group 0 and the V scales of both groups.
        const unsigned char* vt = lds_v[buf];
        union VFrag {
            s16x4 s[2];
            f16x8 h;
        };
        auto load_vfrags = [&](VFrag (&vf)[4], int g) __attribute__((always_inline)) {
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) {
                const unsigned char* at = vt + pv_at[g][tt];
                vf[tt].s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(at));
                vf[tt].s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(at + 16 * kRowBytes));
            }
        };
        VFrag vf[2][4];
        f32x4 gsv[2][2];
        load_vfrags(vf[0], 0);
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            gsv[g][0] = *(const f32x4*)(&lds_vs[buf][g][4 * j]);
            gsv[g][1] = *(const f32x4*)(&lds_vs[buf][g][16 + 4 * j]);
        }
        PREFILL_PHASE_FENCE();
        // ---- online softmax per column --------------------------------------------------------------
        float pr[kColTiles][8];
        bool heavy = false; // some probability of this step is not small against the sum so far
#pragma unroll
        for (int ct = 0; ct < kColTiles; ++ct) {
            float sc[8];
            // only steps that touch a causal or window edge of some column of the wave need the per-token masks
            const bool edge = t0 + kStep > wave_min_hi || t0 < wave_max_lo;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float x = s[e >> 2][ct][e & 3];
                if constexpr (SOFTCAP) {
                    // caps that models use take the five-instruction form (see gqa_prefill_f16), larger ones the precise one
                    x = small_cap ? cap_log2 * fmaf(-2.0f, __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(x * tanh_arg) + 1.0f), 1.0f)
                                  : cap_log2 * soft_tanh(x * q_fac * inv_cap);
                }
                sc[e] = x;
            }
            if (edge) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const unsigned int token = t0 + 16u * (e >> 2) + 4u * j + (e & 3);
                    sc[e] = (token >= vis_lo[ct] && token < vis_hi[ct]) ? sc[e] : kNegInf;
                }
            }
            // the query's power of two is positive, so maxima are taken first and it rides in the multiply-add
            const float mult = SOFTCAP ? 1.0f : q_fac;
            float lane_max = sc[0]; // a chain, so that two comparisons share one instruction
#pragma unroll
            for (int e = 1; e < 8; ++e) {
                lane_max = fmaxf(lane_max, sc[e]);
            }
            // The reference point of the column (running maximum, V window) moves on few steps of a long prefix, so the
            // reduction across the wave's rows and the rescaling sit behind a test of the lane's own maximum.
            if (__any(lane_max * mult > run_max[ct]) || window_moved) {
                const float step_max = wave_max_16x4(lane_max) * mult;
                const float new_max = fmaxf(run_max[ct], step_max);
                const float safe_max = new_max == kNegInf ? 0.0f : new_max;
                const float alpha = __builtin_amdgcn_exp2f(run_max[ct] - safe_max) * acc_fix;
                ref_shift[ct] = v_shift - safe_max;
                run_sum[ct] *= alpha;
                run_max[ct] = new_max;
                if (__any(alpha != 1.0f)) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        acc[ct][t] *= alpha;
                    }
                }
            }
            const float shift = ref_shift[ct];
            float step_sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                pr[ct][e] = __builtin_amdgcn_exp2f(fmaf(sc[e], mult, shift));
                step_sum += pr[ct][e];
            }
            run_sum[ct] += step_sum;
            // the lane's eight probabilities together bound its largest one
            heavy = heavy || step_sum * kLoThreshold > run_sum[ct];
        }
        // ---- O^T += Vcodes^T . P'_g ----------------------------------------------------------------------
        // P' is carried as f16 hi + lo (22 significant bits) while the probabilities a lane holds of this step weigh more
        // than 1/8 of its running sum (a lane sums a quarter of the tokens, so each is < 1/32 of the row's sum);
        // below that the hi term's rounding (2^-12 relative, random sign) moves the normalised output by
        // < 2^-12 / 32 of |v|, so the lo product is skipped.
        const bool lo_pass = __any(heavy);
        PREFILL_PHASE_FENCE();
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const f32x4 gs0 = gsv[g][0];
            const f32x4 gs1 = gsv[g][1];
            Frag phi[kColTiles], plo[kColTiles];
#pragma unroll
            for (int ct = 0; ct < kColTiles; ++ct) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float x0 = pr[ct][2 * e] * (e < 2 ? gs0[2 * e] : gs1[2 * e - 4]);
                    const float x1 = pr[ct][2 * e + 1] * (e < 2 ? gs0[2 * e + 1] : gs1[2 * e - 3]);
                    phi[ct].u[e] = pack_f16_hw(x0, x1);
                }
            }
            if (g == 0) { // group 1's fragments travel while group 0 multiplies
                load_vfrags(vf[1], 1);
            }
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
                for (int ct = 0; ct < kColTiles; ++ct) {
                    acc[ct][g * 4 + tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[g][tt].h, phi[ct].h, acc[ct][g * 4 + tt], 0, 0, 0);
                }
            }
            if (lo_pass) { // rare: one branch around the low-order products
#pragma unroll
                for (int ct = 0; ct < kColTiles; ++ct) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float x0 = pr[ct][2 * e] * (e < 2 ? gs0[2 * e] : gs1[2 * e - 4]);
                        const float x1 = pr[ct][2 * e + 1] * (e < 2 ? gs0[2 * e + 1] : gs1[2 * e - 3]);
                        // formed again rather than read back from phi: a bit cast of a vector element (phi[ct].u[e]) picked
                        // element 0 for every e with this compiler
                        const f16x2 hi = __builtin_bit_cast(f16x2, pack_f16_hw(x0, x1));
                        plo[ct].u[e] = pack_f16_hw(x0 - (float)hi[0], x1 - (float)hi[1]);
                    }
                }
#pragma unroll
                for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
                    for (int ct = 0; ct < kColTiles; ++ct) {
                        acc[ct][g * 4 + tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[g][tt].h, plo[ct].h, acc[ct][g * 4 + tt], 0, 0, 0);
                    }
                }
            }
        }
    };

    // ---- main loop ------------------------------------------------------------------------------------------
    StepRegs regs;
    load_step(regs, part.begin, entry_of(part.begin + st_token));
    unsigned int entry_next = entry_of(part.begin + kStep + st_token);
    store_step(regs, 0);
    load_step(regs, part.begin + kStep, entry_next); // past the range: its last row again
    entry_next = entry_of(part.begin + 2u * kStep + st_token);
    store_step(regs, 1);
    __syncthreads();
    unsigned int wv = 2u; // (biased) exponent of the largest V scale up to the tile being attended
    float v_shift = kPBias + 125.0f;
    // `buf` is a literal at every call, so the LDS addresses of a step differ from the other buffers' only in the
    // instructions' immediate offsets and cost no address arithmetic
    auto attend_tile = [&](unsigned int t0, int buf) __attribute__((always_inline)) {
        const unsigned int wv_now = window_of(buf, wv);
        const bool window_moved = wv_now != wv; // rare: a V scale above everything met so far
        float acc_fix = 1.0f;
        if (window_moved) {
            acc_fix = ldexpf(1.0f, (int)wv - (int)wv_now);
            wv = wv_now;
            v_shift = kPBias + (float)(127 - (int)wv);
        }
        compute_step(buf, t0, v_shift, acc_fix, window_moved);
    };
    // Tiles `step` and `step + 1` are in the buffers of `set`; the two after them travel, one at a time through the same
    // registers, into the other pair, which nobody reads before the barrier.
    auto two_steps = [&](unsigned int step, int set) __attribute__((always_inline)) {
        const unsigned int t0 = part.begin + step * kStep;
        // rows past the end of the visible range repeat its last one: the loads stay inside the sequence's pages
        load_step(regs, t0 + 2u * kStep, entry_next);
        entry_next = entry_of(t0 + 3u * kStep + st_token);
        attend_tile(t0, 2 * set);
        store_step(regs, 2 * (set ^ 1));
        PREFILL_PHASE_FENCE(); // the two tiles are attended one after the other: interleaved, their operands do not fit the registers
        load_step(regs, t0 + 3u * kStep, entry_next);
        entry_next = entry_of(t0 + 4u * kStep + st_token);
        attend_tile(t0 + kStep, 2 * set + 1);
        store_step(regs, 2 * (set ^ 1) + 1);
        __syncthreads();
    };
    unsigned int step = 0;
    for (; step + 4 <= steps; step += 4) {
        two_steps(step, 0);
        two_steps(step + 2u, 1);
    }
    if (step + 2 <= steps) {
        two_steps(step, 0);
        step += 2;
        if (step < steps) { // the odd tile at the end sits in the first buffer of the other pair
            attend_tile(part.begin + step * kStep, 2);
        }
    } else if (step < steps) {
        attend_tile(part.begin + step * kStep, 0);
    }

    // ---- normalise and store ------------------------------------------------------------------------
#pragma unroll
    for (int ct = 0; ct < kColTiles; ++ct) {
        const float total = wave_sum_16x4(run_sum[ct]);
        {
            // recomputed rather than kept: these would sit in registers through the whole main loop
            const unsigned int col = wave * (16u * kColTiles) + ct * 16u + m;
            col_row[ct] = row0 + col / p.group;
            col_head[ct] = kvh * p.group + col % p.group;
            col_valid[ct] = col < cols_used && col_row[ct] < p.rows;
        }
        if (!col_valid[ct]) {
            continue;
        }
        if (p.max_chunks > 1u) {
            store_split_record<8>(p, col_row[ct], col_head[ct], j, run_max[ct], total, acc[ct], v_shift);
            continue;
        }
        // accumulators and sum carry the same power of two (2^8 and the V window), which cancels here
        const float inv = (total > 0.0f && total < __builtin_inff()) ? 1.0f / total : 0.0f;
        const size_t base = ((size_t)col_row[ct] * p.num_heads + col_head[ct]) * kD;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            f32x4 v = acc[ct][t] * inv;
            if (inv == 0.0f) {
                v = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            const size_t at = base + t * 16 + 4 * j;
            if (p.gate != nullptr) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = gated(v[e], p.gate, p.gate_cols, p.gate_dtype, col_row[ct], col_head[ct] * kD + t * 16 + 4 * j + e);
                }
            }
            if (p.out_dtype == 0) {
                *(f32x4*)((float*)p.out + at) = v;
            } else {
                unsigned short* o = (unsigned short*)p.out + at;
                u32x2 packed;
                if (p.out_dtype == 1) {
                    packed = u32x2{pack_bf16_rne(v[0], v[1]), pack_bf16_rne(v[2], v[3])};
                } else {
                    packed = u32x2{(unsigned int)f32_to_f16_bits(v[0]) | ((unsigned int)f32_to_f16_bits(v[1]) << 16),
                                   (unsigned int)f32_to_f16_bits(v[2]) | ((unsigned int)f32_to_f16_bits(v[3]) << 16)};
                }
                *(u32x2*)o = packed;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// The other tile shapes: f16 caches at head_dim 128 / 256, Q8g64 caches at head_dim 64 / 256
// ---------------------------------------------------------------------------------------------
// The same workgroup as gqa_prefill_q8 over a tile layout that does not depend on the row length: chunk c of row r
// sits at r * row_bytes + ((c ^ swz(r)) << 4) with the swizzle cut to the row's chunk bits: it touches chunk bits 1..3,
// so rows of 16 and 32 chunks (one or two whole lines of the 64 banks) take all of it and rows of 8 chunks (half a
// line: the row's parity already picks the half) take bits 1 and 2.
//   f16 rows (src/kv_cache/mod.rs:179-331) are copied as stored: S^T = K . Q' is one accumulator, P = p * 2^8 as
//       f16 hi (+ lo while the step is heavy), no scales and no window.
//   Q8g64 rows are converted as in gqa_prefill_q8 (exact f16 integers, K scales pre-multiplied by the score scale,
//       one accumulator per 64-column group, P'_g = p * v_scale_g, the exponent of the largest V scale carried by
//       the softmax reference).
// head_dim 64 and 128 keep two 16-column tiles per wave (256 columns per workgroup); head_dim 256 keeps one (128
// columns): its accumulators and query fragments fill the registers that the second tile has at 128.
template <int D> struct TileShape {
    static constexpr int kRow = D * 2;            // bytes of one token of one KV head as f16
    static constexpr int kTile = kStep * kRow;    // one 32-token tile
    static constexpr int kChunks = D / 8;         // 16-byte chunks per row
    static constexpr int kCT = D == 256 ? 1 : 2;  // 16-column MFMA tiles per wave
    static constexpr int kCols = 8 * 16 * kCT;    // (row, head-in-group) pairs per workgroup
    static constexpr int kKS = D / 32;            // k-steps of the score product
    static constexpr int kDT = D / 16;            // 16-dim tiles of the output
    static constexpr int kLoads = kChunks / 8;    // staging loads per thread and step (16 bytes of f16, or 8 codes)
    static constexpr int kG = D / 64;             // Q8g64 scale groups per row
    __device__ static __forceinline__ unsigned int swizzle(unsigned int row) { return swz(row) & (unsigned int)(kChunks - 1); }
};

// KV: 0 = Q8g64 (SDT names the scale type: bf16, f16 or f32), 1 = f16 rows
template <int D, int KV, int SDT, bool SOFTCAP, bool POW2>
__global__ __launch_bounds__(512) void gqa_prefill_tiles(GqaPrefillParams p)
{
    using C = TileShape<D>;
    constexpr int CT = C::kCT;
    constexpr int G = C::kG;
    constexpr bool Q8 = KV == 0;
    static_assert(C::kLoads >= 1, "a staging thread owns at least one chunk");
    // Four tile buffers, as in gqa_prefill_q8: a pass attends two tiles while the next two go into the other pair, one
    // barrier per 64 tokens.  The small arrays come first so that as many buffer addresses as possible are a lane
    // register plus an immediate inside the LDS offset field.
    struct Lds {
        float ks[Q8 ? 4 : 1][Q8 ? G : 1][kStep]; // [buffer][group][token], Q8g64 only
        float vs[Q8 ? 4 : 1][Q8 ? G : 1][kStep];
        float top[4][8];                         // [buffer][staging wave]: largest scale it converted
        unsigned char k[4][C::kTile];
        unsigned char v[4][C::kTile];
    };
    __shared__ __align__(16) Lds lds;
    auto& lds_k = lds.k;
    auto& lds_v = lds.v;
    auto& lds_ks = lds.ks;
    auto& lds_vs = lds.vs;
    auto& lds_top = lds.top;

    const unsigned int tid = threadIdx.x;
    const unsigned int lane = tid & 63u;
    const unsigned int wave = tid >> 6;
    const unsigned int m = lane & 15u;
    const unsigned int j = lane >> 4;
    // Workgroups are handed out in the order of their linear index: the row tile is the slow index and the one with the
    // longest range comes first (with the KV head as the slow index, the long tiles of the last KV heads would start when
    // the short tiles of the first ones had finished: a first chunk of 4,096 rows took 495 us instead of 300), and the
    // KV head is the fast index, so that with eight KV heads every XCD reads the cache of one.
    const unsigned int kvh = blockIdx.x % p.num_kv_heads;
    const unsigned int rows_per_wg = max(1u, (unsigned int)C::kCols / p.group);
    const unsigned int row0 = (gridDim.x / p.num_kv_heads - 1u - blockIdx.x / p.num_kv_heads) * rows_per_wg;
    const unsigned int cols_used = rows_per_wg * p.group;

    // visible token range of the workgroup, as in gqa_prefill_q8
    const unsigned int last_row = min(row0 + rows_per_wg, p.rows) - 1u;
    unsigned int t_end = p.position + last_row + 1u;
    unsigned int t_begin = 0;
    if (p.visible_starts != nullptr) { // explicit ranges (src/attention/block.rs:10-16): the union of the rows' own
        t_end = 0u;
        t_begin = 0xffffffffu;
        for (unsigned int r = row0; r <= last_row; ++r) {
            const unsigned int given_end = min(p.visible_ends[r], p.position + p.rows);
            t_end = max(t_end, given_end);
            t_begin = min(t_begin, min(p.visible_starts[r], given_end));
        }
    } else if (p.visible_ends != nullptr) {
        for (unsigned int r = row0; r <= last_row; ++r) {
            t_end = max(t_end, min(p.visible_ends[r], p.position + p.rows));
        }
    }
    if (p.window != 0 && p.visible_starts == nullptr) {
        const unsigned int first_pos = p.position + row0 + 1u;
        t_begin = first_pos > p.window ? first_pos - p.window : 0u;
    }
    t_begin &= ~31u;
    const SplitRange part = split_range(p, t_begin, t_end);
    if (!part.live) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const unsigned int col = wave * (16u * CT) + ct * 16u + m;
            if (col < cols_used && row0 + col / p.group < p.rows && j == 0) {
                store_empty_record(p, row0 + col / p.group, kvh * p.group + col % p.group);
            }
        }
        return;
    }
    const unsigned int steps = (part.end - part.begin + kStep - 1) / kStep;

    // ---- this wave's columns and Q fragments (power-of-two normalised f16, as in gqa_prefill_q8) ----
    unsigned int col_row[CT], col_head[CT];
    bool col_valid[CT];
    Frag qf[CT][C::kKS];
    float q_fac;
    {
        float q_amax = 0.0f;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const unsigned int col = wave * (16u * CT) + ct * 16u + m;
            const unsigned int r = row0 + col / p.group;
            col_row[ct] = r;
            col_head[ct] = kvh * p.group + col % p.group;
            col_valid[ct] = col < cols_used && r < p.rows;
        }
        // two passes over the query (maximum, then conversion): keeping all of it in f32 would not fit the registers
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
            for (int ks = 0; ks < C::kKS; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float x = col_valid[ct] ? load_as_f32(p.q, ((size_t)col_row[ct] * p.num_heads + col_head[ct]) * D + ks * 32 + j * 8 + e, p.q_dtype) : 0.0f;
                    q_amax = fmaxf(q_amax, fabsf(x));
                }
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            q_amax = fmaxf(q_amax, __shfl_xor(q_amax, off));
        }
        const unsigned int q_exp = min(max((__float_as_uint(q_amax) >> 23) & 0xffu, 16u), 240u);
        const float q_mul = __uint_as_float((262u - q_exp) << 23); // 2^(127 + 8 - q_exp)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
            for (int ks = 0; ks < C::kKS; ++ks) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const size_t at = ((size_t)col_row[ct] * p.num_heads + col_head[ct]) * D + ks * 32 + j * 8 + 2 * e;
                    const float x0 = col_valid[ct] ? load_as_f32(p.q, at, p.q_dtype) : 0.0f;
                    const float x1 = col_valid[ct] ? load_as_f32(p.q, at + 1, p.q_dtype) : 0.0f;
                    qf[ct][ks].u[e] = pack_f16_hw(x0 * q_mul, x1 * q_mul);
                }
            }
        }
        q_fac = ldexpf(1.0f, (int)q_exp - 135);
    }

    // What turns the accumulated product into a score in base-2 units (or, under a soft cap, into natural units first).
    // Q8g64 tiles carry the score scale in their K scales, f16 tiles do not.
    const float scale_log2 = SOFTCAP ? p.score_scale : p.score_scale * kLog2e;
    const float score_mult = Q8 ? q_fac : scale_log2 * q_fac;
    const float cap_log2 = p.softcap * kLog2e;
    const float inv_cap = SOFTCAP ? 1.0f / p.softcap : 0.0f;
    const float tanh_arg = SOFTCAP ? score_mult * (2.0f * kLog2e) / p.softcap : 0.0f; // product -> 2 y log2(e), y = score / cap
    const bool small_cap = p.softcap < 256.0f;
    const unsigned int k_row = p.num_kv_heads * (Q8 ? (unsigned int)D : (unsigned int)C::kRow); // bytes of one cache row
    constexpr unsigned int kScaleBytes = SDT == 2 ? 4u : 2u;
    const unsigned int s_row = p.num_kv_heads * G * kScaleBytes;                                // bytes of one scale row
    const bool pow2 = POW2 || (p.block_tokens & (p.block_tokens - 1u)) == 0;
    const unsigned int last_token = t_end - 1u;
    auto entry_of = [&](unsigned int token) __attribute__((always_inline)) -> unsigned int {
        token = min(token, last_token);
        const unsigned int page = pow2 ? token >> p.block_shift : token / p.block_tokens;
        return (POW2 || p.table != nullptr) ? p.table[page] : page;
    };
    auto row_from = [&](unsigned int token, unsigned int entry) __attribute__((always_inline)) -> unsigned long long {
        token = min(token, last_token);
        if (pow2) {
            return ((unsigned long long)entry << p.block_shift) + (token & (p.block_tokens - 1u));
        }
        return (unsigned long long)entry * p.block_tokens + token % p.block_tokens;
    };
    // staging: threads 0..255 take K, 256..511 take V; a thread owns token (tid % 256) / 8 and the chunks cc, cc + 8, ...
    const bool stage_v = tid >= 256u;
    const unsigned int st_token = (tid & 255u) >> 3;
    const unsigned int cc = tid & 7u;
    const unsigned char* st_plane = (stage_v ? p.v_plane : p.k_plane) + (size_t)kvh * (Q8 ? D : C::kRow) + cc * (Q8 ? 8u : 16u);
    const unsigned char* st_scales = Q8 ? (stage_v ? p.v_scales : p.k_scales) + (size_t)kvh * G * kScaleBytes : nullptr;
    struct StageRegs {
        u32x4 chunk[C::kLoads]; // f16 rows: the chunk as stored; Q8g64: eight codes in the first two words
        u32x4 scales;           // Q8g64: the token's G scales (16-bit ones packed two to a word, f32 ones a word each)
    };
    auto load_step = [&](StageRegs& r, unsigned int t0, unsigned int entry) __attribute__((always_inline)) {
        const unsigned long long row = row_from(t0 + st_token, entry);
        const unsigned char* at = st_plane + row * k_row;
#pragma unroll
        for (int u = 0; u < C::kLoads; ++u) {
            if constexpr (Q8) {
                const u32x2 codes = *(const u32x2*)(at + u * 64);
                r.chunk[u] = u32x4{codes[0], codes[1], 0u, 0u};
            } else {
                r.chunk[u] = *(const u32x4*)(at + u * 128);
            }
        }
        if constexpr (Q8) {
            const unsigned char* sp = st_scales + row * s_row; // the scale planes are only known to be 4-byte aligned
            r.scales = u32x4{0u, 0u, 0u, 0u};
            if constexpr (G * kScaleBytes == 2u) {
                r.scales[0] = *(const unsigned short*)sp;
            } else {
#pragma unroll
                for (unsigned int w = 0; w < G * kScaleBytes / 4u; ++w) {
                    r.scales[w] = ((const unsigned int*)sp)[w];
                }
            }
        }
    };
    auto store_step = [&](const StageRegs& r, int buf) __attribute__((always_inline)) {
        unsigned char* tile = stage_v ? lds_v[buf] : lds_k[buf];
#pragma unroll
        for (int u = 0; u < C::kLoads; ++u) {
            u32x4 out = r.chunk[u];
            if constexpr (Q8) {
                unsigned int a, b, c, d;
                codes4_to_f16(r.chunk[u][0], a, b);
                codes4_to_f16(r.chunk[u][1], c, d);
                out = u32x4{a, b, c, d};
            }
            *(u32x4*)(tile + st_token * C::kRow + (((cc + 8u * u) ^ C::swizzle(st_token)) << 4)) = out;
        }
        if constexpr (Q8) {
            // the eight threads of a token all hold its scales; K scales carry the score scale (and log2 e)
            float top = 0.0f;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float sg;
                if constexpr (SDT == 2) {
                    sg = __uint_as_float(r.scales[g]);
                } else {
                    sg = scale_bits_to_f32<SDT>((unsigned short)((r.scales[g >> 1] >> (16 * (g & 1))) & 0xffffu));
                }
                top = fmaxf(top, sg);
                if (cc == 0) {
                    (stage_v ? lds_vs : lds_ks)[buf][g][st_token] = stage_v ? sg : sg * scale_log2;
                }
            }
            if (stage_v) { // largest V scale of the wave's eight tokens (a row of sixteen lanes holds two)
                top = fmaxf(top, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(top), 0x128, 0xf, 0xf, false))); // row_ror:8
                const float rows01 = fmaxf(__uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 0)),
                                           __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 16)));
                const float rows23 = fmaxf(__uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 32)),
                                           __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(top), 48)));
                if (lane == 0) {
                    lds_top[buf][wave] = fmaxf(rows01, rows23);
                }
            }
        }
    };
    // (biased) exponent of the largest V scale of the tile in `buf`, folded into the running one (Q8g64 only)
    auto window_of = [&](int buf, unsigned int wv) __attribute__((always_inline)) -> unsigned int {
        const f32x4 tops = *(const f32x4*)&lds_top[buf][4];
        const float top = fmaxf(fmaxf(tops[0], tops[1]), fmaxf(tops[2], tops[3]));
        return max(wv, (unsigned int)__builtin_amdgcn_readfirstlane(window_exponent(top)));
    };

    f32x4 acc[CT][C::kDT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
        for (int t = 0; t < C::kDT; ++t) {
            acc[ct][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float run_max[CT], run_sum[CT], ref_shift[CT];
    unsigned int vis_lo[CT], vis_hi[CT];
    unsigned int wave_min_hi = 0xffffffffu, wave_max_lo = 0u;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        run_max[ct] = kNegInf;
        run_sum[ct] = 0.0f;
        ref_shift[ct] = kPBias;
        const unsigned int pos = p.position + col_row[ct];
        unsigned int hi = pos + 1u;
        unsigned int lo = (p.window != 0 && pos + 1u > p.window) ? pos + 1u - p.window : 0u;
        if (p.visible_starts != nullptr && col_valid[ct]) { // the row's range as given
            hi = min(p.visible_ends[col_row[ct]], p.position + p.rows);
            lo = min(p.visible_starts[col_row[ct]], hi);
        } else if (p.visible_ends != nullptr && col_valid[ct]) { // a row may read past itself, up to the end of the chunk
            hi = min(max(hi, p.visible_ends[col_row[ct]]), p.position + p.rows);
        }
        vis_hi[ct] = col_valid[ct] ? hi : 0u;
        vis_lo[ct] = lo;
        wave_min_hi = min(wave_min_hi, vis_hi[ct]);
        wave_max_lo = max(wave_max_lo, vis_lo[ct]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        wave_min_hi = min(wave_min_hi, (unsigned int)__shfl_xor((int)wave_min_hi, off));
        wave_max_lo = max(wave_max_lo, (unsigned int)__shfl_xor((int)wave_max_lo, off));
    }
    wave_min_hi = __builtin_amdgcn_readfirstlane(wave_min_hi);
    wave_max_lo = __builtin_amdgcn_readfirstlane(wave_max_lo);

    // LDS byte offsets of the lane's fragments as finished sums.  K: chunk 4 ks + j of row m; the swizzle permutes
    // ks inside a group of four, so four registers serve every k-step (ks / 4 selects 256 bytes further, an immediate).
    // V: chunk 2 tt + (m & 3) / 2 of row tr_row, 8 bytes in; the swizzle permutes tt inside a group of eight.
    constexpr int kQkRegs = C::kKS < 4 ? C::kKS : 4, kPvRegs = C::kDT < 8 ? C::kDT : 8;
    unsigned int qk_at[kQkRegs], pv_at[kPvRegs];
    const unsigned int tr_row = 4u * j + (m >> 2);
#pragma unroll
    for (int k4 = 0; k4 < kQkRegs; ++k4) {
        qk_at[k4] = m * C::kRow + ((((unsigned int)k4 << 2 | j) ^ C::swizzle(m)) << 4);
        asm volatile("" : "+v"(qk_at[k4]));
    }
#pragma unroll
    for (int t8 = 0; t8 < kPvRegs; ++t8) {
        pv_at[t8] = tr_row * C::kRow + ((((unsigned int)t8 << 1 | ((m & 3u) >> 1)) ^ C::swizzle(tr_row)) << 4) + (m & 1u) * 8u;
        asm volatile("" : "+v"(pv_at[t8]));
    }

    // `v_shift` = 8 - (V window exponent) goes into the softmax reference, `acc_fix` is 2^-(growth of that window since
    // the last step): 8 and 1 for f16 rows, which have no scales
    auto compute_step = [&](int buf, unsigned int t0, float v_shift, float acc_fix, bool window_moved) __attribute__((always_inline)) {
        const unsigned char* kt = lds_k[buf];
        const unsigned char* vt = lds_v[buf];
        const int sbuf = Q8 ? buf : 0;
        // ---- S^T = K . Q' (one accumulator per scale group for Q8g64 tiles) ------------------------------
        f32x4 s[2][CT];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                s[i][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            if constexpr (Q8) {
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    Frag k0, k1;
                    k0.u = *(const u32x4*)(kt + qk_at[(2 * g) & 3] + ((2 * g) >> 2) * 256 + i * 16 * C::kRow);
                    k1.u = *(const u32x4*)(kt + qk_at[(2 * g + 1) & 3] + ((2 * g + 1) >> 2) * 256 + i * 16 * C::kRow);
                    const f32x4 gs = *(const f32x4*)(&lds_ks[sbuf][g][i * 16 + 4 * j]);
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        f32x4 d = {0.f, 0.f, 0.f, 0.f};
                        d = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0.h, qf[ct][2 * g].h, d, 0, 0, 0);
                        d = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1.h, qf[ct][2 * g + 1].h, d, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            s[i][ct][r] = fmaf(d[r], gs[r], s[i][ct][r]);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int ks = 0; ks < C::kKS; ++ks) {
                    Frag kf;
                    kf.u = *(const u32x4*)(kt + qk_at[ks & 3] + (ks >> 2) * 256 + i * 16 * C::kRow);
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        s[i][ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf.h, qf[ct][ks].h, s[i][ct], 0, 0, 0);
                    }
                }
            }
        }
        union VFrag {
            s16x4 s[2];
            f16x8 h;
        };
        auto load_vfrag = [&](VFrag& vf, int tt) __attribute__((always_inline)) {
            const unsigned char* at = vt + pv_at[tt & 7] + (tt >> 3) * 256;
            vf.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(at));
            vf.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(at + 16 * C::kRow));
        };
        // the first V^T fragments travel under the softmax
        VFrag vf[2][4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            load_vfrag(vf[0][tt], tt);
        }
        PREFILL_PHASE_FENCE();
        // ---- online softmax per column ----------------------------------------------------------------
        float pr[CT][8];
        bool heavy = false;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            float sc[8];
            const bool edge = t0 + kStep > wave_min_hi || t0 < wave_max_lo;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float x = s[e >> 2][ct][e & 3];
                if constexpr (SOFTCAP) {
                    // tanh(y) = 1 - 2 / (e^(2y) + 1) for the caps models use: the form cancels for tiny y, and its absolute error,
                    // a few units of 2^-24, is multiplied by the cap (3e-6 of a score under a cap of 50); larger caps take the
                    // polynomial-or-exponential form, which keeps the limit of an ever larger cap.  The cap rides in `mult`.
                    if (small_cap) {
                        const float e2y = __builtin_amdgcn_exp2f(x * tanh_arg);
                        x = fmaf(-2.0f, __builtin_amdgcn_rcpf(e2y + 1.0f), 1.0f);
                    } else {
                        x = soft_tanh(x * score_mult * inv_cap);
                    }
                }
                sc[e] = x;
            }
            if (edge) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const unsigned int token = t0 + 16u * (e >> 2) + 4u * j + (e & 3);
                    sc[e] = (token >= vis_lo[ct] && token < vis_hi[ct]) ? sc[e] : kNegInf;
                }
            }
            const float mult = SOFTCAP ? cap_log2 : score_mult; // positive: maxima first, the factor rides in the multiply-add
            float lane_max = sc[0];
#pragma unroll
            for (int e = 1; e < 8; ++e) {
                lane_max = fmaxf(lane_max, sc[e]);
            }
            if (__any(lane_max * mult > run_max[ct]) || window_moved) {
                const float step_max = wave_max_16x4(lane_max) * mult;
                const float new_max = fmaxf(run_max[ct], step_max);
                const float safe_max = new_max == kNegInf ? 0.0f : new_max;
                const float alpha = __builtin_amdgcn_exp2f(run_max[ct] - safe_max) * acc_fix;
                ref_shift[ct] = v_shift - safe_max;
                run_sum[ct] *= alpha;
                run_max[ct] = new_max;
                if (__any(alpha != 1.0f)) {
#pragma unroll
                    for (int t = 0; t < C::kDT; ++t) {
                        acc[ct][t] *= alpha;
                    }
                }
            }
            const float shift = ref_shift[ct];
            float step_sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                pr[ct][e] = __builtin_amdgcn_exp2f(fmaf(sc[e], mult, shift));
                step_sum += pr[ct][e];
            }
            run_sum[ct] += step_sum;
            heavy = heavy || step_sum * kLoThreshold > run_sum[ct];
        }
        // ---- O^T += V^T . P (Q8g64: P'_g = p * v_scale_g, four output tiles per scale group): f16 hi, and lo while a
        // lane's probabilities of this step weigh more than 1/8 of its sum ----
        const bool lo_pass = __any(heavy);
        PREFILL_PHASE_FENCE();
#pragma unroll
        for (int q = 0; q < C::kDT / 4; ++q) {
            f32x4 gs0 = {1.f, 1.f, 1.f, 1.f}, gs1 = {1.f, 1.f, 1.f, 1.f};
            if constexpr (Q8) {
                gs0 = *(const f32x4*)(&lds_vs[sbuf][q][4 * j]);
                gs1 = *(const f32x4*)(&lds_vs[sbuf][q][16 + 4 * j]);
            }
            Frag phi[CT], plo[CT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float x0 = Q8 ? pr[ct][2 * e] * (e < 2 ? gs0[2 * e] : gs1[2 * e - 4]) : pr[ct][2 * e];
                    const float x1 = Q8 ? pr[ct][2 * e + 1] * (e < 2 ? gs0[2 * e + 1] : gs1[2 * e - 3]) : pr[ct][2 * e + 1];
                    phi[ct].u[e] = pack_f16_hw(x0, x1);
                    const f16x2 hi = __builtin_bit_cast(f16x2, pack_f16_hw(x0, x1));
                    plo[ct].u[e] = pack_f16_hw(x0 - (float)hi[0], x1 - (float)hi[1]);
                }
            }
            if (q + 1 < C::kDT / 4) { // the next four fragments travel while these multiply
#pragma unroll
                for (int tt = 0; tt < 4; ++tt) {
                    load_vfrag(vf[(q + 1) & 1][tt], (q + 1) * 4 + tt);
                }
            }
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    acc[ct][q * 4 + tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[q & 1][tt].h, phi[ct].h, acc[ct][q * 4 + tt], 0, 0, 0);
                }
            }
            if (lo_pass) {
#pragma unroll
                for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        acc[ct][q * 4 + tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[q & 1][tt].h, plo[ct].h, acc[ct][q * 4 + tt], 0, 0, 0);
                    }
                }
            }
        }
    };

    // ---- main loop: two tiles are attended per pass while the next two travel, one at a time through the same registers,
    // into the other pair of buffers, which nobody reads before the barrier ----
    StageRegs regs;
    load_step(regs, part.begin, entry_of(part.begin + st_token));
    unsigned int entry_next = entry_of(part.begin + kStep + st_token);
    store_step(regs, 0);
    load_step(regs, part.begin + kStep, entry_next); // past the end of the range the last row repeats: loads stay inside the pages
    entry_next = entry_of(part.begin + 2u * kStep + st_token);
    store_step(regs, 1);
    __syncthreads();
    unsigned int wv = 2u; // Q8g64: (biased) exponent of the largest V scale up to the tile being attended
    float v_shift = Q8 ? kPBias + 125.0f : kPBias;
    auto attend_tile = [&](unsigned int t0, int buf) __attribute__((always_inline)) {
        bool window_moved = false;
        float acc_fix = 1.0f;
        if constexpr (Q8) {
            const unsigned int wv_now = window_of(buf, wv);
            window_moved = wv_now != wv; // rare: a V scale above everything met so far
            if (window_moved) {
                acc_fix = ldexpf(1.0f, (int)wv - (int)wv_now);
                wv = wv_now;
                v_shift = kPBias + (float)(127 - (int)wv);
            }
        }
        compute_step(buf, t0, v_shift, acc_fix, window_moved);
    };
    auto two_steps = [&](unsigned int step, int set) __attribute__((always_inline)) {
        const unsigned int t0 = part.begin + step * kStep;
        load_step(regs, t0 + 2u * kStep, entry_next);
        entry_next = entry_of(t0 + 3u * kStep + st_token);
        attend_tile(t0, 2 * set);
        store_step(regs, 2 * (set ^ 1));
        PREFILL_PHASE_FENCE(); // the two tiles are attended one after the other: interleaved, their operands do not fit the registers
        load_step(regs, t0 + 3u * kStep, entry_next);
        entry_next = entry_of(t0 + 4u * kStep + st_token);
        attend_tile(t0 + kStep, 2 * set + 1);
        store_step(regs, 2 * (set ^ 1) + 1);
        __syncthreads();
    };
    unsigned int step = 0;
    for (; step + 4 <= steps; step += 4) {
        two_steps(step, 0);
        two_steps(step + 2u, 1);
    }
    if (step + 2 <= steps) {
        two_steps(step, 0);
        step += 2;
        if (step < steps) { // the odd tile at the end sits in the first buffer of the other pair
            attend_tile(part.begin + step * kStep, 2);
        }
    } else if (step < steps) {
        attend_tile(part.begin + step * kStep, 0);
    }

    // ---- normalise and store ------------------------------------------------------------------------
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const float total = wave_sum_16x4(run_sum[ct]);
        const unsigned int col = wave * (16u * CT) + ct * 16u + m;
        const unsigned int r = row0 + col / p.group;
        const unsigned int head = kvh * p.group + col % p.group;
        if (!(col < cols_used && r < p.rows)) {
            continue;
        }
        if (p.max_chunks > 1u) {
            store_split_record<C::kDT>(p, r, head, j, run_max[ct], total, acc[ct], v_shift);
            continue;
        }
        // accumulators and sum carry the same power of two (2^8 and, for Q8g64, the V window), which cancels here
        const float inv = (total > 0.0f && total < __builtin_inff()) ? 1.0f / total : 0.0f;
        const size_t base = ((size_t)r * p.num_heads + head) * D;
#pragma unroll
        for (int t = 0; t < C::kDT; ++t) {
            f32x4 v = acc[ct][t] * inv;
            if (inv == 0.0f) {
                v = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            const size_t at = base + t * 16 + 4 * j;
            if (p.gate != nullptr) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = gated(v[e], p.gate, p.gate_cols, p.gate_dtype, r, head * D + t * 16 + 4 * j + e);
                }
            }
            if (p.out_dtype == 0) {
                *(f32x4*)((float*)p.out + at) = v;
            } else {
                unsigned short* o = (unsigned short*)p.out + at;
                u32x2 packed;
                if (p.out_dtype == 1) {
                    packed = u32x2{pack_bf16_rne(v[0], v[1]), pack_bf16_rne(v[2], v[3])};
                } else {
                    packed = u32x2{(unsigned int)f32_to_f16_bits(v[0]) | ((unsigned int)f32_to_f16_bits(v[1]) << 16),
                                   (unsigned int)f32_to_f16_bits(v[2]) | ((unsigned int)f32_to_f16_bits(v[3]) << 16)};
                }
                *(u32x2*)o = packed;
            }
        }
    }
}

template <int D, int KV, int SDT> static hipError_t launch_prefill_tiles(const GqaPrefillParams& p, hipStream_t stream)
{
    const unsigned int cols = TileShape<D>::kCols;
    const unsigned int rows_per_wg = p.group >= cols ? 1u : cols / p.group;
    const dim3 grid((p.rows + rows_per_wg - 1) / rows_per_wg * p.num_kv_heads, 1, p.max_chunks > 1u ? p.max_chunks : 1u);
    const bool cap = p.softcap > 0.0f;
    const bool pow2 = (p.block_tokens & (p.block_tokens - 1u)) == 0 && p.table != nullptr;
    if (cap) {
        pow2 ? gqa_prefill_tiles<D, KV, SDT, true, true><<<grid, dim3(512), 0, stream>>>(p)
             : gqa_prefill_tiles<D, KV, SDT, true, false><<<grid, dim3(512), 0, stream>>>(p);
    } else {
        pow2 ? gqa_prefill_tiles<D, KV, SDT, false, true><<<grid, dim3(512), 0, stream>>>(p)
             : gqa_prefill_tiles<D, KV, SDT, false, false><<<grid, dim3(512), 0, stream>>>(p);
    }
    return hipGetLastError();
}

} // namespace

bool gqa_prefill_half_tiles(unsigned int rows, unsigned int position, unsigned int window, unsigned int num_heads, unsigned int num_kv_heads,
                            unsigned int head_dim, int kv_format, int scale_dtype, int q_dtype)
{
    if (kv_format != 0 || head_dim != (unsigned int)kD || scale_dtype == 2 || num_kv_heads == 0) {
        return false; // not gqa_prefill_q8's geometry
    }
    const unsigned int group = num_heads / num_kv_heads;
    if (group == 0 || group > 128u) {
        return false;
    }
    if (q_dtype == 0) {
        return true; // f32 queries travel as two f16 fragments: a wave has the registers for one column tile of them
    }
    if ((unsigned long long)rows * group <= 128u) {
        return true; // the whole chunk fits a half tile: a full one would be half empty at least
    }
    if (window != 0u) {
        return false;
    }
    const unsigned int full_rows = 256u / group;
    const unsigned long long full_tiles = ((unsigned long long)rows + full_rows - 1) / full_rows * num_kv_heads;
    // measured on 32 query / 8 KV heads: 2,048 rows at position 0 140 -> 122 us, 256 rows 40 -> 26 us; at position 1,024
    // (ranges 1 : 3) the half tiles' dearer steps cost what the evening out gains, 190 -> 200 us
    return full_tiles <= kComputeUnitsPrefill && (unsigned long long)position * 4u <= rows;
}

hipError_t launch_gqa_prefill(const GqaPrefillParams& p, int kv_format, int scale_dtype, hipStream_t stream)
{
    if (kv_format == 1) { // f16 rows
        if (p.head_dim == 128u) {
            return launch_prefill_tiles<128, 1, 0>(p, stream);
        }
        if (p.head_dim == 256u) {
            return launch_prefill_tiles<256, 1, 0>(p, stream);
        }
        return hipErrorInvalidValue;
    }
    if (kv_format != 0 || scale_dtype < 0 || scale_dtype > 2) {
        return hipErrorInvalidValue;
    }
    if (p.head_dim == 64u) {
        return scale_dtype == 0 ? launch_prefill_tiles<64, 0, 0>(p, stream)
                                : scale_dtype == 1 ? launch_prefill_tiles<64, 0, 1>(p, stream) : launch_prefill_tiles<64, 0, 2>(p, stream);
    }
    if (p.head_dim == 256u) {
        return scale_dtype == 0 ? launch_prefill_tiles<256, 0, 0>(p, stream)
                                : scale_dtype == 1 ? launch_prefill_tiles<256, 0, 1>(p, stream) : launch_prefill_tiles<256, 0, 2>(p, stream);
    }
    if (p.head_dim != (unsigned int)kD) {
        return hipErrorInvalidValue;
    }
    if (scale_dtype == 2) { // f32 scales at head_dim 128: the tile kernel (gqa_prefill_q8 reads 16-bit scales)
        return launch_prefill_tiles<128, 0, 2>(p, stream);
    }
    const unsigned int full_rows = p.group >= 256u ? 1u : 256u / p.group;
    const bool halves = gqa_prefill_half_tiles(p.rows, p.position, p.window, p.num_heads, p.num_kv_heads, p.head_dim, kv_format, scale_dtype, p.q_dtype);
    const unsigned int rows_per_wg = halves ? (p.group >= 128u ? 1u : 128u / p.group) : full_rows;
    const dim3 grid((p.rows + rows_per_wg - 1) / rows_per_wg * p.num_kv_heads, 1, p.max_chunks > 1u ? p.max_chunks : 1u);
    const bool cap = p.softcap > 0.0f;
    const bool pow2 = (p.block_tokens & (p.block_tokens - 1u)) == 0 && p.table != nullptr;
    const dim3 block(kThreads);
    auto launch = [&](auto sdt, auto softcap, auto table_pow2) {
        constexpr int S = decltype(sdt)::value;
        constexpr bool C = decltype(softcap)::value, P = decltype(table_pow2)::value;
        if (halves && p.q_dtype == 0) {
            gqa_prefill_q8<S, C, P, 1, true><<<grid, block, 0, stream>>>(p);
        } else if (halves) {
            gqa_prefill_q8<S, C, P, 1><<<grid, block, 0, stream>>>(p);
        } else {
            gqa_prefill_q8<S, C, P, 2><<<grid, block, 0, stream>>>(p);
        }
    };
    using std::integral_constant;
    if (scale_dtype == 0) {
        if (cap) {
            pow2 ? launch(integral_constant<int, 0>{}, std::true_type{}, std::true_type{}) : launch(integral_constant<int, 0>{}, std::true_type{}, std::false_type{});
        } else {
            pow2 ? launch(integral_constant<int, 0>{}, std::false_type{}, std::true_type{}) : launch(integral_constant<int, 0>{}, std::false_type{}, std::false_type{});
        }
    } else {
        if (cap) {
            pow2 ? launch(integral_constant<int, 1>{}, std::true_type{}, std::true_type{}) : launch(integral_constant<int, 1>{}, std::true_type{}, std::false_type{});
        } else {
            pow2 ? launch(integral_constant<int, 1>{}, std::false_type{}, std::true_type{}) : launch(integral_constant<int, 1>{}, std::false_type{}, std::false_type{});
        }
    }
    return hipGetLastError();
}

} // namespace zllm

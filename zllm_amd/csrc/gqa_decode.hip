// GQA split-KV flash decoding over a paged Q8g64 (or f16) KV cache — gfx950.
//
// Work decomposition
//   grid = (work item, kv-head block x head block); work item = (sequence, split), numbered
//   densely over the batch; one wave64 per KV head.
//   The waves of a workgroup cover neighbouring KV heads of the SAME tokens, so
//   together they read whole cache rows (all KV heads of a token are contiguous:
//   row = num_kv_heads * head_dim bytes) and share the row's scale line.
//   Waves never synchronise with each other.
//
// Per wave, per 32-token step (two 16-token tiles):
//   S^T[token, head] = K[token, :] . Q[head, :]      int8 MFMA 16x16x64, A = K codes as stored,
//                                                    B = Q in 24-bit fixed point, three 8-bit digits
//     one MFMA pair per 64-column scale group, so the group scale is applied to the finished
//     integer dot: s = sum_g scale_g * dot_g  (no per-element multiply, no K conversion)
//   online softmax: row max / row sum over the four 16-lane groups by wave shuffles
//   O^T[dim, head] += V^T[dim, token] . P'[token, head]   bf16 MFMA 16x16x32, A = V codes
//     (exact in bf16), B = P' = p * v_scale_g split into bf16 hi + lo (16 significant bits)
//   The C layout of S^T (lane = head column, 4 token rows) is exactly the B layout
//   needed for P', so probabilities never leave their registers.
//
// Two kernels share that step: gqa_decode_q8_dma128 (head_dim 128, pages of >= 16 tokens, no ring)
// streams K, V and scales global -> LDS with non-temporal full-line loads; gqa_decode_q8_partial
// covers every other geometry with a two-deep register pipeline.
//
// Why MFMA for a bandwidth-bound op: with 8 query heads per KV head the path needs
// 7.8 FMA per KV byte; at 70 % of 8 TB/s that is 43 T FMA/s, above the 39 T FMA/s
// the chip's (non-packed) FP32 vector units can issue.  On the matrix cores the
// same work is < 15 % of peak and the vector units only convert V codes and probabilities.
#include <type_traits>

#include "common.hpp"
#include "kernels.hpp"

namespace zllm {

namespace {

constexpr float kLog2e = 1.4426950408889634f;

union Frag {
    u32x4 u;
    bf16x8 b;
    f16x8 h;
};

__device__ __forceinline__ float byte_to_f32(unsigned int w, int e)
{
    return (float)(int)(signed char)((w >> (8 * e)) & 0xffu);
}

__device__ __forceinline__ float fast_tanh(float x)
{
    // small |x|: odd Taylor polynomial (the exponential form cancels to zero there);
    // otherwise tanh(x) = 1 - 2 / (exp(2x) + 1), which saturates cleanly.
    const float x2 = x * x;
    const float poly = x * (1.0f + x2 * (-1.0f / 3.0f + x2 * (2.0f / 15.0f + x2 * (-17.0f / 315.0f))));
    const float e = __builtin_amdgcn_exp2f(fminf(fabsf(x) * (2.0f * kLog2e), 80.0f));
    const float big = copysignf(1.0f - __fdividef(2.0f, e + 1.0f), x);
    return fabsf(x) < 0.1f ? poly : big;
}

// tanh(y) from t = 2 y log2(e): 1 - 2 / (2^t + 1), five instructions against fifteen.  The form cancels for tiny y: its
// absolute error is a few units of 2^-24, which the cap multiplies -- 3e-6 of a score under a cap of 50, nothing a softmax
// sees, but not the limit of an ever larger cap.  Caps up to kSmallCap use it; larger ones take fast_tanh.
constexpr float kSmallCap = 256.0f;
__device__ __forceinline__ float tanh_of_exponent(float t)
{
    return fmaf(-2.0f, __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(t) + 1.0f), 1.0f);
}

template <int G> struct ScaleRow; // G 16-bit scales of one token / KV head
template <> struct ScaleRow<1> {
    unsigned short v;
    __device__ __forceinline__ unsigned short get(int) const { return v; }
};
template <> struct ScaleRow<2> {
    unsigned int v;
    __device__ __forceinline__ unsigned short get(int a) const { return (unsigned short)(a == 0 ? (v & 0xffffu) : (v >> 16)); }
};
template <> struct ScaleRow<3> { // head_dim 192: three 16-bit words, two-byte aligned
    unsigned short v[3];
    __device__ __forceinline__ unsigned short get(int a) const { return v[a]; }
};
template <> struct ScaleRow<4> {
    u32x2 v;
    __device__ __forceinline__ unsigned short get(int a) const
    {
        const unsigned int w = a < 2 ? v.x : v.y;
        return (unsigned short)((a & 1) == 0 ? (w & 0xffffu) : (w >> 16));
    }
};

// f32 scales (the CUDA backend's convention, src/kernel/cuda/attention.rs:331-341): G floats per token and KV head.
template <int G> struct ScaleRowF32 {
    float v[G];
    __device__ __forceinline__ float get(int a) const { return v[a]; }
};
// Row type and value of a stored scale for a scale dtype (0 bf16, 1 f16, 2 f32).
template <int G, int SDT> struct ScaleRowOf {
    typedef ScaleRow<G> type;
};
template <int G> struct ScaleRowOf<G, 2> {
    typedef ScaleRowF32<G> type;
};
template <int SDT, class Row> __device__ __forceinline__ float scale_of(const Row& row, int a)
{
    if constexpr (SDT == 2) {
        return row.get(a);
    } else {
        return scale_bits_to_f32<SDT>(row.get(a));
    }
}

// Everything one wave loads for a 32-token step of a Q8g64 cache.
//   FAST (pages of >= 16 tokens): the 16 scale rows a 16-lane row needs in a step (2 tiles x 4 token slots x
//   {K, V}) are loaded one per lane and handed out with DPP row broadcasts — one load instead of sixteen.
//   Generic: every lane loads the scale rows of its eight token slots itself.
template <int G, bool FAST, int SDT> struct Q8Step {
    typedef typename ScaleRowOf<G, SDT>::type Row;
    u32x4 k[2][G];        // K codes: tile i, group a -> 16 codes of the lane's token
    unsigned int v[8][G]; // V codes: token slot s = i*4 + r, group a -> 4 codes (dims a*64 + 4m .. +4)
    Row ks[FAST ? 1 : 8]; // FAST: lane x of a row holds scale row (kv = x>>3, tile (x>>2)&1, slot x&3)
    Row vs[FAST ? 1 : 8];
};

// lane `n` of each 16-lane row, broadcast to the row (v_mov_b32 row_newbcast)
template <int N> __device__ __forceinline__ unsigned int row_bcast(unsigned int v)
{
    return __builtin_amdgcn_update_dpp(0u, v, 0x150 + N, 0xf, 0xf, false);
}

template <int G, int N> __device__ __forceinline__ ScaleRow<G> row_bcast_scales(const ScaleRow<G>& r)
{
    ScaleRow<G> out;
    if constexpr (G == 1) {
        out.v = (unsigned short)row_bcast<N>((unsigned int)r.v);
    } else if constexpr (G == 2) {
        out.v = row_bcast<N>(r.v);
    } else {
        out.v.x = row_bcast<N>(r.v.x);
        out.v.y = row_bcast<N>(r.v.y);
    }
    return out;
}

// A workgroup's waves: `items_per_group` work items side by side, each with one wave per KV head of the block (all KV
// heads when they fit the workgroup).  With one or two KV heads -- a small model, or one GPU's share of the heads -- a
// workgroup of one item would be one or two waves on a CU, far too few loads in flight; the waves share nothing, so
// several items ride in one workgroup instead.
struct WaveItem {
    unsigned int kvh, head_block, item;
};
__device__ __forceinline__ WaveItem wave_item(const GqaDecodeParams& p)
{
    const unsigned int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned int items = max(p.items_per_group, 1u);
    const unsigned int waves = (blockDim.x >> 6) / items; // per item
    const unsigned int kvh_blocks = (p.num_kv_heads + waves - 1) / waves;
    const unsigned int sub = wave / waves;
    WaveItem w;
    w.kvh = (blockIdx.y % kvh_blocks) * waves + (wave - sub * waves);
    w.head_block = blockIdx.y / kvh_blocks;
    w.item = blockIdx.x * items + sub;
    return w;
}

// Split-KV work items are numbered densely over the batch: item = (sequence b, split c) with
// c < splits(b), sequences in order.  Workgroups are handed to the XCDs round-robin by their linear id, so
// a dense numbering spreads the live workgroups of a ragged batch evenly (a [split][sequence] grid leaves
// gaps where short sequences end, and one XCD can end up with more live workgroups than CUs).  Every wave
// finds its item by a prefix sum over the sequences' split counts; ids past the last item exit.
// `span_out` is the split length of the item's sequence: its visible range cut into equal 32-aligned parts (never
// longer than the planned chunk_tokens), so that a ragged batch has no full-length splits next to short remainders --
// the longest split sets the kernel's duration.
// `row_out` is the item's row in the split record arrays: sequence x max_chunks + split, or, when the records are numbered
// densely, the item number itself -- the first split of a sequence then leaves its row in first_rows for the merge, and an
// item past the rows the host sized (a total_kv_tokens hint below the real sum) is dropped rather than written out of bounds.
__device__ __forceinline__ bool locate_split(const GqaDecodeParams& p, unsigned int item, unsigned int lane, unsigned int& b_out,
                                             unsigned int& chunk_out, unsigned int& len_out, unsigned int& first_out, unsigned int& span_out,
                                             unsigned int& row_out)
{
    if (p.record_rows != 0u && item >= p.record_rows) {
        return false;
    }
    unsigned int base = 0;
    for (unsigned int b0 = 0; b0 < p.batch; b0 += 64u) {
        const unsigned int i = b0 + lane;
        unsigned int n = 0, len = 0, first = 0, span = p.chunk_tokens;
        if (i < p.batch) {
            len = p.kv_lens[i];
            first = p.first_visible != nullptr ? p.first_visible[i] : 0u;
            first = min(first, len);
            const unsigned int first_al = first & ~31u;
            n = min(p.max_chunks, (len - first_al + p.chunk_tokens - 1u) / p.chunk_tokens);
            if (n > 0) {
                span = min(p.chunk_tokens, (((len - first_al + n - 1u) / n) + 31u) & ~31u);
            }
        }
        unsigned int incl = n; // inclusive prefix sum over the wave
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const unsigned int up = __shfl_up(incl, d);
            incl += lane >= (unsigned int)d ? up : 0u;
        }
        const unsigned int total = __builtin_amdgcn_readlane(incl, 63);
        if (item < base + total) {
            const unsigned int local = item - base;
            const unsigned long long hit = __ballot(local >= incl - n && local < incl);
            const unsigned int src = (unsigned int)__builtin_ctzll(hit);
            b_out = b0 + src;
            chunk_out = local - (__builtin_amdgcn_readlane(incl, src) - __builtin_amdgcn_readlane(n, src));
            len_out = __builtin_amdgcn_readlane(len, src); // already here: no second trip to memory for them
            first_out = __builtin_amdgcn_readlane(first, src);
            span_out = __builtin_amdgcn_readlane(span, src);
            row_out = b_out * p.max_chunks + chunk_out;
            if (p.record_rows != 0u) {
                row_out = item;
                if (chunk_out == 0u && lane == 0u) {
                    p.first_rows[b_out] = item; // every wave of the split writes the same number
                }
            }
            return true;
        }
        base += total;
    }
    return false;
}

// Q fragments: B operand of the int8 MFMA, lane = (head column m, k-slice j).
// The head's query row is quantized to 24-bit fixed point and split into three signed-byte digits,
// q = step * (256 * hi + lo + ex / 256) with step = max|q| / 32512, hi in [-127, 127], lo and ex in [-128, 127]:
// K codes then feed the matrix cores as raw bytes and the integer dot products are exact
// (|256 * dot_hi + dot_lo| < 2^28 for 64 columns).  Two digits were not enough: with a score scale of 0.2 over
// x8 outlier channels a 2^-17 step of the row's largest element moves outputs of magnitude 20 by up to 3e-3.
// Fetching and quantizing are separate so that a kernel can start the fetch, issue other loads, and
// quantize when the data is needed.
template <int D> struct QueryRaw {
    u32x4 v[D / 64][4]; // 16 consecutive elements per scale group: four vectors of f32, or two of 16-bit values
};

template <int D>
__device__ __forceinline__ QueryRaw<D> fetch_query(const GqaDecodeParams& p, unsigned int b, unsigned int head, bool head_valid, unsigned int j)
{
    constexpr int G = D / 64;
    QueryRaw<D> raw;
    const size_t q_index = ((size_t)b * p.num_heads + head) * D + j * 16;
#pragma unroll
    for (int a = 0; a < G; ++a) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            raw.v[a][w] = u32x4{0u, 0u, 0u, 0u};
        }
    }
    if (head_valid) {
        if (p.q_dtype == 0) {
#pragma unroll
            for (int a = 0; a < G; ++a) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    raw.v[a][w] = *(const u32x4*)((const float*)p.q + q_index + a * 64 + 4 * w);
                }
            }
        } else {
#pragma unroll
            for (int a = 0; a < G; ++a) {
#pragma unroll
                for (int w = 0; w < 2; ++w) {
                    raw.v[a][w] = *(const u32x4*)((const unsigned short*)p.q + q_index + a * 64 + 8 * w);
                }
            }
        }
    }
    return raw;
}

template <int G> struct QueryDigits {
    i32x4 hi[G], lo[G], ex[G];
};

template <int D>
__device__ __forceinline__ void quantize_query(const GqaDecodeParams& p, const QueryRaw<D>& raw, QueryDigits<D / 64>& qd, float& q_step)
{
    constexpr int G = D / 64;
    float x[G][16];
#pragma unroll
    for (int a = 0; a < G; ++a) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            if (p.q_dtype == 0) {
                x[a][e] = __uint_as_float(raw.v[a][e / 4][e % 4]);
            } else {
                const unsigned int word = raw.v[a][e / 8][(e % 8) / 2];
                const unsigned short bits = (unsigned short)((e & 1) ? (word >> 16) : (word & 0xffffu));
                x[a][e] = p.q_dtype == 1 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits);
            }
        }
    }
    float q_absmax = 0.0f;
#pragma unroll
    for (int a = 0; a < G; ++a) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            q_absmax = fmaxf(q_absmax, fabsf(x[a][e]));
        }
    }
    q_absmax = wave_max_16x4(q_absmax);
    const bool q_ok = q_absmax > 0.0f && q_absmax < __builtin_inff();
    q_step = q_ok ? q_absmax * (1.0f / 32512.0f) : 0.0f;
    const float inv_step = q_ok ? (32512.0f * 256.0f) / q_absmax : 0.0f; // to units of the last digit
#pragma unroll
    for (int a = 0; a < G; ++a) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            unsigned int hi_word = 0, lo_word = 0, ex_word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                int qi = (int)rintf(x[a][4 * w + e] * inv_step); // |x * inv_step| <= 2^23: an exact integer
                qi = max(-32512 * 256, min(32512 * 256, qi));
                const int top = (qi + 128) >> 8; // the upper two digits, |top| <= 32512
                const int ex = qi - top * 256;
                const int hi = (top + 128) >> 8;
                const int lo = top - hi * 256;
                hi_word |= ((unsigned int)hi & 0xffu) << (8 * e);
                lo_word |= ((unsigned int)lo & 0xffu) << (8 * e);
                ex_word |= ((unsigned int)ex & 0xffu) << (8 * e);
            }
            qd.hi[a][w] = (int)hi_word;
            qd.lo[a][w] = (int)lo_word;
            qd.ex[a][w] = (int)ex_word;
        }
    }
}

template <int D>
__device__ __forceinline__ void load_query_digits(const GqaDecodeParams& p, unsigned int b, unsigned int head, bool head_valid,
                                                  unsigned int j, QueryDigits<D / 64>& qd, float& q_step)
{
    const QueryRaw<D> raw = fetch_query<D>(p, b, head, head_valid, j);
    quantize_query<D>(p, raw, qd, q_step);
}

// One 32-token step, first half: scores, masking and the online-softmax update.
//   k[i][a]   16 K codes of the lane's token of tile i, scale group a (raw bytes = int8 MFMA A operand)
//   ksr[i*4+r] scale row of token slot (tile i, row 4j + r) -- the C layout of the score tile
// Leaves the step's probabilities in pr[] (same slots) and rescales acc when the running max moved.
template <int G, int SDT, bool SOFTCAP, class Row>
__device__ __forceinline__ void qk_softmax_step(const u32x4 (&k)[2][G], const Row (&ksr)[8], const QueryDigits<G>& qd,
                                            float scale_log2, float inv_cap, float cap_log2,
                                            unsigned int t0, unsigned int j, unsigned int first, unsigned int len,
                                            float& run_max, float& run_sum, f32x4 (&acc)[G * 4], float (&pr)[8])
{
    constexpr int MT = G * 4;
    // ---- S^T = K . Q^T, one accumulator per scale group -----------------------------
    float sc[8];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        float tile_s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int a = 0; a < G; ++a) {
            const i32x4 kc = __builtin_bit_cast(i32x4, k[i][a]);
            const i32x4 zero = {0, 0, 0, 0};
            const i32x4 dh = __builtin_amdgcn_mfma_i32_16x16x64_i8(kc, qd.hi[a], zero, 0, 0, 0);
            const i32x4 dl = __builtin_amdgcn_mfma_i32_16x16x64_i8(kc, qd.lo[a], zero, 0, 0, 0);
            const i32x4 de = __builtin_amdgcn_mfma_i32_16x16x64_i8(kc, qd.ex[a], zero, 0, 0, 0);
            f32x4 d;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                d[r] = fmaf((float)de[r], 1.0f / 256.0f, (float)(dh[r] * 256 + dl[r]));
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                tile_s[r] = fmaf(d[r], scale_of<SDT>(ksr[i * 4 + r], a), tile_s[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float x = tile_s[r] * scale_log2;
            if constexpr (SOFTCAP) {
                x = cap_log2 < kSmallCap * kLog2e ? cap_log2 * tanh_of_exponent(x * (inv_cap * 2.0f * kLog2e)) : cap_log2 * fast_tanh(x * inv_cap);
            }
            sc[i * 4 + r] = x;
        }
    }
    if (t0 < first || t0 + 32u > len) { // only the first and the last step of a visible range have slots to mask (wave-uniform)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const unsigned int token = t0 + 16u * (e >> 2) + 4u * j + (e & 3);
            sc[e] = (token >= first && token < len) ? sc[e] : kNegInf;
        }
    }
    // ---- online softmax (base 2) -----------------------------------------------------
    float step_max = sc[0];
#pragma unroll
    for (int e = 1; e < 8; ++e) {
        step_max = fmaxf(step_max, sc[e]);
    }
    step_max = wave_max_16x4(step_max);
    const float new_max = fmaxf(run_max, step_max);
    const float safe_max = new_max == kNegInf ? 0.0f : new_max;
    const float alpha = __builtin_amdgcn_exp2f(run_max - safe_max);
    float step_sum = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        pr[e] = __builtin_amdgcn_exp2f(sc[e] - safe_max);
        step_sum += pr[e];
    }
    run_sum = run_sum * alpha + step_sum;
    run_max = new_max;
    if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            acc[t] *= alpha;
        }
    }
}

// Second half: O^T += V^T . P' with P' = p * v_scale split into bf16 hi + lo.
//   v[i*4+r][a]  4 V codes (dims a*64 + 4m .. +4) of token slot (tile i, row 4j + r)
template <int G, int SDT, class Row>
__device__ __forceinline__ void pv_step(const unsigned int (&v)[8][G], const Row (&vsr)[8], const float (&pr)[8],
                                    f32x4 (&acc)[G * 4])
{
    // ---- O^T += V^T . P', P' = p * v_scale split into bf16 hi + lo --------------------
#pragma unroll
    for (int a = 0; a < G; ++a) {
        Frag phi, plo;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float x0 = pr[2 * e] * scale_of<SDT>(vsr[2 * e], a);
            const float x1 = pr[2 * e + 1] * scale_of<SDT>(vsr[2 * e + 1], a);
            unsigned int hi, lo;
            split_bf16_pair(x0, x1, hi, lo);
            phi.u[e] = hi;
            plo.u[e] = lo;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Frag vf;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                vf.u[c] = pack_bf16_trunc(byte_to_f32(v[2 * c][a], e), byte_to_f32(v[2 * c + 1][a], e));
            }
            f32x4 d = acc[a * 4 + e];
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, phi.b, d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, plo.b, d, 0, 0, 0);
            acc[a * 4 + e] = d;
        }
    }
}

// A FAST path loads whole 16-token tiles, so on the first and last step of a visible range the rows outside
// [first, len) are whatever their page holds.  Their probabilities are exact zeros, but 0 * scale is NaN when the
// stale scale bits read as NaN or infinity, and one NaN in P' poisons every dimension of the head.  Clearing the
// scale rows of those slots (wave-uniform test, edge steps only) makes them contribute exact zeros.
template <int G, class Row>
__device__ __forceinline__ void clear_hidden_scale_rows(Row (&vsr)[8], unsigned int t0, unsigned int j, unsigned int first,
                                                        unsigned int len)
{
    if (t0 >= first && t0 + 32u <= len) {
        return;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const unsigned int token = t0 + 16u * (e >> 2) + 4u * j + (e & 3);
        if (token < first || token >= len) {
            vsr[e] = Row{};
        }
    }
}

// NBUF = steps of KV kept in registers: loads run NBUF - 1 steps (32 tokens each) ahead of the MFMA work.
// With pages scattered over a large pool every page costs an address translation as well as an HBM access,
// and one step of prefetch leaves the wave waiting ~3.5 us per step.
template <int D, int SDT, bool FAST, bool SOFTCAP, int NBUF>
__global__ __launch_bounds__(D > 128 ? 256 : 512) void gqa_decode_q8_partial(GqaDecodeParams p)
{
    constexpr int G = D / 64;           // scale groups per head row
    typedef typename ScaleRowOf<G, SDT>::type Row;
    constexpr unsigned int kScaleBytes = SDT == 2 ? 4u : 2u;
    static_assert(!(FAST && SDT == 2), "f32 scales run the generic path");
    constexpr int MT = D / 16;          // output M tiles
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int m = lane & 15u;  // MFMA row / column index of this lane
    const unsigned int j = lane >> 4;   // k-slice index of this lane
    const WaveItem mine = wave_item(p);
    const unsigned int kvh = mine.kvh;
    const unsigned int head_block = mine.head_block;
    unsigned int b, chunk, len, first, span, row;
    if (kvh >= p.num_kv_heads || !locate_split(p, mine.item, threadIdx.x & 63u, b, chunk, len, first, span, row)) {
        return;
    }
    const unsigned int first_al = first & ~31u;
    const unsigned long long c_start64 = (unsigned long long)first_al + (unsigned long long)chunk * span;
    const unsigned int head_in_group = head_block * 16u + m;
    const bool head_valid = head_in_group < p.group;
    const unsigned int head = kvh * p.group + head_in_group;

    const size_t stat_index = ((size_t)row * p.num_heads + head) * 2;
    if (c_start64 >= len) {
        if (head_valid && j == 0) {
            p.stats[stat_index] = kNegInf;
            p.stats[stat_index + 1] = 0.0f;
        }
        return;
    }
    const unsigned int c_start = (unsigned int)c_start64;
    const unsigned int c_end = (unsigned int)min((unsigned long long)len, c_start64 + span);
    const unsigned int steps = (c_end - c_start + 31u) / 32u;

    QueryDigits<G> qd;
    float q_step; // value of one unit of the middle digit for this lane's head
    load_query_digits<D>(p, b, head, head_valid, j, qd, q_step);

    const unsigned int* table = p.tables + (p.table_shared ? 0 : (size_t)b * p.table_stride);
    const unsigned int k_row = p.num_kv_heads * D;           // bytes per cache row (codes)
    const unsigned int s_row = p.num_kv_heads * G * kScaleBytes; // bytes per scale row
    const unsigned char* k_base = p.k_plane + (size_t)kvh * D;
    const unsigned char* v_base = p.v_plane + (size_t)kvh * D;
    const unsigned char* ks_base = p.k_scales + (size_t)kvh * G * kScaleBytes;
    const unsigned char* vs_base = p.v_scales + (size_t)kvh * G * kScaleBytes;
    const unsigned int block_mask = p.block_tokens - 1u;
    const unsigned int lo_tile = first & ~15u;
    const unsigned int hi_tile = (len - 1u) & ~15u;

    // physical row of the first token of the (clamped) 16-token tile starting at T.  When the split spans
    // at most 128 pages (and no ring), the wave loads its block-table entries once into two registers
    // (lane i = entry first_page + i / + 64 + i) and reads them with v_readlane: no table load inside the loop.
    const unsigned int first_page = min(max(c_start, lo_tile), hi_tile) >> p.block_shift;
    const unsigned int last_page = p.table_stride != 0 ? p.table_stride - 1u : 0u;
    const bool cached_table = FAST && p.ring_capacity == 0 && ((min(max(c_end - 1u, lo_tile), hi_tile) >> p.block_shift) - first_page) < 128u;
    unsigned int entries0 = 0, entries1 = 0;
    if (cached_table) {
        entries0 = p.tables != nullptr ? table[min(first_page + lane, last_page)] : first_page + lane;
        entries1 = p.tables != nullptr ? table[min(first_page + 64u + lane, last_page)] : first_page + 64u + lane;
    }
    // Pin the two registers here: the wait for their loads is placed at this point, once, instead of in
    // front of every v_readlane inside the loop (where a full vmcnt(0) would also drain the KV prefetch).
    asm volatile("" : "+v"(entries0), "+v"(entries1));
    auto tile_row = [&](unsigned int T) __attribute__((always_inline)) -> unsigned long long {
        unsigned int t = min(max(T, lo_tile), hi_tile);
        if (p.ring_capacity != 0) {
            t %= p.ring_capacity;
        }
        unsigned int entry;
        if (cached_table) {
            const unsigned int idx = __builtin_amdgcn_readfirstlane((t >> p.block_shift) - first_page);
            const unsigned int e0 = __builtin_amdgcn_readlane(entries0, idx & 63u);
            const unsigned int e1 = __builtin_amdgcn_readlane(entries1, idx & 63u);
            entry = idx < 64u ? e0 : e1;
        } else {
            entry = p.tables != nullptr ? __builtin_amdgcn_readfirstlane(table[t >> p.block_shift]) : (t >> p.block_shift);
        }
        return ((unsigned long long)entry << p.block_shift) + (t & block_mask);
    };
    // physical row of one token (generic path: any page size / ring)
    auto token_row = [&](unsigned int t) __attribute__((always_inline)) -> unsigned long long {
        t = min(max(t, first), len - 1u);
        return paged_row(p.tables != nullptr ? table : nullptr, t, p.block_tokens, p.ring_capacity);
    };

    // lane-constant byte offsets (FAST path): every load is `uniform tile base + lane offset [+ immediate]`
    const unsigned int k_off = m * k_row + j * 16u;
    unsigned int v_off[4], s_off = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        v_off[r] = (4u * j + r) * k_row + 4u * m;
    }
    const unsigned int sx = lane & 15u;                   // this lane's role in the scale load
    const bool sx_value = (sx >> 3) != 0;                 // V scales (else K)
    const bool sx_tile1 = ((sx >> 2) & 1u) != 0;          // second tile of the step
    s_off = (4u * j + (sx & 3u)) * s_row;
    const unsigned char* s_plane = sx_value ? vs_base : ks_base;

    auto load_step = [&](Q8Step<G, FAST, SDT>& s, unsigned int t0) __attribute__((always_inline)) {
        if constexpr (FAST) {
            const unsigned long long R0 = tile_row(t0);
            const unsigned long long R1 = tile_row(t0 + 16u);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const unsigned long long R = i == 0 ? R0 : R1;
                const unsigned char* kt = k_base + R * k_row; // uniform
                const unsigned char* vt = v_base + R * k_row;
#pragma unroll
                for (int a = 0; a < G; ++a) {
                    s.k[i][a] = *(const u32x4*)(kt + k_off + a * 64);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
#pragma unroll
                    for (int a = 0; a < G; ++a) {
                        s.v[i * 4 + r][a] = *(const unsigned int*)(vt + v_off[r] + a * 64);
                    }
                }
            }
            const unsigned long long Rs = sx_tile1 ? R1 : R0;
            s.ks[0] = *(const Row*)(s_plane + Rs * s_row + s_off);
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const unsigned long long rk = token_row(t0 + 16u * i + m);
                const unsigned char* kr = k_base + rk * k_row + j * 16u;
#pragma unroll
                for (int a = 0; a < G; ++a) {
                    s.k[i][a] = *(const u32x4*)(kr + a * 64);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const unsigned long long row = token_row(t0 + 16u * i + 4u * j + r);
                    const unsigned char* vr = v_base + row * k_row + 4u * m;
#pragma unroll
                    for (int a = 0; a < G; ++a) {
                        s.v[i * 4 + r][a] = *(const unsigned int*)(vr + a * 64);
                    }
                    s.ks[i * 4 + r] = *(const Row*)(ks_base + row * s_row);
                    s.vs[i * 4 + r] = *(const Row*)(vs_base + row * s_row);
                }
            }
        }
    };

    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    float run_max = kNegInf; // log2 units
    float run_sum = 0.0f;    // lane-partial (this lane's 8 token slots per step)
    const float scale_log2 = (SOFTCAP ? p.score_scale : p.score_scale * kLog2e) * q_step;
    const float inv_cap = SOFTCAP ? 1.0f / p.softcap : 0.0f;
    const float cap_log2 = p.softcap * kLog2e;

    auto compute_step = [&](const Q8Step<G, FAST, SDT>& s, unsigned int t0) __attribute__((always_inline)) {
        // scale rows of this lane's eight token slots (K then V)
        Row ksr[8], vsr[8];
        if constexpr (FAST) {
            ksr[0] = row_bcast_scales<G, 0>(s.ks[0]);
            ksr[1] = row_bcast_scales<G, 1>(s.ks[0]);
            ksr[2] = row_bcast_scales<G, 2>(s.ks[0]);
            ksr[3] = row_bcast_scales<G, 3>(s.ks[0]);
            ksr[4] = row_bcast_scales<G, 4>(s.ks[0]);
            ksr[5] = row_bcast_scales<G, 5>(s.ks[0]);
            ksr[6] = row_bcast_scales<G, 6>(s.ks[0]);
            ksr[7] = row_bcast_scales<G, 7>(s.ks[0]);
            vsr[0] = row_bcast_scales<G, 8>(s.ks[0]);
            vsr[1] = row_bcast_scales<G, 9>(s.ks[0]);
            vsr[2] = row_bcast_scales<G, 10>(s.ks[0]);
            vsr[3] = row_bcast_scales<G, 11>(s.ks[0]);
            vsr[4] = row_bcast_scales<G, 12>(s.ks[0]);
            vsr[5] = row_bcast_scales<G, 13>(s.ks[0]);
            vsr[6] = row_bcast_scales<G, 14>(s.ks[0]);
            vsr[7] = row_bcast_scales<G, 15>(s.ks[0]);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                ksr[e] = s.ks[e];
                vsr[e] = s.vs[e];
            }
        }
        float pr[8];
        qk_softmax_step<G, SDT, SOFTCAP>(s.k, ksr, qd, scale_log2, inv_cap, cap_log2, t0, j, first, len, run_max, run_sum, acc, pr);
        clear_hidden_scale_rows<G>(vsr, t0, j, first, len);
        pv_step<G, SDT>(s.v, vsr, pr, acc);
    };

    // ---- software pipeline: loads of steps n+1 .. n+NBUF-1 in flight while step n computes ----------
    Q8Step<G, FAST, SDT> buf[NBUF];
#pragma unroll
    for (int u = 0; u < NBUF - 1; ++u) {
        if ((unsigned int)u < steps) {
            load_step(buf[u], c_start + u * 32u);
        }
    }
    // The main loop issues its loads unconditionally (past the end it re-reads the last step, an L2 hit):
    // a conditional load would make the compiler merge "loads in flight" with "none in flight" and wait for
    // everything before each compute step, which serialises the prefetch.
    unsigned int base = 0;
    for (; base + NBUF <= steps; base += NBUF) {
#pragma unroll
        for (int u = 0; u < NBUF; ++u) {
            const unsigned int step = base + u;
            load_step(buf[(u + NBUF - 1) % NBUF], c_start + min(step + NBUF - 1, steps - 1u) * 32u);
            compute_step(buf[u], c_start + step * 32u);
        }
    }
#pragma unroll
    for (int u = 0; u < NBUF - 1; ++u) {
        if (base + u < steps) {
            compute_step(buf[u], c_start + (base + u) * 32u);
        }
    }

    // ---- write the un-normalised partial and (max, sum) -------------------------------------
    const float total = wave_sum_16x4(run_sum);
    if (head_valid) {
        if (j == 0) {
            p.stats[stat_index] = run_max;
            p.stats[stat_index + 1] = total;
        }
        float* out = p.partial + ((size_t)row * p.num_heads + head) * D;
        // tile (a, e), register r holds dim a*64 + 16*j + 4*r + e
#pragma unroll
        for (int a = 0; a < G; ++a) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const f32x4 v = {acc[a * 4 + 0][r], acc[a * 4 + 1][r], acc[a * 4 + 2][r], acc[a * 4 + 3][r]};
                *(f32x4*)(out + a * 64 + 16 * j + 4 * r) = v;
            }
        }
    }
}

// ---- head_dim 128: K, V and scale rows travel global -> LDS without touching registers ---------
// Each wave owns a private LDS region (no barriers): rings of two 32-token steps for the K codes, the V
// codes and the scale rows of its KV head.  global_load_lds moves 64 x 16 B per instruction; eight
// neighbouring lanes fetch one whole 128-byte row slice, so every request is a full cache line and the
// loads can be marked non-temporal (lines are used exactly once).  The 16-byte chunk a lane fetches is
// XOR-swizzled with its row, which makes the later ds_read_b128 of MFMA operands bank-conflict free.
// The compiler does not order LDS reads against these loads, so the waits are explicit: loads are issued
// in a fixed order, unconditionally, and s_waitcnt vmcnt(N) counts the instructions issued since.
constexpr int kDmaPlaneStep = 2 * 16 * 128;                              // one plane, one step, one KV head
constexpr int kDmaScaleStep = 2 * 32 * 4;                                // K and V scale rows of one step
constexpr int kDmaWaveBytes = 4 * kDmaPlaneStep + 2 * kDmaScaleStep;     // 16896
constexpr int kDmaWaves = 8;
constexpr int kAuxNonTemporal = 2; // cache-policy bits of the load builtin: nt

template <int N> __device__ __forceinline__ void wait_vmcnt()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void wait_lds_reads()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;

template <int SDT, bool SOFTCAP>
__global__ __launch_bounds__(512) void gqa_decode_q8_dma128(GqaDecodeParams p)
{
    constexpr int D = 128, G = 2, MT = 8;
    __shared__ __attribute__((aligned(1024))) unsigned char lds_all[kDmaWaves * kDmaWaveBytes];
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int m = lane & 15u;
    const unsigned int j = lane >> 4;
    const unsigned int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const WaveItem mine = wave_item(p);
    const unsigned int kvh = mine.kvh;
    const unsigned int head_block = mine.head_block;
    if (kvh >= p.num_kv_heads) {
        return;
    }
    // The item's place in the batch depends on every sequence's length, which is one trip to memory; the block-table
    // entries it then needs are a second one before the first row can be requested.  When every sequence fills all
    // planned splits, item i is split i % max_chunks of sequence i / max_chunks: the entries of that guess are
    // requested together with the lengths and are kept if the guess turns out right.
    const unsigned int last_page = p.table_stride != 0 ? p.table_stride - 1u : 0u;
    const unsigned int guess_b = min(mine.item / p.max_chunks, p.batch - 1u);
    const unsigned int guess_page = ((mine.item - guess_b * p.max_chunks) * p.chunk_tokens) >> p.block_shift;
    const unsigned int* guess_table = p.tables + (p.table_shared ? 0 : (size_t)guess_b * p.table_stride);
    unsigned int entries0 = 0, entries1 = 0;
    if (p.tables != nullptr) {
        entries0 = guess_table[min(guess_page + lane, last_page)];
        entries1 = guess_table[min(guess_page + 64u + lane, last_page)];
    }
    unsigned int b, chunk, len, first, span, row;
    if (!locate_split(p, mine.item, threadIdx.x & 63u, b, chunk, len, first, span, row)) {
        return;
    }
    const unsigned int first_al = first & ~31u;
    const unsigned long long c_start64 = (unsigned long long)first_al + (unsigned long long)chunk * span;
    const unsigned int head_in_group = head_block * 16u + m;
    const bool head_valid = head_in_group < p.group;
    const unsigned int head = kvh * p.group + head_in_group;
    const size_t stat_index = ((size_t)row * p.num_heads + head) * 2;
    if (c_start64 >= len) {
        if (head_valid && j == 0) {
            p.stats[stat_index] = kNegInf;
            p.stats[stat_index + 1] = 0.0f;
        }
        return;
    }
    const unsigned int c_start = (unsigned int)c_start64;
    const unsigned int c_end = (unsigned int)min((unsigned long long)len, c_start64 + span);
    const unsigned int steps = (c_end - c_start + 31u) / 32u;

    const unsigned int* table = p.tables + (p.table_shared ? 0 : (size_t)b * p.table_stride);
    const unsigned int k_row = p.num_kv_heads * D;
    const unsigned int s_row = p.num_kv_heads * G * 2u;
    const unsigned char* k_base = p.k_plane + (size_t)kvh * D;
    const unsigned char* v_base = p.v_plane + (size_t)kvh * D;
    const unsigned int block_mask = p.block_tokens - 1u;
    const unsigned int lo_tile = first & ~15u;
    const unsigned int hi_tile = (len - 1u) & ~15u;

    // block-table entries of this split: lane i holds entry first_page + i (+ 64); the launcher keeps a
    // split within 128 pages
    const unsigned int first_page = min(max(c_start, lo_tile), hi_tile) >> p.block_shift;
    if (p.tables == nullptr) {
        entries0 = first_page + lane;
        entries1 = first_page + 64u + lane;
    } else if (table != guess_table || first_page != guess_page) {
        entries0 = table[min(first_page + lane, last_page)];
        entries1 = table[min(first_page + 64u + lane, last_page)];
    }
    // the query fetch rides along with the table loads; it is quantized after the first KV loads are out
    const QueryRaw<D> q_raw = fetch_query<D>(p, b, head, head_valid, j);
    asm volatile("" : "+v"(entries0), "+v"(entries1)); // their wait happens here, not inside the loop
    auto tile_row = [&](unsigned int T) __attribute__((always_inline)) -> unsigned long long {
        const unsigned int t = min(max(T, lo_tile), hi_tile);
        const unsigned int idx = __builtin_amdgcn_readfirstlane((t >> p.block_shift) - first_page) & 127u;
        const unsigned int e0 = __builtin_amdgcn_readlane(entries0, idx & 63u);
        const unsigned int e1 = __builtin_amdgcn_readlane(entries1, idx & 63u);
        const unsigned int entry = idx < 64u ? e0 : e1;
        return ((unsigned long long)entry << p.block_shift) + (t & block_mask);
    };

    // ---- LDS map of this wave -----------------------------------------------------------------
    unsigned char* const wave_lds = lds_all + wave * kDmaWaveBytes;
    unsigned char* const lds_k = wave_lds;                      // [slot 2][tile 2][row 16][128]
    unsigned char* const lds_v = wave_lds + 2 * kDmaPlaneStep;  // same
    unsigned char* const lds_s = wave_lds + 4 * kDmaPlaneStep;  // [slot 2][plane K,V][token 32][4]

    // global side of a code-tile load: lane -> (row lane / 8 [+ 8], swizzled 16-byte chunk)
    const unsigned int code_goff = (lane >> 3) * k_row + (((lane & 7u) ^ (lane >> 3)) << 4);
    // global side of the scale load: lane -> (plane lane / 32, token lane % 32)
    const bool s_tile1 = ((lane >> 4) & 1u) != 0;
    const unsigned char* s_lane_base = (lane >= 32u ? p.v_scales : p.k_scales) + (size_t)kvh * G * 2u + (size_t)(lane & 15u) * s_row;
    // LDS side: MFMA operand addresses (chunk c of row r sits at r * 128 + ((c ^ (r & 7)) << 4))
    unsigned int k_lds[G], v_lds[4];
#pragma unroll
    for (int a = 0; a < G; ++a) {
        k_lds[a] = m * 128u + (((4u * a + j) ^ (m & 7u)) << 4);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const unsigned int row = 4u * j + r;
        v_lds[r] = row * 128u + (((m >> 2) ^ (row & 7u)) << 4) + (m & 3u) * 4u; // group 0; group 1 = ^ 64
    }
    const unsigned int s_lds = 16u * j;

    auto issue_codes = [&](const unsigned char* plane_base, unsigned char* ring, int slot, unsigned int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const unsigned long long R = tile_row(t0 + 16u * i);
            const unsigned char* src = plane_base + R * k_row; // uniform
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                __builtin_amdgcn_global_load_lds((global_ptr_t)(src + (size_t)h * 8u * k_row + code_goff),
                                                 (lds_ptr_t)(ring + slot * kDmaPlaneStep + i * 2048 + h * 1024), 16, 0, kAuxNonTemporal);
            }
        }
    };
    auto issue_scales = [&](int slot, unsigned int t0) __attribute__((always_inline)) {
        const unsigned long long R0 = tile_row(t0);
        const unsigned long long R1 = tile_row(t0 + 16u);
        const unsigned long long R = s_tile1 ? R1 : R0;
        __builtin_amdgcn_global_load_lds((global_ptr_t)(s_lane_base + R * s_row), (lds_ptr_t)(lds_s + slot * kDmaScaleStep), 4, 0, 0);
    };

    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    float run_max = kNegInf;
    float run_sum = 0.0f;

    // prologue: steps 0 and 1 in the same order the loop issues them; the query is fetched and quantized
    // while these loads are in flight
    {
        const unsigned int t1 = c_start + min(1u, steps - 1u) * 32u;
        issue_codes(k_base, lds_k, 0, c_start);
        issue_scales(0, c_start);
        issue_codes(v_base, lds_v, 0, c_start);
        issue_codes(k_base, lds_k, 1, t1);
        issue_scales(1, t1);
        issue_codes(v_base, lds_v, 1, t1);
    }
    QueryDigits<G> qd;
    float q_step;
    quantize_query<D>(p, q_raw, qd, q_step);

    const float scale_log2 = (SOFTCAP ? p.score_scale : p.score_scale * kLog2e) * q_step;
    const float inv_cap = SOFTCAP ? 1.0f / p.softcap : 0.0f;
    const float cap_log2 = p.softcap * kLog2e;

    // Issue order per step n (9 instructions): K(n+2) x4, scales(n+2) x1, [QK, softmax], V(n+2) x4.
    //   K(n), scales(n) complete  <=> at most 13 newer loads outstanding (V(n), K/S/V(n+1))
    //   V(n) complete             <=> at most 14 newer loads outstanding (K/S/V(n+1), K/S(n+2))
    // The last two steps of a split request nothing (behind = batches of loads still behind this step's: 2 in the
    // steady state, then 1, then 0) and wait with the counts that follow from that.
    auto step = [&](auto slot_c, auto behind_c, unsigned int n) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_c)::value;
        constexpr int behind = decltype(behind_c)::value;
        const unsigned int t0 = c_start + n * 32u;
        const unsigned int t_next = c_start + (n + 2u) * 32u;
        wait_vmcnt<behind == 0 ? 4 : 13>();
        u32x4 k[2][G];
        ScaleRow<G> ksr[8], vsr[8];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int a = 0; a < G; ++a) {
                k[i][a] = *(const u32x4*)(lds_k + slot * kDmaPlaneStep + i * 2048 + k_lds[a]);
            }
            const u32x4 ks4 = *(const u32x4*)(lds_s + slot * kDmaScaleStep + i * 64 + s_lds);
            const u32x4 vs4 = *(const u32x4*)(lds_s + slot * kDmaScaleStep + 128 + i * 64 + s_lds);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                ksr[i * 4 + r].v = ks4[r];
                vsr[i * 4 + r].v = vs4[r];
            }
        }
        wait_lds_reads();
        if (behind == 2) {
            issue_codes(k_base, lds_k, slot, t_next);
            issue_scales(slot, t_next);
        }
        float pr[8];
        qk_softmax_step<G, SDT, SOFTCAP>(k, ksr, qd, scale_log2, inv_cap, cap_log2, t0, j, first, len, run_max, run_sum, acc, pr);
        wait_vmcnt<behind == 2 ? 14 : behind == 1 ? 9 : 0>();
        unsigned int v[8][G];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                v[i * 4 + r][0] = *(const unsigned int*)(lds_v + slot * kDmaPlaneStep + i * 2048 + v_lds[r]);
                v[i * 4 + r][1] = *(const unsigned int*)(lds_v + slot * kDmaPlaneStep + i * 2048 + (v_lds[r] ^ 64u));
            }
        }
        wait_lds_reads();
        if (behind == 2) {
            issue_codes(v_base, lds_v, slot, t_next);
        }
        clear_hidden_scale_rows<G>(vsr, t0, j, first, len);
        pv_step<G, SDT>(v, vsr, pr, acc);
    };
    using slot0 = std::integral_constant<int, 0>;
    using slot1 = std::integral_constant<int, 1>;
    using behind0 = std::integral_constant<int, 0>;
    using behind1 = std::integral_constant<int, 1>;
    using behind2 = std::integral_constant<int, 2>;

    unsigned int n = 0;
    for (; n + 4u <= steps; n += 2u) { // both steps have two more behind them
        step(slot0{}, behind2{}, n);
        step(slot1{}, behind2{}, n + 1u);
    }
    const unsigned int rest = steps - n; // 1 (a one-step split), 2 or 3
    if (rest == 3u) {
        step(slot0{}, behind2{}, n);
        step(slot1{}, behind1{}, n + 1u);
        step(slot0{}, behind0{}, n + 2u);
    } else if (rest == 2u) {
        step(slot0{}, behind1{}, n);
        step(slot1{}, behind0{}, n + 1u);
    } else {
        step(slot0{}, behind1{}, n); // the prologue's second batch (a repeat of the first) is still behind it
    }
    wait_vmcnt<0>(); // no load may still be writing this workgroup's LDS when the wave ends

    const float total = wave_sum_16x4(run_sum);
    if (head_valid) {
        if (j == 0) {
            p.stats[stat_index] = run_max;
            p.stats[stat_index + 1] = total;
        }
        float* out = p.partial + ((size_t)row * p.num_heads + head) * D;
#pragma unroll
        for (int a = 0; a < G; ++a) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const f32x4 v = {acc[a * 4 + 0][r], acc[a * 4 + 1][r], acc[a * 4 + 2][r], acc[a * 4 + 3][r]};
                *(f32x4*)(out + a * 64 + 16 * j + 4 * r) = v;
            }
        }
    }
}

// ---- f16 KV (no scales): f16 MFMA, Q and P split into f16 hi + lo -------------------------
template <int D> struct F16Step {
    u32x4 k[2][D / 32];     // K: tile i, k-step ks -> 8 f16 (dims ks*32 + j*8 .. +8)
    u32x4 v[8][D / 128];    // V: token slot s -> D/16 f16 (dims m*(D/16) ..), 16 B units
};

template <int D, bool FAST>
__global__ __launch_bounds__(D > 128 ? 256 : 512) void gqa_decode_f16_partial(GqaDecodeParams p)
{
    static_assert(D % 128 == 0, "f16 KV path supports head_dim 128 and 256");
    constexpr int KS = D / 32;  // QK k-steps
    constexpr int MT = D / 16;  // output M tiles
    constexpr int VU = D / 128; // 16-byte units of V per lane per token
    constexpr float kPScale = 16384.0f; // keeps f16(p) out of the subnormal range
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int m = lane & 15u;
    const unsigned int j = lane >> 4;
    const WaveItem mine = wave_item(p);
    const unsigned int kvh = mine.kvh;
    const unsigned int head_block = mine.head_block;
    unsigned int b, chunk, len, first, span, row;
    if (kvh >= p.num_kv_heads || !locate_split(p, mine.item, threadIdx.x & 63u, b, chunk, len, first, span, row)) {
        return;
    }
    const unsigned int first_al = first & ~31u;
    const unsigned long long c_start64 = (unsigned long long)first_al + (unsigned long long)chunk * span;
    const unsigned int head_in_group = head_block * 16u + m;
    const bool head_valid = head_in_group < p.group;
    const unsigned int head = kvh * p.group + head_in_group;
    const size_t stat_index = ((size_t)row * p.num_heads + head) * 2;
    if (c_start64 >= len) {
        if (head_valid && j == 0) {
            p.stats[stat_index] = kNegInf;
            p.stats[stat_index + 1] = 0.0f;
        }
        return;
    }
    const unsigned int c_start = (unsigned int)c_start64;
    const unsigned int c_end = (unsigned int)min((unsigned long long)len, c_start64 + span);
    const unsigned int steps = (c_end - c_start + 31u) / 32u;

    // Q: per-head power-of-two normalisation keeps q inside the f16 range; hi + lo split.  The lane's 8 KS elements
    // (k-step ks -> dims ks*32 + j*8 .. +8) are fetched as 16-byte vectors, all requested before the first is used.
    float q_norm = 1.0f;
    Frag qhi[KS], qlo[KS];
    {
        float x[KS][8];
        const size_t q_index = ((size_t)b * p.num_heads + head) * D + j * 8;
        if (!head_valid) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[ks][e] = 0.0f;
                }
            }
        } else if (p.q_dtype == 0) {
            u32x4 raw[KS][2];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                raw[ks][0] = *(const u32x4*)((const float*)p.q + q_index + ks * 32);
                raw[ks][1] = *(const u32x4*)((const float*)p.q + q_index + ks * 32 + 4);
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[ks][e] = __uint_as_float(raw[ks][e >> 2][e & 3]);
                }
            }
        } else {
            u32x4 raw[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                raw[ks] = *(const u32x4*)((const unsigned short*)p.q + q_index + ks * 32);
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const unsigned int word = raw[ks][e >> 1];
                    const unsigned short bits = (unsigned short)((e & 1) ? (word >> 16) : (word & 0xffffu));
                    x[ks][e] = p.q_dtype == 1 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits);
                }
            }
        }
        float amax = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                amax = fmaxf(amax, fabsf(x[ks][e]));
            }
        }
        amax = wave_max_16x4(amax);
        if (amax > 0.0f && amax < __builtin_inff()) {
            int ex;
            frexpf(amax, &ex);        // amax = f * 2^ex, f in [0.5, 1)
            q_norm = ldexpf(1.0f, -ex); // |q| * q_norm < 1
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float scaled = x[ks][e] * q_norm;
                const _Float16 h = (_Float16)scaled;
                qhi[ks].h[e] = h;
                qlo[ks].h[e] = (_Float16)(scaled - (float)h);
            }
        }
    }

    const unsigned int* table = p.tables + (p.table_shared ? 0 : (size_t)b * p.table_stride);
    const unsigned int k_row = p.num_kv_heads * D * 2u; // bytes per cache row
    const unsigned char* k_base = p.k_plane + (size_t)kvh * D * 2u;
    const unsigned char* v_base = p.v_plane + (size_t)kvh * D * 2u;
    const unsigned int block_mask = p.block_tokens - 1u;
    const unsigned int lo_tile = first & ~15u;
    const unsigned int hi_tile = (len - 1u) & ~15u;
    auto tile_row = [&](unsigned int T) __attribute__((always_inline)) -> unsigned long long {
        unsigned int t = min(max(T, lo_tile), hi_tile);
        if (p.ring_capacity != 0) {
            t %= p.ring_capacity;
        }
        const unsigned int entry = p.tables != nullptr ? __builtin_amdgcn_readfirstlane(table[t >> p.block_shift]) : (t >> p.block_shift);
        return ((unsigned long long)entry << p.block_shift) + (t & block_mask);
    };
    auto token_row = [&](unsigned int t) __attribute__((always_inline)) -> unsigned long long {
        t = min(max(t, first), len - 1u);
        return paged_row(p.tables != nullptr ? table : nullptr, t, p.block_tokens, p.ring_capacity);
    };
    auto load_step = [&](F16Step<D>& s, unsigned int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            unsigned long long R = 0;
            if constexpr (FAST) {
                R = tile_row(t0 + 16u * i);
            }
            const unsigned long long rk = FAST ? R + m : token_row(t0 + 16u * i + m);
            const unsigned char* kr = k_base + rk * k_row + j * 16u;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                s.k[i][ks] = *(const u32x4*)(kr + ks * 64);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const unsigned long long row = FAST ? R + 4u * j + r : token_row(t0 + 16u * i + 4u * j + r);
                const unsigned char* vr = v_base + row * k_row + m * (D / 8);
#pragma unroll
                for (int u = 0; u < VU; ++u) {
                    s.v[i * 4 + r][u] = *(const u32x4*)(vr + u * 16);
                }
            }
        }
    };

    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    float run_max = kNegInf;
    float run_sum = 0.0f;
    const float scale_eff = (p.softcap > 0.0f ? p.score_scale : p.score_scale * kLog2e) / q_norm;
    const float cap_log2 = p.softcap * kLog2e;
    const float tanh_arg = p.softcap > 0.0f ? scale_eff * (2.0f * kLog2e) / p.softcap : 0.0f; // raw product -> 2 y log2(e), y = score / cap

    auto compute_step = [&](F16Step<D>& s, unsigned int t0) __attribute__((always_inline)) {
        if (FAST && (t0 < first || t0 + 32u > len)) {
            // whole tiles are loaded: a slot outside [first, len) holds whatever its page does, and 0 * NaN would
            // poison the head -- such slots multiply as zeros (edge steps only, wave-uniform test)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const unsigned int token = t0 + 16u * (e >> 2) + 4u * j + (e & 3);
                if (token < first || token >= len) {
#pragma unroll
                    for (int u = 0; u < VU; ++u) {
                        s.v[e][u] = u32x4{0u, 0u, 0u, 0u};
                    }
                }
            }
        }
        float sc[8];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            f32x4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                Frag kf;
                kf.u = s.k[i][ks];
                d = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf.h, qhi[ks].h, d, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf.h, qlo[ks].h, d, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float x = d[r] * scale_eff;
                if (p.softcap > 0.0f) {
                    x = p.softcap < kSmallCap ? cap_log2 * tanh_of_exponent(d[r] * tanh_arg) : cap_log2 * fast_tanh(x / p.softcap);
                }
                const unsigned int token = t0 + 16u * i + 4u * j + r;
                sc[i * 4 + r] = (token >= first && token < len) ? x : kNegInf;
            }
        }
        float step_max = sc[0];
#pragma unroll
        for (int e = 1; e < 8; ++e) {
            step_max = fmaxf(step_max, sc[e]);
        }
        step_max = wave_max_16x4(step_max);
        const float new_max = fmaxf(run_max, step_max);
        const float safe_max = new_max == kNegInf ? 0.0f : new_max;
        const float alpha = __builtin_amdgcn_exp2f(run_max - safe_max);
        float pr[8];
        float step_sum = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            pr[e] = __builtin_amdgcn_exp2f(sc[e] - safe_max);
            step_sum += pr[e];
        }
        run_sum = run_sum * alpha + step_sum;
        run_max = new_max;
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                acc[t] *= alpha;
            }
        }
        Frag phi, plo;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = pr[e] * kPScale;
            const _Float16 h = (_Float16)x;
            phi.h[e] = h;
            plo.h[e] = (_Float16)(x - (float)h);
        }
        // V^T fragments: element t of the lane's D/16 dims, across the 8 token slots
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int u = t / 8;         // which 16-byte unit
            const int w = (t % 8) / 2;   // dword inside the unit
            const bool upper = (t & 1) != 0;
            Frag vf;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const unsigned int a0 = s.v[2 * c][u][w];
                const unsigned int a1 = s.v[2 * c + 1][u][w];
                vf.u[c] = upper ? __builtin_amdgcn_perm(a1, a0, 0x07060302u) : __builtin_amdgcn_perm(a1, a0, 0x05040100u);
            }
            f32x4 d = acc[t];
            d = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf.h, phi.h, d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf.h, plo.h, d, 0, 0, 0);
            acc[t] = d;
        }
    };

    F16Step<D> buf0, buf1;
    load_step(buf0, c_start);
    unsigned int step = 0;
    while (true) {
        const unsigned int t0 = c_start + step * 32u;
        if (step + 1 < steps) {
            load_step(buf1, t0 + 32u);
        }
        compute_step(buf0, t0);
        if (++step >= steps) {
            break;
        }
        if (step + 1 < steps) {
            load_step(buf0, t0 + 64u);
        }
        compute_step(buf1, t0 + 32u);
        if (++step >= steps) {
            break;
        }
    }

    const float total = wave_sum_16x4(run_sum);
    if (head_valid) {
        if (j == 0) {
            p.stats[stat_index] = run_max;
            p.stats[stat_index + 1] = total;
        }
        float* out = p.partial + ((size_t)row * p.num_heads + head) * D;
        // tile t, register r holds dim (4*j + r) * (D/16) + t ; undo the P scaling
#pragma unroll
        for (int t = 0; t < MT; ++t) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                out[(4 * j + r) * (D / 16) + t] = acc[t][r] * (1.0f / kPScale);
            }
        }
    }
}

// Where a merge finds the records of record group `b`: `base` is its first row, `last` the largest split index whose
// address may be formed (loads are issued before the split count is known and clamped to it).  Densely numbered records
// start at the row the group's first split left in first_rows; a group without splits never wrote its entry, so what is
// read there is clamped into the arrays and never used.
__device__ __forceinline__ void merge_rows(const GqaDecodeParams& p, unsigned int b, size_t& base, unsigned int& last)
{
    base = (size_t)b * p.max_chunks;
    last = p.max_chunks - 1u;
    if (p.record_rows != 0u) {
        const unsigned int first = min(p.first_rows[b], p.record_rows - 1u);
        base = first;
        last = min(last, p.record_rows - 1u - first);
    }
}

// ---- split combine by log-sum-exp ---------------------------------------------------------
// out[b, head, :] = sum_c partial_c * 2^(m_c - m) / sum_c l_c * 2^(m_c - m); zero when nothing
// was visible.  Same algebra as gqa_decode_merge_f32
// (src/kernel/rocm/hip/tensor/attention/source.hip:1339-1362), in base 2.
__global__ __launch_bounds__(256) void gqa_decode_merge(GqaDecodeParams p)
{
    // one workgroup per (head, sequence): threads = (dim quad) x (split lane); every split lane folds
    // its share of the splits with independent loads, then the lanes are combined through LDS.
    const unsigned int quads = p.head_dim / 4u;
    const unsigned int lanes = 256u / quads;
    const unsigned int quad = threadIdx.x % quads;
    const unsigned int sl = threadIdx.x / quads;
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    unsigned int chunks = p.fixed_chunks;
    if (chunks == 0u) {
        unsigned int len = p.kv_lens[b];
        if (p.query_rows > 1u) { // record row b of a multi-row call: its sequence's length less the chunk rows after it
            const unsigned int behind = p.query_rows - 1u - b % p.query_rows;
            len = p.kv_lens[b / p.query_rows];
            len = len > behind ? len - behind : 0u;
        }
        unsigned int first = p.first_visible != nullptr ? p.first_visible[b] : 0u;
        first = min(first, len);
        const unsigned int first_al = first & ~31u;
        chunks = min(p.max_chunks, (len - first_al + p.chunk_tokens - 1u) / p.chunk_tokens);
    }
    if (sl >= lanes) {
        chunks = 0u; // a width whose quads do not divide the workgroup leaves its last threads without a share
    }
    size_t base;
    unsigned int last;
    merge_rows(p, b, base, last);
    const float* stats = p.stats + (base * p.num_heads + head) * 2;
    const size_t stat_stride = (size_t)p.num_heads * 2;
    const float* partial = p.partial + (base * p.num_heads + head) * p.head_dim + quad * 4u;
    const size_t partial_stride = (size_t)p.num_heads * p.head_dim;

    // single pass, four splits per trip with all eight loads issued before any is used
    float m = kNegInf;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float l = 0.0f;
    // Record addresses are clamped to the planned splits, not to this sequence's own count, so that the first trip's
    // loads do not wait for the length: what a dead split's record holds is never used.
    auto fold = [&](unsigned int c0, auto trip_c) __attribute__((always_inline)) {
        constexpr int U = decltype(trip_c)::value;
        float cm[U], cl[U];
        f32x4 part[U];
        float2 st[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned int c = min(c0 + u * lanes, last);
            st[u] = *(const float2*)(stats + c * stat_stride);
            part[u] = *(const f32x4*)(partial + c * partial_stride);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool live = c0 + u * lanes < chunks;
            cm[u] = live ? st[u].x : kNegInf;
            cl[u] = live ? st[u].y : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (cl[u] > 0.0f) {
                const float nm = fmaxf(m, cm[u]);
                const float a = __builtin_amdgcn_exp2f(m - nm); // m = -inf -> 0
                const float w = __builtin_amdgcn_exp2f(cm[u] - nm);
                acc = acc * a + part[u] * w;
                l = l * a + cl[u] * w;
                m = nm;
            }
        }
    };
    // the first trip runs whatever the split count is (its loads do not wait for the length); a trip is one round trip
    // to memory, so a plan with many short splits (few KV heads, short contexts) takes eight records per trip from the start
    unsigned int next = sl;
    if (p.max_chunks > 4u * lanes) {
        fold(next, std::integral_constant<int, 8>{});
        next += 8u * lanes;
    } else {
        fold(next, std::integral_constant<int, 4>{});
        next += 4u * lanes;
    }
    for (unsigned int c0 = next; c0 < chunks; c0 += 8u * lanes) {
        fold(c0, std::integral_constant<int, 8>{});
    }
    __shared__ float sm[256];
    __shared__ float sl_sum[256];
    __shared__ f32x4 sacc[256];
    sm[threadIdx.x] = m;
    sl_sum[threadIdx.x] = l;
    sacc[threadIdx.x] = acc;
    __syncthreads();
    if (sl == 0) {
        float gm = kNegInf;
        for (unsigned int i = 0; i < lanes; ++i) {
            gm = fmaxf(gm, sm[i * quads + quad]);
        }
        const float safe_g = gm == kNegInf ? 0.0f : gm;
        f32x4 total = {0.f, 0.f, 0.f, 0.f};
        float denom = 0.0f;
        for (unsigned int i = 0; i < lanes; ++i) {
            const float li = sl_sum[i * quads + quad];
            if (li > 0.0f) {
                const float w = __builtin_amdgcn_exp2f(sm[i * quads + quad] - safe_g);
                denom += li * w;
                total += sacc[i * quads + quad] * w;
            }
        }
        f32x4 result = {0.f, 0.f, 0.f, 0.f};
        if (denom > 0.0f && denom < __builtin_inff()) {
            result = total * (1.0f / denom);
        }
        if (p.gate != nullptr) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                result[e] = gated(result[e], p.gate, p.gate_cols, p.gate_dtype, b, head * p.head_dim + quad * 4u + e);
            }
        }
        const size_t at = ((size_t)b * p.num_heads + head) * p.head_dim + quad * 4u;
        if (p.out_dtype == 0) {
            *(f32x4*)(p.out + at) = result;
        } else if (p.out_dtype == 1) {
            *(u32x2*)((unsigned short*)p.out + at) = u32x2{pack_bf16_rne(result[0], result[1]), pack_bf16_rne(result[2], result[3])};
        } else {
            *(u32x2*)((unsigned short*)p.out + at) = u32x2{(unsigned int)f32_to_f16_bits(result[0]) | ((unsigned int)f32_to_f16_bits(result[1]) << 16),
                                                            (unsigned int)f32_to_f16_bits(result[2]) | ((unsigned int)f32_to_f16_bits(result[3]) << 16)};
        }
    }
}

// The merge for a call of few rows cut into hundreds of splits (one sequence alone on the GPU gets a split per compute
// unit and KV-head block: 256 or 512 records per head).  One workgroup per (row, head) folds them in four to eight
// dependent round trips on as many compute units as the call has heads, and a single thread per column quad then walks
// the split lanes' results in LDS.  Here a workgroup takes 32 columns of a (row, head): 256 threads = 32 split lanes x 8
// column quads, eight records per lane and trip (256 splits: one round trip, requested before the sequence length is
// known), the eight lanes of a quad inside a wave meet through lane exchanges and the four waves through LDS.
// grid = (heads, rows, head_dim / 32).
__global__ __launch_bounds__(256) void gqa_decode_merge_wide(GqaDecodeParams p)
{
    const unsigned int head = blockIdx.x;
    const unsigned int b = blockIdx.y;
    const unsigned int quad = threadIdx.x & 7u;
    const unsigned int sl = threadIdx.x >> 3;
    const unsigned int column = blockIdx.z * 32u + quad * 4u;
    size_t base;
    unsigned int last;
    merge_rows(p, b, base, last);
    const float* stats = p.stats + (base * p.num_heads + head) * 2;
    const size_t stat_stride = (size_t)p.num_heads * 2;
    const float* partial = p.partial + (base * p.num_heads + head) * p.head_dim + column;
    const size_t partial_stride = (size_t)p.num_heads * p.head_dim;
    // first trip: addresses clamped to the planned splits, so the loads do not wait for the length
    float2 st[8];
    f32x4 part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const unsigned int c = min(sl + 32u * u, last);
        st[u] = *(const float2*)(stats + c * stat_stride);
        part[u] = *(const f32x4*)(partial + c * partial_stride);
    }
    unsigned int chunks = p.fixed_chunks;
    if (chunks == 0u) {
        unsigned int len = p.kv_lens[b];
        if (p.query_rows > 1u) { // record row b of a multi-row call: its sequence's length less the chunk rows after it
            const unsigned int behind = p.query_rows - 1u - b % p.query_rows;
            len = p.kv_lens[b / p.query_rows];
            len = len > behind ? len - behind : 0u;
        }
        unsigned int first = p.first_visible != nullptr ? p.first_visible[b] : 0u;
        first = min(first, len);
        const unsigned int first_al = first & ~31u;
        chunks = min(p.max_chunks, (len - first_al + p.chunk_tokens - 1u) / p.chunk_tokens);
    }
    float m = kNegInf, l = 0.0f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (unsigned int c0 = sl;; c0 += 256u) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (c0 + 32u * u < chunks && st[u].y > 0.0f) {
                const float nm = fmaxf(m, st[u].x);
                const float a = __builtin_amdgcn_exp2f(m - nm); // m = -inf -> 0
                const float w = __builtin_amdgcn_exp2f(st[u].x - nm);
                acc = acc * a + part[u] * w;
                l = l * a + st[u].y * w;
                m = nm;
            }
        }
        if (c0 - sl + 256u >= chunks) { // the same for every thread of the workgroup
            break;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const unsigned int c = min(c0 + 256u + 32u * u, last);
            st[u] = *(const float2*)(stats + c * stat_stride);
            part[u] = *(const f32x4*)(partial + c * partial_stride);
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
#pragma unroll
    for (int step = 8; step <= 32; step *= 2) {
        const float om = __shfl_xor(m, step), ol = __shfl_xor(l, step);
        const f32x4 oacc = {__shfl_xor(acc[0], step), __shfl_xor(acc[1], step), __shfl_xor(acc[2], step), __shfl_xor(acc[3], step)};
        fold(m, l, acc, om, ol, oacc);
    }
    __shared__ float wave_m[4][8], wave_l[4][8];
    __shared__ f32x4 wave_acc[4][8];
    if ((threadIdx.x & 63u) < 8u) {
        wave_m[threadIdx.x >> 6][quad] = m;
        wave_l[threadIdx.x >> 6][quad] = l;
        wave_acc[threadIdx.x >> 6][quad] = acc;
    }
    __syncthreads();
    if (threadIdx.x < 8u) {
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            fold(m, l, acc, wave_m[w][quad], wave_l[w][quad], wave_acc[w][quad]);
        }
        f32x4 result = {0.f, 0.f, 0.f, 0.f};
        if (l > 0.0f && l < __builtin_inff()) {
            result = acc * (1.0f / l);
        }
        if (p.gate != nullptr) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                result[e] = gated(result[e], p.gate, p.gate_cols, p.gate_dtype, b, head * p.head_dim + column + e);
            }
        }
        const size_t at = ((size_t)b * p.num_heads + head) * p.head_dim + column;
        if (p.out_dtype == 0) {
            *(f32x4*)(p.out + at) = result;
        } else if (p.out_dtype == 1) {
            *(u32x2*)((unsigned short*)p.out + at) = u32x2{pack_bf16_rne(result[0], result[1]), pack_bf16_rne(result[2], result[3])};
        } else {
            *(u32x2*)((unsigned short*)p.out + at) = u32x2{(unsigned int)f32_to_f16_bits(result[0]) | ((unsigned int)f32_to_f16_bits(result[1]) << 16),
                                                            (unsigned int)f32_to_f16_bits(result[2]) | ((unsigned int)f32_to_f16_bits(result[3]) << 16)};
        }
    }
}

// The combine for plans of nine to thirty-two splits at head_dim 128 -- a batch of long sequences cut into one round of
// workgroups, config 2's own plan: one wave per (head, sequence), a lane owns four output dimensions and every other
// split, all sixteen record loads of the lane issued before the first is used, the two halves of the wave combined with
// one lane exchange.  No LDS and no barrier: the kernel is one memory round trip, the exchange and the store.
__global__ __launch_bounds__(256) void gqa_decode_merge_wave(GqaDecodeParams p)
{
    const unsigned int lane = threadIdx.x & 63u;
    const unsigned int quad = lane & 31u;
    const unsigned int sl = lane >> 5;
    const unsigned int head = blockIdx.x * 4u + (threadIdx.x >> 6);
    const unsigned int b = blockIdx.y;
    if (head >= p.num_heads) {
        return;
    }
    size_t base;
    unsigned int last;
    merge_rows(p, b, base, last);
    const float* stats = p.stats + (base * p.num_heads + head) * 2;
    const size_t stat_stride = (size_t)p.num_heads * 2;
    const float* partial = p.partial + (base * p.num_heads + head) * 128u + quad * 4u;
    const size_t partial_stride = (size_t)p.num_heads * 128u;
    // addresses are clamped to the planned splits, so that the loads do not wait for the length
    float2 st[16];
    f32x4 part[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const unsigned int c = min(sl + 2u * u, last);
        st[u] = *(const float2*)(stats + c * stat_stride);
        part[u] = *(const f32x4*)(partial + c * partial_stride);
    }
    unsigned int chunks = p.fixed_chunks;
    if (chunks == 0u) {
        unsigned int len = p.kv_lens[b];
        if (p.query_rows > 1u) {
            const unsigned int behind = p.query_rows - 1u - b % p.query_rows;
            len = p.kv_lens[b / p.query_rows];
            len = len > behind ? len - behind : 0u;
        }
        unsigned int first = p.first_visible != nullptr ? p.first_visible[b] : 0u;
        first = min(first, len);
        const unsigned int first_al = first & ~31u;
        chunks = min(p.max_chunks, (len - first_al + p.chunk_tokens - 1u) / p.chunk_tokens);
    }
    float m = kNegInf, l = 0.0f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const float cl = sl + 2u * u < chunks ? st[u].y : 0.0f;
        if (cl > 0.0f) {
            const float nm = fmaxf(m, st[u].x);
            const float a = __builtin_amdgcn_exp2f(m - nm); // m = -inf -> 0
            const float w = __builtin_amdgcn_exp2f(st[u].x - nm);
            acc = acc * a + part[u] * w;
            l = l * a + cl * w;
            m = nm;
        }
    }
    // the other half of the wave holds the other splits of the same four dimensions
    const float om = __shfl_xor(m, 32), ol = __shfl_xor(l, 32);
    const f32x4 oacc = {__shfl_xor(acc[0], 32), __shfl_xor(acc[1], 32), __shfl_xor(acc[2], 32), __shfl_xor(acc[3], 32)};
    if (sl != 0u) {
        return;
    }
    const float gm = fmaxf(l > 0.0f ? m : kNegInf, ol > 0.0f ? om : kNegInf);
    const float wa = l > 0.0f ? __builtin_amdgcn_exp2f(m - gm) : 0.0f;
    const float wb = ol > 0.0f ? __builtin_amdgcn_exp2f(om - gm) : 0.0f;
    const float denom = l * wa + ol * wb;
    f32x4 result = {0.f, 0.f, 0.f, 0.f};
    if (denom > 0.0f && denom < __builtin_inff()) {
        result = (acc * wa + oacc * wb) * (1.0f / denom);
    }
    if (p.gate != nullptr) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            result[e] = gated(result[e], p.gate, p.gate_cols, p.gate_dtype, b, head * 128u + quad * 4u + e);
        }
    }
    const size_t at = ((size_t)b * p.num_heads + head) * 128u + quad * 4u;
    if (p.out_dtype == 0) {
        *(f32x4*)(p.out + at) = result;
    } else if (p.out_dtype == 1) {
        *(u32x2*)((unsigned short*)p.out + at) = u32x2{pack_bf16_rne(result[0], result[1]), pack_bf16_rne(result[2], result[3])};
    } else {
        *(u32x2*)((unsigned short*)p.out + at) = u32x2{(unsigned int)f32_to_f16_bits(result[0]) | ((unsigned int)f32_to_f16_bits(result[1]) << 16),
                                                        (unsigned int)f32_to_f16_bits(result[2]) | ((unsigned int)f32_to_f16_bits(result[3]) << 16)};
    }
}

// The same combine for plans of at most eight splits (large batches, short contexts): a thread owns four output
// dimensions of one (head, sequence) and folds the few records itself, 256 / (head_dim / 4) heads a workgroup.  One
// workgroup of 256 threads per (head, sequence) is mostly idle lanes there, and with hundreds of sequences the launch
// of tens of thousands of them costs more than the combine (512 sequences x 64 heads, two splits: 37 us, 10 us here).
__global__ __launch_bounds__(256) void gqa_decode_merge_few(GqaDecodeParams p)
{
    const unsigned int quads = p.head_dim / 4u;
    const unsigned int heads_here = 256u / quads;
    const unsigned int quad = threadIdx.x % quads;
    const unsigned int head = blockIdx.x * heads_here + threadIdx.x / quads;
    const unsigned int b = blockIdx.y;
    if (head >= p.num_heads) {
        return;
    }
    unsigned int chunks = p.fixed_chunks;
    if (chunks == 0u) {
        unsigned int len = p.kv_lens[b];
        if (p.query_rows > 1u) {
            const unsigned int behind = p.query_rows - 1u - b % p.query_rows;
            len = p.kv_lens[b / p.query_rows];
            len = len > behind ? len - behind : 0u;
        }
        unsigned int first = p.first_visible != nullptr ? p.first_visible[b] : 0u;
        first = min(first, len);
        const unsigned int first_al = first & ~31u;
        chunks = min(p.max_chunks, (len - first_al + p.chunk_tokens - 1u) / p.chunk_tokens);
    }
    size_t base;
    unsigned int last;
    merge_rows(p, b, base, last);
    const float* stats = p.stats + (base * p.num_heads + head) * 2;
    const size_t stat_stride = (size_t)p.num_heads * 2;
    const float* partial = p.partial + (base * p.num_heads + head) * p.head_dim + quad * 4u;
    const size_t partial_stride = (size_t)p.num_heads * p.head_dim;
    float m = kNegInf, l = 0.0f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (unsigned int c0 = 0; c0 == 0u || c0 < chunks; c0 += 4u) { // the first trip's loads do not wait for the length
        float2 st[4];
        f32x4 part[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const unsigned int c = min(c0 + u, last);
            st[u] = *(const float2*)(stats + c * stat_stride);
            part[u] = *(const f32x4*)(partial + c * partial_stride);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float cl = c0 + u < chunks ? st[u].y : 0.0f;
            if (cl > 0.0f) {
                const float nm = fmaxf(m, st[u].x);
                const float a = __builtin_amdgcn_exp2f(m - nm); // m = -inf -> 0
                const float w = __builtin_amdgcn_exp2f(st[u].x - nm);
                acc = acc * a + part[u] * w;
                l = l * a + cl * w;
                m = nm;
            }
        }
    }
    f32x4 result = {0.f, 0.f, 0.f, 0.f};
    if (l > 0.0f && l < __builtin_inff()) {
        result = acc * (1.0f / l);
    }
    if (p.gate != nullptr) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            result[e] = gated(result[e], p.gate, p.gate_cols, p.gate_dtype, b, head * p.head_dim + quad * 4u + e);
        }
    }
    const size_t at = ((size_t)b * p.num_heads + head) * p.head_dim + quad * 4u;
    if (p.out_dtype == 0) {
        *(f32x4*)(p.out + at) = result;
    } else if (p.out_dtype == 1) {
        *(u32x2*)((unsigned short*)p.out + at) = u32x2{pack_bf16_rne(result[0], result[1]), pack_bf16_rne(result[2], result[3])};
    } else {
        *(u32x2*)((unsigned short*)p.out + at) = u32x2{(unsigned int)f32_to_f16_bits(result[0]) | ((unsigned int)f32_to_f16_bits(result[1]) << 16),
                                                        (unsigned int)f32_to_f16_bits(result[2]) | ((unsigned int)f32_to_f16_bits(result[3]) << 16)};
    }
}

// Visible ranges of the rows of a prefill chunk, for the route that runs every row as one item of the split-KV
// decode kernels: lens[r] = end and first[r] = start of key_range(position + r, position + rows), or of
// key_range_with_visible_end when the row carries an explicit end (src/attention/gqa.rs:54-68).
__global__ __launch_bounds__(256) void prefill_row_ranges(unsigned int* lens, unsigned int* first, const unsigned int* visible_ends,
                                                          const unsigned int* visible_starts, unsigned int rows, unsigned int position,
                                                          unsigned int window)
{
    const unsigned int r = blockIdx.x * 256u + threadIdx.x;
    if (r >= rows) {
        return;
    }
    const unsigned int pos = position + r;
    unsigned int end = pos + 1u;
    const unsigned int start = (window != 0 && end > window) ? end - window : 0u;
    if (visible_starts != nullptr) { // an explicit range (BlockAttentionSpec::visible, src/attention/block.rs:10-16): taken as given
        const unsigned int given_end = min(visible_ends[r], position + rows);
        lens[r] = given_end;
        first[r] = min(visible_starts[r], given_end);
        return;
    }
    if (visible_ends != nullptr) {
        end = min(max(end, visible_ends[r]), position + rows);
    }
    lens[r] = end;
    first[r] = min(start, end);
}

template <int D, int SDT>
hipError_t launch_q8(const GqaDecodeParams& p, bool fast, dim3 grid, dim3 block, hipStream_t stream)
{
    const bool cap = p.softcap > 0.0f;
    if constexpr (D == 128) {
        // direct-to-LDS pipeline: needs the whole split's block-table entries in two registers (128 pages)
        if (fast && p.ring_capacity == 0 && p.chunk_tokens <= 127u * p.block_tokens && block.x <= 64u * kDmaWaves) {
            if (cap) {
                gqa_decode_q8_dma128<SDT, true><<<grid, block, 0, stream>>>(p);
            } else {
                gqa_decode_q8_dma128<SDT, false><<<grid, block, 0, stream>>>(p);
            }
            return hipGetLastError();
        }
    }
    if constexpr (D != 192) { // three scale words a row do not travel as one register: head_dim 192 loads them per token
        if (fast) {
            if (cap) {
                gqa_decode_q8_partial<D, SDT, true, true, 2><<<grid, block, 0, stream>>>(p);
            } else {
                gqa_decode_q8_partial<D, SDT, true, false, 2><<<grid, block, 0, stream>>>(p);
            }
            return hipGetLastError();
        }
    }
    {
        if (cap) {
            gqa_decode_q8_partial<D, SDT, false, true, 2><<<grid, block, 0, stream>>>(p);
        } else {
            gqa_decode_q8_partial<D, SDT, false, false, 2><<<grid, block, 0, stream>>>(p);
        }
    }
    return hipGetLastError();
}

template <int D> hipError_t launch_q8_d(const GqaDecodeParams& p, int scale_dtype, bool fast, dim3 grid, dim3 block, hipStream_t stream)
{
    if (scale_dtype == 2) {
        // f32 scales: every lane fetches the scale rows of its token slots itself (the tile paths move 16-bit scales)
        if (p.softcap > 0.0f) {
            gqa_decode_q8_partial<D, 2, false, true, 2><<<grid, block, 0, stream>>>(p);
        } else {
            gqa_decode_q8_partial<D, 2, false, false, 2><<<grid, block, 0, stream>>>(p);
        }
        return hipGetLastError();
    }
    if (scale_dtype == 0) {
        return launch_q8<D, 0>(p, fast, grid, block, stream);
    }
    return launch_q8<D, 1>(p, fast, grid, block, stream);
}

} // namespace

unsigned int gqa_decode_max_waves(unsigned int head_dim)
{
    return head_dim > 128u ? 4u : 8u; // head_dim 256 needs the larger register file share
}

unsigned int gqa_decode_items_per_group(unsigned int head_dim, unsigned int num_kv_heads)
{
    // four waves keep a CU's loads flowing (measured with four KV heads: 5.8 TB/s); more items than that only add
    // partial records for the merge.  waves x items never passes the kernels' launch bound (gqa_decode_max_waves
    // waves): three KV heads of head_dim 256 are three of the four waves a workgroup may have, so they run one item.
    const unsigned int max_waves = gqa_decode_max_waves(head_dim);
    const unsigned int waves = num_kv_heads < max_waves ? num_kv_heads : max_waves;
    const unsigned int wanted = num_kv_heads < 4u ? (num_kv_heads == 1u ? 4u : 2u) : 1u;
    const unsigned int fit = max_waves / waves;
    return wanted < fit ? wanted : fit;
}

hipError_t launch_gqa_decode(const GqaDecodeParams& args, int kv_format, int scale_dtype, unsigned int stages, hipStream_t stream)
{
    GqaDecodeParams p = args;
    const unsigned int max_waves = gqa_decode_max_waves(p.head_dim);
    const unsigned int waves = p.num_kv_heads < max_waves ? p.num_kv_heads : max_waves;
    const unsigned int kvh_blocks = (p.num_kv_heads + waves - 1) / waves;
    const unsigned int head_blocks = (p.group + 15u) / 16u;
    p.items_per_group = gqa_decode_items_per_group(p.head_dim, p.num_kv_heads);
    // densely numbered records are sized for the live splits: no workgroups beyond them
    const unsigned int items = p.record_rows != 0u ? p.record_rows : p.max_chunks * p.batch;
    const dim3 grid((items + p.items_per_group - 1u) / p.items_per_group, kvh_blocks * head_blocks, 1);
    const dim3 block(waves * p.items_per_group * 64u);
    const bool pow2 = (p.block_tokens & (p.block_tokens - 1u)) == 0;
    const bool fast = pow2 && p.block_tokens >= 16u && p.ring_capacity % 16u == 0;
    hipError_t err = hipSuccess;
    if (stages == 2u) {
        // merge only
    } else if (kv_format == 0) {
        switch (p.head_dim) {
        case 64: err = launch_q8_d<64>(p, scale_dtype, fast, grid, block, stream); break;
        case 128: err = launch_q8_d<128>(p, scale_dtype, fast, grid, block, stream); break;
        case 192: err = launch_q8_d<192>(p, scale_dtype, fast, grid, block, stream); break;
        case 256: err = launch_q8_d<256>(p, scale_dtype, fast, grid, block, stream); break;
        default: return hipErrorInvalidValue;
        }
    } else {
        if (p.head_dim == 128) {
            if (fast) {
                gqa_decode_f16_partial<128, true><<<grid, block, 0, stream>>>(p);
            } else {
                gqa_decode_f16_partial<128, false><<<grid, block, 0, stream>>>(p);
            }
        } else if (p.head_dim == 256) {
            if (fast) {
                gqa_decode_f16_partial<256, true><<<grid, block, 0, stream>>>(p);
            } else {
                gqa_decode_f16_partial<256, false><<<grid, block, 0, stream>>>(p);
            }
        } else {
            return hipErrorInvalidValue;
        }
        err = hipGetLastError();
    }
    if (err != hipSuccess || stages == 1u) {
        return err;
    }
    return launch_split_merge(p, stream);
}

hipError_t launch_prefill_row_ranges(unsigned int* lens, unsigned int* first, const unsigned int* visible_ends, const unsigned int* visible_starts,
                                     unsigned int rows, unsigned int position, unsigned int window, hipStream_t stream)
{
    prefill_row_ranges<<<dim3((rows + 255u) / 256u), dim3(256), 0, stream>>>(lens, first, visible_ends, visible_starts, rows, position, window);
    return hipGetLastError();
}

hipError_t launch_split_merge(const GqaDecodeParams& p, hipStream_t stream)
{
    const unsigned int quads = p.head_dim / 4u;
    if (p.max_chunks <= 8u && quads <= 256u && 256u % quads == 0u) {
        const unsigned int heads_here = 256u / quads;
        gqa_decode_merge_few<<<dim3((p.num_heads + heads_here - 1u) / heads_here, p.batch), dim3(256), 0, stream>>>(p);
    } else if (p.head_dim % 32u == 0u && ((p.max_chunks > 8u * (256u / quads) && p.num_heads * p.batch <= 512u) ||
                                          (p.max_chunks > 4u * (256u / quads) && p.num_heads * p.batch <= 256u))) {
        // more splits than one workgroup per (row, head) reads in a round trip, and few such pairs
        gqa_decode_merge_wide<<<dim3(p.num_heads, p.batch, p.head_dim / 32u), dim3(256), 0, stream>>>(p);
    } else if (p.head_dim == 128u && p.max_chunks <= 32u) {
        gqa_decode_merge_wave<<<dim3((p.num_heads + 3u) / 4u, p.batch), dim3(256), 0, stream>>>(p);
    } else {
        gqa_decode_merge<<<dim3(p.num_heads, p.batch), dim3(256), 0, stream>>>(p);
    }
    return hipGetLastError();
}

} // namespace zllm

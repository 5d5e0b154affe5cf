// Query rows, KV splits and split record rows of the MLA decode kernels: shared by the partial kernels and the merges.
#pragma once

#include "common.hpp"
#include "kernels.hpp"

namespace zllm {

// Query row v of the call: its sequence and the number of tokens it sees.  With query_rows > 1 the rows of a
// sequence are the last query_rows tokens of its context, each seeing everything up to and including itself
// (src/kernel/cpu/mla.rs:1016-1018: row r of a chunk at query_start sees query_start + r + 1 tokens).
__device__ __forceinline__ unsigned int visible_tokens(const unsigned int* ctx_lens, unsigned int query_rows, unsigned int v, unsigned int& sequence)
{
    sequence = v / query_rows;
    const unsigned int behind = query_rows - 1u - v % query_rows; // rows of the chunk after this one
    const unsigned int len = ctx_lens[sequence];
    return len > behind ? len - behind : 0u;
}

// Densely numbered split records (record_rows != 0; never together with a selection): work item `item` is split
// `chunk` of query row `b`, rows in order, each with min(max_chunks, ceil(tokens / chunk_tokens)) splits; the item number
// is also the record row.  Every wave of the workgroup runs the same prefix sum over the rows' split counts.  The first
// split of a row leaves its item number in first_rows for the merge; items past the last live split, and past the rows
// the host sized, find nothing.
__device__ __forceinline__ bool mla_locate_split(const MlaDecodeParams& p, unsigned int item, unsigned int lane, unsigned int& b_out,
                                                 unsigned int& chunk_out)
{
    if (item >= p.record_rows) {
        return false;
    }
    unsigned int base = 0;
    for (unsigned int b0 = 0; b0 < p.batch; b0 += 64u) {
        const unsigned int v = b0 + lane;
        unsigned int n = 0;
        if (v < p.batch) {
            unsigned int seq;
            const unsigned int len = visible_tokens(p.ctx_lens, p.query_rows, v, seq);
            n = min(p.max_chunks, (len + p.chunk_tokens - 1u) / p.chunk_tokens);
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
            if (chunk_out == 0u && lane == 0u) {
                p.first_rows[b_out] = item; // every wave, and every head block, writes the same number
            }
            return true;
        }
        base += total;
    }
    return false;
}

// Where a merge finds the records of query row `b`: its first record row, and its split count cut to the rows there are
// (a row whose first split was dropped never wrote its entry: what is read there is clamped into the arrays).
__device__ __forceinline__ size_t mla_merge_base(const MlaDecodeParams& p, unsigned int b, unsigned int& chunks)
{
    if (p.record_rows == 0u) {
        return (size_t)b * p.max_chunks;
    }
    const unsigned int first = min(p.first_rows[b], p.record_rows - 1u);
    chunks = min(chunks, p.record_rows - first);
    return first;
}

} // namespace zllm

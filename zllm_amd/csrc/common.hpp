// Shared device helpers for the gfx950 attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace zllm {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr float kNegInf = -__builtin_inff();

// bf16 <-> f32, bit-compatible with zllm_bf16_to_f32 / zllm_f32_to_bf16
// (src/kernel/rocm/hip/hiprtc.rs:62-75): round-to-nearest-even by adding
// 0x7fff + lsb, NaN not special-cased.
__device__ __forceinline__ float bf16_bits_to_f32(unsigned short v)
{
    return __uint_as_float(((unsigned int)v) << 16);
}

__device__ __forceinline__ unsigned short f32_to_bf16_bits(float value)
{
    const unsigned int bits = __float_as_uint(value);
    const unsigned int rounding = 0x7fffu + ((bits >> 16) & 1u);
    return (unsigned short)((bits + rounding) >> 16);
}

__device__ __forceinline__ float f16_bits_to_f32(unsigned short v)
{
    union {
        unsigned short u;
        _Float16 h;
    } c;
    c.u = v;
    return (float)c.h;
}

__device__ __forceinline__ unsigned short f32_to_f16_bits(float value)
{
    union {
        unsigned short u;
        _Float16 h;
    } c;
    c.h = (_Float16)value; // v_cvt_f16_f32: IEEE round-to-nearest-even
    return c.u;
}

// Stored scale -> f32; numbering of zllm_scale (hiprtc.rs:104-116).
template <int SCALE_DTYPE> __device__ __forceinline__ float scale_bits_to_f32(unsigned short v)
{
    if constexpr (SCALE_DTYPE == 0) {
        return bf16_bits_to_f32(v);
    } else {
        return f16_bits_to_f32(v);
    }
}

__device__ __forceinline__ float load_as_f32(const void* base, size_t index, int dtype)
{
    if (dtype == 0) {
        return ((const float*)base)[index];
    }
    if (dtype == 1) {
        return bf16_bits_to_f32(((const unsigned short*)base)[index]);
    }
    return f16_bits_to_f32(((const unsigned short*)base)[index]);
}

// Logical token -> physical cache row
// (src/kernel/rocm/hip/attention/paged_mla/source.hip:46-54), with the optional
// sliding-window ring applied first (src/kernel/cuda/attention.rs:82-88).
// out * sigmoid(gate): the output gate of a gated attention layer (src/backend/cpu/context.rs:419-432).
// `row` indexes the gate's rows, `column` its columns (ignored when the gate has one column).
__device__ __forceinline__ float gated(float value, const void* gate, unsigned int gate_cols, int gate_dtype, size_t row, unsigned int column)
{
    const float g = load_as_f32(gate, row * gate_cols + (gate_cols == 1u ? 0u : column), gate_dtype);
    return value * (1.0f / (1.0f + __expf(-g)));
}

__device__ __forceinline__ unsigned long long paged_row(const unsigned int* table, unsigned int token,
                                                        unsigned int block_tokens, unsigned int ring_capacity)
{
    if (ring_capacity != 0) {
        token %= ring_capacity;
    }
    if (table == nullptr) {
        return token;
    }
    return (unsigned long long)table[token / block_tokens] * block_tokens + token % block_tokens;
}

// Two f32 -> packed bf16x2 (low half = a).  Truncation is exact for the small
// integers (|x| <= 255) it is used on.
__device__ __forceinline__ unsigned int pack_bf16_trunc(float lo, float hi)
{
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

// Two f32 -> packed bf16x2 with round-to-nearest-even.
__device__ __forceinline__ unsigned int pack_bf16_rne(float lo, float hi)
{
    return (unsigned int)f32_to_bf16_bits(lo) | ((unsigned int)f32_to_bf16_bits(hi) << 16);
}

// Same rounding for finite values, one v_cvt_pk_bf16_f32 (used where NaN payloads do not matter:
// attention probabilities and query fragments, never cache contents).
__device__ __forceinline__ unsigned int pack_bf16_hw(float lo, float hi)
{
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, bf16x2_t));
}

// hi + lo bf16 split of two values: hi = bf16(x), lo = bf16(x - hi); 16 significant bits together.
__device__ __forceinline__ void split_bf16_pair(float x0, float x1, unsigned int& hi, unsigned int& lo)
{
    hi = pack_bf16_hw(x0, x1);
    const float h0 = __uint_as_float(hi << 16);
    const float h1 = __uint_as_float(hi & 0xffff0000u);
    lo = pack_bf16_hw(x0 - h0, x1 - h1);
}

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// two f32 -> packed f16, round to nearest even (v_cvt_pk_f16_f32)
__device__ __forceinline__ unsigned int pack_f16_hw(float lo, float hi)
{
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(f32x2{lo, hi}, f16x2));
}

// Four int8 codes of a word -> four f16 integers (exact), 5 instructions: flipping the sign bits turns a code c
// into the unsigned byte c + 128; placed under the exponent byte 0x64 it reads as the f16 number 1024 + 128 + c,
// and one packed subtraction removes the offset.
__device__ __forceinline__ void codes4_to_f16(unsigned int word, unsigned int& lo, unsigned int& hi)
{
    const unsigned int biased = word ^ 0x80808080u;
    const f16x2 offset = {(_Float16)-1152.0f, (_Float16)-1152.0f};
    lo = __builtin_bit_cast(unsigned int, __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(0x64646464u, biased, 0x04010400u)) + offset);
    hi = __builtin_bit_cast(unsigned int, __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(0x64646464u, biased, 0x04030402u)) + offset);
}

// Reductions across the four 16-lane rows of a wave (lanes l, l^16, l^32, l^48): every lane ends up with
// the result.  v_permlane16_swap / v_permlane32_swap exchange rows inside the vector ALU, so the reduction
// does not take the round trip through the LDS crossbar that a generic lane shuffle does.
typedef unsigned int u32x2_swap __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float wave_max_16x4(float v)
{
    const unsigned int bits = __float_as_uint(v);
    // swap odd rows of the first copy with even rows of the second: {r0, r0, r2, r2} and {r1, r1, r3, r3}
    const u32x2_swap a = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    const float m = fmaxf(__uint_as_float(a.x), __uint_as_float(a.y));
    const unsigned int mbits = __float_as_uint(m);
    // swap the upper half of the first copy with the lower half of the second
    const u32x2_swap b = __builtin_amdgcn_permlane32_swap(mbits, mbits, false, false);
    return fmaxf(__uint_as_float(b.x), __uint_as_float(b.y));
}

__device__ __forceinline__ float wave_sum_16x4(float v)
{
    const unsigned int bits = __float_as_uint(v);
    const u32x2_swap a = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    const float s = __uint_as_float(a.x) + __uint_as_float(a.y);
    const unsigned int sbits = __float_as_uint(s);
    const u32x2_swap b = __builtin_amdgcn_permlane32_swap(sbits, sbits, false, false);
    return __uint_as_float(b.x) + __uint_as_float(b.y);
}

} // namespace zllm

// Pieces shared by the kernels that run a contraction on the matrix cores with float32 accuracy: operand types of
// v_mfma_f32_32x32x16_bf16 and the exact split of a float32 number into three bf16 numbers.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstddef>

namespace dbk_mfma {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// two float32 bit patterns -> their upper halves as (bf16 e0, bf16 e1), e0 in the low half
__device__ __forceinline__ unsigned pack_upper_halves(unsigned e0, unsigned e1) { return __builtin_amdgcn_perm(e1, e0, 0x07060302u); }

// w = hi + mid + lo, each with at most 8 significant bits (truncations of the running remainder; the subtractions are exact)
__device__ __forceinline__ void split3(float w, unsigned& lo, unsigned& mid, unsigned& hi)
{
    // (the low halves stay in mid and lo as they come: the packing takes the upper halves only)
    hi = __float_as_uint(w) & 0xffff0000u;
    const float r1 = w - __uint_as_float(hi);
    mid = __float_as_uint(r1);
    const float r2 = r1 - __uint_as_float(mid & 0xffff0000u);
    lo = __float_as_uint(r2);
}

// D += A . B for one 32 x 32 tile and 16 values of the contraction index. Lane l supplies row (A) / column (B) l & 31
// and contraction values 8 * (l >> 5) .. + 7; it receives column l & 31, rows (i & 3) + 8 * (i >> 2) + 4 * (l >> 5).
__device__ __forceinline__ f32x16_t mfma_bf16(const uint4& a, const uint4& b, const f32x16_t& c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// Four bytes of X at offset o (any alignment); bytes past the end read as 254, "nothing".
__device__ __forceinline__ unsigned load_letters4(const uint8_t* __restrict__ X, size_t N, size_t o)
{
    unsigned v;
    if (o + 4 <= N) {
        __builtin_memcpy(&v, X + o, 4);
    } else {
        v = 0xfefefefeu;
#pragma unroll
        for (int t = 0; t < 4; ++t)
            if (o + t < N) v = (v & ~(0xffu << (8 * t))) | ((unsigned)X[o + t] << (8 * t));
    }
    return v;
}

}  // namespace dbk_mfma

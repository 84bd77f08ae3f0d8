// Pieces shared by the scan kernels: the 6-letter alphabet and the [tap][letter][filter] LDS table.
#pragma once
#include "dbk_common.h"

namespace dbk_scan {

constexpr int FT = 64;        // filters per tile = lanes per wave
constexpr int NL = 6;         // letters in the LDS table
constexpr int PSUB = 16;      // positions accumulated in registers at a time

__device__ __forceinline__ unsigned letter_of(unsigned code)
{
    return code < 4u ? code : (code == 254u ? 5u : 4u);
}

// Builds lut[(j*NL + l)*FT + fl] for filters [f0, f0+FT) from W (4m, F); missing filters read as 0.
// With mpad > m the table gets all-zero rows for taps m..mpad-1.
template <typename T>
__device__ void build_letter_table(T* lut, const T* __restrict__ W, unsigned m, unsigned F, unsigned f0, unsigned mpad = 0)
{
    if (mpad < m) mpad = m;
    for (unsigned e = threadIdx.x; e < mpad * FT; e += blockDim.x) {
        unsigned j = e / FT, fl = e % FT;
        unsigned f = f0 + fl;
        T w0 = 0, w1 = 0, w2 = 0, w3 = 0;
        if (f < F && j < m) {
            w0 = W[(4 * j + 0) * (size_t)F + f];
            w1 = W[(4 * j + 1) * (size_t)F + f];
            w2 = W[(4 * j + 2) * (size_t)F + f];
            w3 = W[(4 * j + 3) * (size_t)F + f];
        }
        T z = w0;
        z += w1;
        z += w2;
        z += w3;
        T* row = lut + (size_t)j * NL * FT + fl;
        row[0 * FT] = w0;
        row[1 * FT] = w1;
        row[2 * FT] = w2;
        row[3 * FT] = w3;
        row[4 * FT] = z * (T)0.25;
        row[5 * FT] = (T)0;
    }
}


inline size_t lds_limit()
{
    static size_t cached = 0;
    if (!cached) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && v > 0)
            cached = (size_t)v;
        else
            cached = 65536;
    }
    return cached;
}


}  // namespace dbk_scan

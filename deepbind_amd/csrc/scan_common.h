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

// Number of 4-letter words covering the window of PSUB positions and MT taps.
template <int MT> struct window { static constexpr int words = (PSUB + MT - 1 + 3) / 4; };

// Reads the letters of the window starting at 4-byte aligned xl+p0 into scalar registers (all lanes of
// a wave look at the same positions).
template <int MT>
__device__ __forceinline__ void load_window(const uint8_t* xl, unsigned p0, unsigned (&wq)[window<MT>::words])
{
    const unsigned* xw = reinterpret_cast<const unsigned*>(xl + p0);
#pragma unroll
    for (int t = 0; t < window<MT>::words; ++t) wq[t] = (unsigned)__builtin_amdgcn_readfirstlane((int)xw[t]);
}

// Bytes to stage so that every window word of a chunk with `rows` positions holds valid letters.
template <int MT>
__device__ __forceinline__ unsigned window_span(unsigned rows) { return ((rows + PSUB - 1) & ~(unsigned)(PSUB - 1)) + 4 * window<MT>::words - PSUB; }

__device__ __forceinline__ unsigned window_letter(const unsigned* wq, int q) { return (wq[q >> 2] >> ((q & 3) * 8)) & 0xffu; }

// scan16 for filters of at most MT taps with the letters in scalar registers: one address add per
// letter, then every (position, tap) pair is a single LDS read with an immediate offset. The table
// must have been built with MT taps (zero rows past m). Taps are added in ascending order per
// position, exactly as scan16 does.
template <int MT, typename T>
__device__ __forceinline__ void scan16_window(const T* __restrict__ lut, const unsigned (&wq)[window<MT>::words], unsigned lane,
                                              T acc[PSUB])
{
#pragma unroll
    for (int p = 0; p < PSUB; ++p) acc[p] = (T)0;
#pragma unroll
    for (int q = 0; q < PSUB + MT - 1; ++q) {
        const T* col = lut + window_letter(wq, q) * FT + lane;
#pragma unroll
        for (int p = 0; p < PSUB; ++p) {
            const int j = q - p;
            if (j >= 0 && j < MT) acc[p] += col[j * NL * FT];
        }
        // pin the running sums every fourth letter: otherwise the scheduler issues the whole window's reads
        // first and finishes one position's chain at a time, holding ~400 loaded values in registers
        if ((q & 3) == 3) {
            static_assert(PSUB == 16, "the pin below lists 16 accumulators");
            asm volatile("" : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]),
                         "+v"(acc[7]), "+v"(acc[8]), "+v"(acc[9]), "+v"(acc[10]), "+v"(acc[11]), "+v"(acc[12]), "+v"(acc[13]),
                         "+v"(acc[14]), "+v"(acc[15]));
        }
    }
}

// Stages letters for absolute positions [c0, c0+cnt) into xl; past the end of X -> "nothing".
__device__ __forceinline__ void stage(uint8_t* xl, const uint8_t* __restrict__ X, size_t N, size_t c0, unsigned cnt)
{
    for (unsigned t = threadIdx.x; t < cnt; t += blockDim.x) {
        size_t g = c0 + t;
        xl[t] = g < N ? (uint8_t)letter_of(X[g]) : (uint8_t)5;
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

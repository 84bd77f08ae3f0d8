// Fused motif scan + bias + ReLU + region pooling, forward and backward, general path.
//
// The (N, F) activation map is never written: a workgroup owns a tile of 64 filters (one lane per
// filter) and walks whole regions, each wave scanning 16 positions at a time in registers and
// folding them straight into the region's running max / argmax / sum. This path takes any filter
// length that fits in LDS, any region table and every letter code; the k-mer table kernel in
// scanpool_kmer.hip is the fast path for bulk scoring and falls back to this one.
//
// Backward: the max part is 1-sparse (one position per region and filter), the average part is
// dense and needs the forward recomputed for the ReLU mask. Both accumulate into per-wave private
// [tap][channel][filter] tables in LDS (a lane only ever touches its own filter column, so no
// atomics), the workgroup folds its waves in a fixed order into one slab in HBM, and a second
// kernel sums the slabs in a fixed tree: bit-reproducible gradients.
//
// Reference chain being fused: kangaroo/_ext/corr1ord.py:97-138, deepity/std/elemwise.py:71-82,162-180,
// kangaroo/_ext/poolrgn.py:56-82,153-180 with kernels corr1ord.cuh:139-157, poolrgn.cuh:44-160,
// poolrgn_bprop.cuh:45-127, corr1ord_bprop.cuh:91-137.
#include "dbk_common.h"
#include "scan_common.h"

namespace dbk_scanpool_general {

using namespace dbk_scan;

constexpr unsigned XCH_SUBS = 4;          // sub-chunks of PSUB positions per wave and staging round

// A workgroup's place in its launch: (x, y) of a grid of gx by gy. The kernels of a training step take it as an
// argument instead of reading blockIdx / gridDim, so that one launch can hold the grids of several model groups.
struct wg_t { unsigned x, y, gx, gy; };
__device__ __forceinline__ wg_t this_wg() { return wg_t{blockIdx.x, blockIdx.y, gridDim.x, gridDim.y}; }

// Scans PSUB positions starting at chunk-relative p0 for this lane's filter.
__device__ __forceinline__ void scan16(const float* __restrict__ lut, const uint8_t* __restrict__ xl, unsigned m,
                                       unsigned p0, unsigned lane, float acc[PSUB])
{
#pragma unroll
    for (int p = 0; p < PSUB; ++p) acc[p] = 0.0f;
    for (unsigned j = 0; j < m; ++j) {
        const float* row = lut + (size_t)j * NL * FT + lane;
        const uint8_t* xs = xl + p0 + j;
#pragma unroll
        for (int p = 0; p < PSUB; ++p) acc[p] += row[(unsigned)xs[p] * FT];
    }
}

// MT > 0: filters of at most MT taps, letters held in scalar registers (scan16_window); MT == 0: any length.
template <int PT, bool WANT_ARGMAX, int MT>
__device__ __forceinline__ void scanpool_fprop_body(const wg_t wg, const float* __restrict__ W, const float* __restrict__ bias,
                                                    unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                    const uint32_t* __restrict__ R, size_t P,
                                                    float* __restrict__ pooled, uint32_t* __restrict__ argmax,
                                                    const unsigned* __restrict__ run_if_flag,
                                                    unsigned long long* __restrict__ act)
{
    extern __shared__ __align__(16) unsigned char smem[];
    // when given, the launch only does work if the device flag is set (fallback behind the k-mer kernel)
    if (run_if_flag && run_if_flag[0] == 0) return;
    const unsigned nw = blockDim.x >> 6;
    const unsigned chunk = nw * XCH_SUBS * PSUB;
    // up to 16 taps: the lane's filter weights live in register planes and the scan needs no table in LDS
    // (measured: 7.2 vs 9.1 us on a 128-sequence batch of width 16; with 24 taps the planes take 144 registers,
    // a CU holds two workgroups instead of three and the LDS table is the faster choice: 19.5 vs 21.7 us)
    constexpr bool PLANES = MT == 8 || MT == 16;
    constexpr int PMT = PLANES ? MT : 8;
    float* lut = reinterpret_cast<float*>(smem);
    float* red = lut + (PLANES ? 0 : (size_t)(MT ? MT : m) * NL * FT);   // [nw][3][FT]: max, index, sum
    uint8_t* xl = reinterpret_cast<uint8_t*>(red + (size_t)nw * 3 * FT);

    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned f0 = wg.y * FT, f = f0 + lane;
    const size_t n = N + 1 >= (size_t)m + 1 ? N - m + 1 : 0;    // rows the scan defines; later rows are relu(bias)
    grad_planes<PMT> planes;
    if constexpr (PLANES) weight_planes_load<PMT>(planes, W, m, F, f);
    else build_letter_table(lut, W, m, F, f0, MT);
    const float bf = f < F ? bias[f] : 0.0f;

    for (size_t r = wg.x; r < P; r += wg.gx) {
        const size_t a = R[2 * r], b = R[2 * r + 1];
        float mx = -1.0f, sum = 0.0f;
        size_t xi = a;
        for (size_t c0 = a; c0 < b; c0 += chunk) {
            const unsigned rows = (unsigned)((b - c0) < chunk ? (b - c0) : chunk);
            __syncthreads();
            stage(xl, X, N, c0, MT ? window_span<MT ? MT : 1>(rows) : rows + m - 1);
            __syncthreads();
#pragma unroll 1
            for (unsigned s = 0; s < XCH_SUBS; ++s) {
                const unsigned p0 = (s * nw + wave) * PSUB;
                if (p0 >= rows) break;
                float acc[PSUB];
                if constexpr (PLANES) {
                    unsigned wq[window<PMT>::words];
                    load_window<PMT>(xl, p0, wq);
                    scan16_planes<PMT>(planes, wq, acc);
                } else if (MT) {
                    unsigned wq[window<MT ? MT : 1>::words];
                    load_window<MT ? MT : 1>(xl, p0, wq);
                    scan16_window<MT ? MT : 1>(lut, wq, lane, acc);
                } else {
                    scan16(lut, xl, m, p0, lane, acc);
                }
                if (act) {
                    // which rectifiers are open, for the backward pass: one 64-bit lane mask per (row, filter tile);
                    // lane p of the wave stores row p's
                    unsigned long long mine = 0;
#pragma unroll
                    for (int p = 0; p < PSUB; ++p) {
                        const size_t i = c0 + p0 + p;
                        const unsigned long long open = __ballot(((i < n ? acc[p] : 0.0f) + bf) > 0.0f);
                        if (lane == (unsigned)p) mine = open;
                    }
                    if (lane < (unsigned)PSUB && p0 + lane < rows) act[(c0 + p0 + lane) * wg.gy + wg.y] = mine;
                }
#pragma unroll
                for (int p = 0; p < PSUB; ++p) {
                    const size_t i = c0 + p0 + p;
                    if (p0 + p < rows) {
                        float z = (i < n ? acc[p] : 0.0f) + bf;
                        z = z > 0.0f ? z : 0.0f;
                        if (PT != DBK_PT_AVG) { if (z > mx) { mx = z; xi = i; } }
                        if (PT != DBK_PT_MAX) sum += z;
                    }
                }
            }
        }
        // fold the waves: larger value wins, equal values keep the earlier row
        red[(wave * 3 + 0) * FT + lane] = mx;
        red[(wave * 3 + 1) * FT + lane] = __uint_as_float((unsigned)(xi - a));
        red[(wave * 3 + 2) * FT + lane] = sum;
        __syncthreads();
        if (wave == 0 && f < F) {
            float bm = red[lane];
            unsigned bi = __float_as_uint(red[FT + lane]);
            float bs = red[2 * FT + lane];
            for (unsigned w = 1; w < nw; ++w) {
                float vm = red[(w * 3 + 0) * FT + lane];
                unsigned vi = __float_as_uint(red[(w * 3 + 1) * FT + lane]);
                if (vm > bm || (vm == bm && vi < bi)) { bm = vm; bi = vi; }
                bs += red[(w * 3 + 2) * FT + lane];
            }
            const size_t j = r * F + f;
            const float cnt = (float)(b - a);
            bm = bm > 0.0f ? bm : 0.0f;                          // only an empty region gets here with bm < 0
            if (PT == DBK_PT_MAX) pooled[j] = bm;
            else if (PT == DBK_PT_AVG) pooled[j] = bs / cnt;
            else { pooled[2 * j] = bm; pooled[2 * j + 1] = bs / cnt; }
            if (WANT_ARGMAX && PT != DBK_PT_AVG) argmax[j] = (uint32_t)((a + bi) * F + f);
        }
        __syncthreads();                                         // red[] is reused by the next region
    }
}

template <int PT, bool WANT_ARGMAX, int MT>
__global__ __launch_bounds__(256) void scanpool_fprop_kernel(const float* __restrict__ W, const float* __restrict__ bias,
                                                             unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                             const uint32_t* __restrict__ R, size_t P,
                                                             float* __restrict__ pooled, uint32_t* __restrict__ argmax,
                                                             const unsigned* __restrict__ run_if_flag,
                                                             unsigned long long* __restrict__ act)
{
    scanpool_fprop_body<PT, WANT_ARGMAX, MT>(this_wg(), W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag, act);
}

// The same forward pass with four filters per lane, for batches of many regions (filters of 17-24 taps).
//
// The kernel above spends one 4-byte LDS read per (position, tap, filter): a wave's read moves 256 bytes and the
// LDS delivers ~104 B/clk/CU of those, which is what bounds it once the GPU is full. Here a lane owns the four
// filters l, l+16, l+32, l+48 of the tile and the table row is laid out [16 lanes][4 filters], so the 16 lanes
// of a quarter wave read one aligned 256-byte line with ds_read_b128 (~216 B/clk/CU), and the four quarters of
// the wave work on four consecutive windows of 16 positions. A wave therefore takes 64 positions of ONE region
// at a time and the four waves of a workgroup walk four different regions: no workgroup barrier after the
// table is built. The letters of a quarter's window sit in ten vector registers (they differ between the
// quarters); one bit-field extract and one address add per letter serve up to 16 (position, tap) reads.
// Per position the taps are added in ascending order, as everywhere else: maxima and argmax are the bits of
// the kernel above; averages add the same rectified values in another order (quarter by quarter).
constexpr unsigned WIDE_SPAN = 4 * PSUB;                          // positions per wave and round

template <int PT, bool WANT_ARGMAX, int MT>
__device__ __forceinline__ void scanpool_fprop_wide_body(const wg_t wg, const float* __restrict__ W, const float* __restrict__ bias,
                                                         unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                         const uint32_t* __restrict__ R, size_t P,
                                                         float* __restrict__ pooled, uint32_t* __restrict__ argmax,
                                                         unsigned long long* __restrict__ act)
{
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr unsigned NWORD = wide_shape<MT>::words, XB = wide_shape<MT>::xbytes;
    const unsigned nw = blockDim.x >> 6;
    float* lut = reinterpret_cast<float*>(smem);                   // [MT*NL][16][4]
    // the wave's index, region bounds and loop control are wave-uniform: kept in scalar registers
    const unsigned lane = threadIdx.x & 63, wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned qd = lane >> 4, l = lane & 15;
    uint8_t* xw = smem + (size_t)MT * NL * FT * sizeof(float) + (size_t)wave * XB;   // this wave's letters
    const unsigned f0 = wg.y * FT;
    const size_t n = N + 1 >= (size_t)m + 1 ? N - m + 1 : 0;    // rows the scan defines; later rows are relu(bias)
    build_letter_table<float, true>(lut, W, m, F, f0, MT);
    float bf[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) bf[c] = f0 + c * 16 + l < F ? bias[f0 + c * 16 + l] : 0.0f;
    __syncthreads();
    const float4* lut4 = reinterpret_cast<const float4*>(lut) + l;

    for (size_t r = (size_t)wg.x * nw + wave; r < P; r += (size_t)wg.gx * nw) {
        const size_t a = (unsigned)__builtin_amdgcn_readfirstlane((int)R[2 * r]), b = (unsigned)__builtin_amdgcn_readfirstlane((int)R[2 * r + 1]);
        float mx[4] = {-1.0f, -1.0f, -1.0f, -1.0f}, sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        unsigned xi[4] = {0u, 0u, 0u, 0u};                        // row of the maximum, relative to a
        for (size_t c0 = a; c0 < b; c0 += WIDE_SPAN) {
            const unsigned rows = (unsigned)((b - c0) < WIDE_SPAN ? (b - c0) : WIDE_SPAN);
            // ---- the round's letters, then this quarter's window: 16 positions x MT taps x 4 filters
            unsigned wq[NWORD];
            wide_stage<MT>(xw, X, N, c0, lane, wq);
            float4 acc[PSUB];
            scan16_wide<MT>(lut4, wq, acc);
            // ---- bias, rectifier, pooling; optionally the activity masks of the 64 rows
            const unsigned pq = PSUB * qd;                         // first position of this quarter's window
            unsigned long long mine = 0ull;
#pragma unroll
            for (int p = 0; p < PSUB; ++p) {
                const size_t i = c0 + pq + p;
                const bool defined = i < n;
                float z[4] = {acc[p].x, acc[p].y, acc[p].z, acc[p].w};
#pragma unroll
                for (int c = 0; c < 4; ++c) z[c] = (defined ? z[c] : 0.0f) + bf[c];
                if (act) {
                    // ballot c holds, for each quarter, 16 bits: filters 16c .. 16c+15 of that quarter's row p
                    unsigned lo = 0u, hi = 0u;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const unsigned long long open = __ballot(z[c] > 0.0f);
                        const unsigned part = (unsigned)(open >> (16u * qd)) & 0xffffu;
                        if (c < 2) lo |= part << (16 * c);
                        else hi |= part << (16 * (c - 2));
                    }
                    if (l == (unsigned)p) mine = ((unsigned long long)hi << 32) | lo;
                }
                if (pq + p < rows) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float zr = z[c] > 0.0f ? z[c] : 0.0f;
                        if (PT != DBK_PT_AVG) { if (zr > mx[c]) { mx[c] = zr; xi[c] = (unsigned)(i - a); } }
                        if (PT != DBK_PT_MAX) sum[c] += zr;
                    }
                }
            }
            if (act && pq + l < rows) act[(c0 + pq + l) * wg.gy + wg.y] = mine;
        }
        // ---- fold the four quarters: larger value wins, equal values keep the earlier row
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int d = 16; d <= 32; d <<= 1) {
                const float vm = __shfl_xor(mx[c], d, 64);
                const unsigned vi = (unsigned)__shfl_xor((int)xi[c], d, 64);
                const float vs = __shfl_xor(sum[c], d, 64);
                if (vm > mx[c] || (vm == mx[c] && vi < xi[c])) { mx[c] = vm; xi[c] = vi; }
                sum[c] += vs;
            }
        }
        if (qd == 0) {
            const float cnt = (float)(b - a);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const unsigned f = f0 + c * 16 + l;
                if (f >= F) continue;
                const size_t j = r * F + f;
                const float bm = mx[c] > 0.0f ? mx[c] : 0.0f;      // only an empty region gets here with a negative maximum
                if (PT == DBK_PT_MAX) pooled[j] = bm;
                else if (PT == DBK_PT_AVG) pooled[j] = sum[c] / cnt;
                else { pooled[2 * j] = bm; pooled[2 * j + 1] = sum[c] / cnt; }
                if (WANT_ARGMAX && PT != DBK_PT_AVG) argmax[j] = (uint32_t)((a + xi[c]) * F + f);
            }
        }
    }
}

template <int PT, bool WANT_ARGMAX, int MT>
__global__ __launch_bounds__(256) void scanpool_fprop_wide_kernel(const float* __restrict__ W, const float* __restrict__ bias,
                                                                  unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                                  const uint32_t* __restrict__ R, size_t P,
                                                                  float* __restrict__ pooled, uint32_t* __restrict__ argmax,
                                                                  unsigned long long* __restrict__ act)
{
    scanpool_fprop_wide_body<PT, WANT_ARGMAX, MT>(this_wg(), W, bias, m, F, X, N, R, P, pooled, argmax, act);
}

}  // namespace dbk_scanpool_general

#include "scan_mfma.h"

namespace dbk_scanpool_general {

// ---------------------------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void add_tap(float* cell, unsigned l, float g, float gq)
{
    if (l < 4u) {
        cell[l * FT] += g;
    } else if (l == 4u) {
        cell[0 * FT] += gq;
        cell[1 * FT] += gq;
        cell[2 * FT] += gq;
        cell[3 * FT] += gq;
    }
}

template <int PT>
__global__ __launch_bounds__(256) void scanpool_bprop_kernel(const float* __restrict__ W, const float* __restrict__ bias,
                                                             unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                             const uint32_t* __restrict__ R, size_t P,
                                                             const float* __restrict__ pooled, const uint32_t* __restrict__ argmax,
                                                             const float* __restrict__ dpooled,
                                                             float* __restrict__ slabs, size_t stride)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const unsigned nw = blockDim.x >> 6;
    const unsigned chunk = nw * XCH_SUBS * PSUB;
    const unsigned tab = m * 4 * FT;
    float* lut = reinterpret_cast<float*>(smem);                   // only used when the average part is present
    float* acc_tab = lut + (PT == DBK_PT_MAX ? 0 : (size_t)m * NL * FT);
    float* dbacc = acc_tab + (size_t)nw * tab;                     // [nw][FT]
    uint8_t* xl = reinterpret_cast<uint8_t*>(dbacc + (size_t)nw * FT);

    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned f0 = blockIdx.y * FT, f = f0 + lane;
    const size_t n = N + 1 >= (size_t)m + 1 ? N - m + 1 : 0;
    if (PT != DBK_PT_MAX) build_letter_table(lut, W, m, F, f0);
    for (unsigned e = threadIdx.x; e < nw * tab + nw * FT; e += blockDim.x) acc_tab[e] = 0.0f;
    const float bf = f < F ? bias[f] : 0.0f;
    float* mine = acc_tab + (size_t)wave * tab + lane;
    float db = 0.0f;
    __syncthreads();

    for (size_t r = blockIdx.x; r < P; r += gridDim.x) {
        const size_t a = R[2 * r], b = R[2 * r + 1];
        const size_t j0 = r * F + f;
        // ---- max part: one position per (region, filter); wave (r mod nw) does it
        if (PT != DBK_PT_AVG && (r % nw) == wave && f < F) {
            const float pv = PT == DBK_PT_MAX ? pooled[j0] : pooled[2 * j0];
            const float g = (pv > 0.0f) ? (PT == DBK_PT_MAX ? dpooled[j0] : dpooled[2 * j0]) : 0.0f;
            if (g != 0.0f) {
                const size_t i = argmax[j0] / F;
                db += g;
                if (i < n) {
                    const float gq = g * 0.25f;
                    for (unsigned j = 0; j < m; ++j) add_tap(mine + (size_t)j * 4 * FT, letter_of(X[i + j]), g, gq);
                }
            }
        }
        // ---- average part: recompute the map, mask by ReLU, spread davg/count
        if (PT != DBK_PT_MAX) {
            const float gavg = f < F ? (PT == DBK_PT_AVG ? dpooled[j0] : dpooled[2 * j0 + 1]) / (float)(b - a) : 0.0f;
            for (size_t c0 = a; c0 < b; c0 += chunk) {
                const unsigned rows = (unsigned)((b - c0) < chunk ? (b - c0) : chunk);
                __syncthreads();
                stage(xl, X, N, c0, rows + m - 1);
                __syncthreads();
    #pragma unroll 1
            for (unsigned s = 0; s < XCH_SUBS; ++s) {
                    const unsigned p0 = (s * nw + wave) * PSUB;
                    if (p0 >= rows) break;
                    float acc[PSUB];
                    scan16(lut, xl, m, p0, lane, acc);
#pragma unroll
                    for (int p = 0; p < PSUB; ++p) {
                        const size_t i = c0 + p0 + p;
                        if (p0 + p < rows) {
                            const float z = (i < n ? acc[p] : 0.0f) + bf;
                            const float g = z > 0.0f ? gavg : 0.0f;
                            db += g;
                            if (i < n) {
                                const float gq = g * 0.25f;
                                for (unsigned j = 0; j < m; ++j) add_tap(mine + (size_t)j * 4 * FT, xl[p0 + p + j], g, gq);
                            }
                        }
                    }
                }
            }
        }
    }
    dbacc[wave * FT + lane] = db;
    __syncthreads();
    float* outW = slabs + (size_t)blockIdx.x * stride;
    for (unsigned e = threadIdx.x; e < tab; e += blockDim.x) {
        float s = acc_tab[e];
        for (unsigned w = 1; w < nw; ++w) s += acc_tab[(size_t)w * tab + e];
        const unsigned row = e / FT, fl = e % FT;
        if (f0 + fl < F) outW[(size_t)row * F + f0 + fl] = s;
    }
    if (wave == 0 && f < F) {
        float s = dbacc[lane];
        for (unsigned w = 1; w < nw; ++w) s += dbacc[w * FT + lane];
        outW[(size_t)4 * m * F + f] = s;
    }
}

// For up to four positions i_u with gradients g_u: adds g_u at (tap j, letter of X[i_u+j]) for j < m into
// this lane's column of a [tap][channel][FT] table. Taps go eight at a time: the letters of all four
// positions are loaded first (32 independent global loads in flight), then each position's eight cells
// are read, updated and written (distinct taps are distinct cells), positions in ascending order.
// Adds g[u] at the MT-letter windows starting at pos[u], u = 0..3, into this lane's private column of the
// LDS slab, laid out [tap][A, C, G, T, mean-of-four][filter]: every letter, "mean of the four" included,
// touches exactly one cell, so a batch of eight taps is one LDS round trip (the mean row is spread over
// the four channels when the slab is written out).
constexpr int SPARSE_ROWS = 5;
template <int MT>
__device__ __forceinline__ void add_positions4(float* mine, const uint8_t* __restrict__ X, size_t N, const size_t (&pos)[4],
                                               const float (&g)[4], const bool (&on)[4], unsigned m)
{
    // The letters of all four windows first, so that their loads are in flight together: a window of MT
    // letters starting at any byte is MT/4 + 1 aligned 32-bit words shifted into place; a word is only
    // fetched if it starts before the end of the stream.
    static_assert(MT % 8 == 0, "windows are taken eight letters at a time");
    constexpr int NW = MT / 4 + 1;
    unsigned w[4][NW], sh[4];
    const uintptr_t xend = reinterpret_cast<uintptr_t>(X) + N;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const uintptr_t addr = reinterpret_cast<uintptr_t>(X) + pos[u];
        const uintptr_t base = addr & ~(uintptr_t)3;
        sh[u] = (unsigned)(addr & 3);
#pragma unroll
        for (int t = 0; t < NW; ++t)
            w[u][t] = (on[u] && base + 4 * t < xend) ? *reinterpret_cast<const unsigned*>(base + 4 * t) : 0xffffffffu;
    }
#pragma unroll
    for (unsigned j0 = 0; j0 < (unsigned)MT; j0 += 8) {
        if (j0 >= m) break;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const unsigned lo = __builtin_amdgcn_alignbyte(w[u][j0 / 4 + 1], w[u][j0 / 4], sh[u]);
            const unsigned hi = __builtin_amdgcn_alignbyte(w[u][j0 / 4 + 2], w[u][j0 / 4 + 1], sh[u]);     // j0/4 + 2 <= MT/4
            unsigned l[8];
#pragma unroll
            for (unsigned t = 0; t < 8; ++t) {
                const unsigned code = ((t < 4 ? lo : hi) >> ((t & 3) * 8)) & 0xffu;
                l[t] = (on[u] && j0 + t < m) ? letter_of(code) : 5u;
            }
            float v[8];
#pragma unroll
            for (unsigned t = 0; t < 8; ++t) v[t] = l[t] < 5u ? mine[((j0 + t) * SPARSE_ROWS + l[t]) * FT] : 0.0f;
#pragma unroll
            for (unsigned t = 0; t < 8; ++t)
                if (l[t] < 5u) mine[((j0 + t) * SPARSE_ROWS + l[t]) * FT] = v[t] + g[u];
        }
    }
}
// One wave; in a launch of wider workgroups only the first wave of a workgroup may enter.
// The end of a backward workgroup: its four waves hold their sums of the filter gradient in registers (lane = filter)
// and add them up in wave order into the workgroup's slab. Eight taps per round: every wave stores its 8 x 4 sums per
// lane side by side in LDS (128 KB would be needed for all 24 taps of four waves at once), then all 256 threads add
// the four copies of 8 elements each ((w0 + w1) + w2) + w3 and store them: two barriers per round and every LDS access of
// a round in flight together, where one wave after the other adding into one shared copy took four barriers and a
// dependent read-add-write per sum (measured on a calibration batch: 5.4 + 2.0 us of a 17.7 us workgroup; now 1.3).
constexpr int FOLD_TAPS = 8;
constexpr unsigned FOLD_ROUND = FOLD_TAPS * 4 * FT;              // floats of one wave's round
constexpr size_t FOLD_BYTES = (4 * (size_t)FOLD_ROUND + 4 * FT) * sizeof(float);   // four waves' rounds + their bias sums
template <int MT, typename V>
__device__ __forceinline__ void fold_waves_into_slab(unsigned char* smem_base, V value, float db, unsigned m, unsigned F, unsigned f0,
                                                     float* __restrict__ out)
{
    float* area = reinterpret_cast<float*>(smem_base);
    float* dbacc = area + 4 * FOLD_ROUND;
    const unsigned lane = threadIdx.x & 63, wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), nw = blockDim.x >> 6;
#pragma unroll
    for (int t0 = 0; t0 < MT; t0 += FOLD_TAPS) {
        __syncthreads();                                           // whatever lay here, and the last round's sums, are no longer read
        if (t0 == 0) dbacc[wave * FT + lane] = db;
        float* mine = area + wave * FOLD_ROUND + lane;
#pragma unroll
        for (int j = 0; j < FOLD_TAPS; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (t0 + j < MT) mine[(j * 4 + c) * FT] = value(t0 + j, c);
        __syncthreads();
#pragma unroll
        for (unsigned u = 0; u < FOLD_ROUND / 256; ++u) {
            const unsigned e = threadIdx.x + u * 256, row = (unsigned)t0 * 4 + e / FT, fl = e % FT;
            float v = area[e];
            for (unsigned w = 1; w < nw; ++w) v += area[w * FOLD_ROUND + e];
            if (row < 4 * m && f0 + fl < F) out[(size_t)row * F + f0 + fl] = v;
        }
    }
    if (wave == 0 && f0 + lane < F) {
        float t = dbacc[lane];
        for (unsigned w = 1; w < nw; ++w) t += dbacc[w * FT + lane];
        out[(size_t)4 * m * F + f0 + lane] = t;
    }
}

template <int PT, int MT>
__device__ __forceinline__ void scanpool_bprop_sparse_body(const wg_t wg, unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                           size_t P, const float* __restrict__ pooled,
                                                           const uint32_t* __restrict__ argmax, const float* __restrict__ dpooled,
                                                           float* __restrict__ slabs, size_t stride)
{
    extern __shared__ __align__(16) unsigned char smem[];
    float* table = reinterpret_cast<float*>(smem);
    const unsigned lane = threadIdx.x;
    const unsigned f = wg.y * FT + lane;
    const size_t n = N + 1 >= (size_t)m + 1 ? N - m + 1 : 0;
    float* mine = table + lane;                                   // a lane only ever touches its own column: no barriers needed
    for (unsigned row = 0; row < SPARSE_ROWS * m; ++row) mine[row * FT] = 0.0f;
    float db = 0.0f;
    if (f < F) {
        const size_t gx = wg.gx;
        for (size_t r = wg.x; r < P; r += 4 * gx) {
            float g[4];
            size_t pos[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const size_t ru = r + u * gx;
                g[u] = 0.0f;
                pos[u] = 0;
                if (ru < P) {
                    const size_t j0 = ru * F + f;
                    const float pv = PT == DBK_PT_MAX ? pooled[j0] : pooled[2 * j0];
                    const float gd = PT == DBK_PT_MAX ? dpooled[j0] : dpooled[2 * j0];
                    pos[u] = argmax[j0] / F;
                    g[u] = pv > 0.0f ? gd : 0.0f;
                }
            }
            bool on[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (g[u] != 0.0f) db += g[u];
                on[u] = g[u] != 0.0f && pos[u] < n;
            }
            add_positions4<MT>(mine, X, N, pos, g, on, m);
        }
        float* out = slabs + (size_t)wg.x * stride;
        for (unsigned j = 0; j < m; ++j) {
            const float* tap = mine + (size_t)j * SPARSE_ROWS * FT;
            const float q = 0.25f * tap[4 * FT];
            float* o = out + (size_t)(4 * j) * F + f;
            o[0] = tap[0] + q;
            o[F] = tap[FT] + q;
            o[2 * (size_t)F] = tap[2 * FT] + q;
            o[3 * (size_t)F] = tap[3 * FT] + q;
        }
        out[(size_t)4 * m * F + f] = db;
    }
}

template <int PT, int MT>
__global__ __launch_bounds__(64) void scanpool_bprop_sparse_kernel(unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                                   size_t P, const float* __restrict__ pooled,
                                                                   const uint32_t* __restrict__ argmax, const float* __restrict__ dpooled,
                                                                   float* __restrict__ slabs, size_t stride)
{
    scanpool_bprop_sparse_body<PT, MT>(this_wg(), m, F, X, N, P, pooled, argmax, dpooled, slabs, stride);
}

// Dense half of the backward pass (avg and max+avg pooling), filters of at most MT taps: every
// position of a region receives davg/count where the recomputed activation is positive. A lane keeps
// its filter's whole [tap][channel] gradient column in registers: the letter at a position is the
// same for all 64 lanes (lanes are filters), so it is read once into scalar registers, turned into
// four scalar weights (1 for the matching channel, 1/4 each for N, else 0) and applied as fused
// multiply-adds whose products are exact, i.e. one rounding per addition as in the reference's add.
template <int PT, int MT>
__global__ __launch_bounds__(256) void scanpool_bprop_dense_kernel(const float* __restrict__ W, const float* __restrict__ bias,
                                                                   unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                                   const uint32_t* __restrict__ R, size_t P,
                                                                   const float* __restrict__ pooled, const uint32_t* __restrict__ argmax,
                                                                   const float* __restrict__ dpooled,
                                                                   float* __restrict__ slabs, size_t stride)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const unsigned nw = blockDim.x >> 6;
    const unsigned chunk = nw * XCH_SUBS * PSUB;
    float* lut = reinterpret_cast<float*>(smem);                   // [MT][NL][FT]; the memory is reused for the cross-wave fold at the end
    uint8_t* xl = reinterpret_cast<uint8_t*>(lut + (size_t)MT * NL * FT + (size_t)nw * FT);   // 4-byte aligned: everything before it is float

    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned f0 = blockIdx.y * FT, f = f0 + lane;
    const size_t n = N + 1 >= (size_t)m + 1 ? N - m + 1 : 0;
    build_letter_table(lut, W, m, F, f0, MT);
    const float bf = f < F ? bias[f] : 0.0f;
    float db = 0.0f;
    grad_planes<MT> planes;                                        // [letter][tap] accumulators in fixed registers
    planes.clear();

    for (size_t r = blockIdx.x; r < P; r += gridDim.x) {
        const size_t a = R[2 * r], b = R[2 * r + 1];
        const size_t j0 = r * F + f;
        const float gavg = f < F ? (PT == DBK_PT_AVG ? dpooled[j0] : dpooled[2 * j0 + 1]) / (float)(b - a) : 0.0f;
        // max+avg pooling: the maximum's gradient joins the average's at the winning row before the
        // rectifier, as it does in the unpooled gradient map of the layer-by-layer chain
        float gmax = 0.0f;
        size_t imax = ~(size_t)0;
        if (PT == DBK_PT_ALL && f < F && pooled[2 * j0] > 0.0f) { gmax = dpooled[2 * j0]; imax = argmax[j0] / F; }
        for (size_t c0 = a; c0 < b; c0 += chunk) {
            const unsigned rows = (unsigned)((b - c0) < chunk ? (b - c0) : chunk);
            __syncthreads();
            stage(xl, X, N, c0, window_span<MT>(rows));
            __syncthreads();
#pragma unroll 1
            for (unsigned s = 0; s < XCH_SUBS; ++s) {
                const unsigned p0 = (s * nw + wave) * PSUB;
                if (p0 >= rows) break;
                // letters of this sub-chunk's window, four per scalar register (letters past the region's
                // own window only ever meet zero table rows, g == 0 or taps >= m)
                unsigned wq[window<MT>::words];
                load_window<MT>(xl, p0, wq);
                float g[PSUB];
                scan16_window<MT>(lut, wq, lane, g);
#pragma unroll
                for (int p = 0; p < PSUB; ++p) {
                    const size_t i = c0 + p0 + p;
                    const float z = (i < n ? g[p] : 0.0f) + bf;
                    float gg = (p0 + p < rows && z > 0.0f) ? gavg : 0.0f;
                    if (PT == DBK_PT_ALL) gg += (p0 + p < rows && i == imax) ? gmax : 0.0f;
                    db += gg;
                    g[p] = i < n ? gg : 0.0f;                   // rows past the scan's end carry bias only
                }
                grad_planes_window<MT>(planes, wq, g);         // one add per (position, tap), the letter picks the plane
            }
        }
    }
    float aw[MT][4];
    grad_planes_read<MT>(planes, aw);
    // the waves' sums, added in wave order through the (now unused) letter table's memory, into the workgroup's slab
    fold_waves_into_slab<MT>(smem, [&](int j, int c) { return aw[j][c]; }, db, m, F, f0, slabs + (size_t)blockIdx.x * stride);
}

// Fixed-shape tree sum over slabs of nW + nB entries each: dW[e] += total (or = total with overwrite) for e < nW,
// dbias[e - nW] = total after that.
__global__ void reduce_slabs_kernel(float* __restrict__ dW, float* __restrict__ dbias, const float* __restrict__ slabs,
                                    size_t nW, size_t nB, unsigned nslab, bool overwrite)
{
    const size_t nelem = nW + nB;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < nelem; e += (size_t)gridDim.x * blockDim.x) {
        const float total = slab_sum(slabs, nelem, e, nslab);
        if (e < nW) dW[e] = overwrite ? total : dW[e] + total;
        else dbias[e - nW] = total;
    }
}

// The mask-driven backward through bit counts. At every row of a region whose rectifier is open the average-pooling
// gradient is the SAME number c = dpooled / rows, so the filter gradient needs no pass over the rows:
//     dW[tap][letter][f] += c * popcount(open_f & (is_letter >> tap))
// with one bit per row: open_f from the forward pass's activity masks (stored one 64-bit lane mask per row; turned
// into one row mask per lane = filter with a six-stage butterfly of lane exchanges), is_letter from five ballots over the chunk's
// letters (wave-uniform, shifted in scalar registers). A wave walks whole regions in chunks of 64 rows: per chunk
// ~7 vector instructions per (tap, letter) whatever the number of rows, against one half-rate index-mode add per
// (row, tap) in the kernels above: a third of their issue slots at 53 rows, a fifth at 64. The max-pooling gradient
// lands on one row per (region, filter): that row's letters are cut out of the same letter bits, once per region.
// A lane keeps the 5 x MT sums of its filter in registers over all its regions (ascending), the waves fold them
// into the workgroup's slab as above. Deterministic; c * count is rounded once where the kernels above add c count
// times, so the sums agree with theirs to rounding, not bit for bit.
// PT: DBK_PT_AVG / ALL read the masks; DBK_PT_MAX needs none.
// Transposes the 64 x 64 bit matrix whose row i is lane i's (lo, hi): afterwards bit i of lane j is what bit j of
// lane i was. Six butterfly stages (block sizes 32 ... 1): a lane and its partner lane ^ d swap the off-diagonal
// d x d blocks they hold between them.
__device__ __forceinline__ void transpose_masks(unsigned& lo, unsigned& hi, unsigned lane)
{
    {   // d = 32: whole words change places
        const unsigned plo = (unsigned)__shfl_xor((int)lo, 32, 64), phi = (unsigned)__shfl_xor((int)hi, 32, 64);
        if (lane & 32u) lo = phi; else hi = plo;
    }
#pragma unroll
    for (unsigned d = 16; d >= 1; d >>= 1) {
        // bits whose index has bit d clear, within a word
        const unsigned keep = d == 16 ? 0x0000ffffu : d == 8 ? 0x00ff00ffu : d == 4 ? 0x0f0f0f0fu : d == 2 ? 0x33333333u : 0x55555555u;
        const unsigned plo = (unsigned)__shfl_xor((int)lo, (int)d, 64), phi = (unsigned)__shfl_xor((int)hi, (int)d, 64);
        if (lane & d) {
            lo = ((plo >> d) & keep) | (lo & ~keep);
            hi = ((phi >> d) & keep) | (hi & ~keep);
        } else {
            lo = (lo & keep) | ((plo & keep) << d);
            hi = (hi & keep) | ((phi & keep) << d);
        }
    }
}
template <int PT, int MT>
__device__ __forceinline__ void scanpool_bprop_bits_body(const wg_t wg, unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                         const uint32_t* __restrict__ R, size_t P,
                                                         const float* __restrict__ pooled, const uint32_t* __restrict__ argmax,
                                                         const float* __restrict__ dpooled,
                                                         const unsigned long long* __restrict__ act,
                                                         float* __restrict__ slabs, size_t stride)
{
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr bool DENSE = PT != DBK_PT_MAX, PEAK = PT != DBK_PT_AVG;
    const unsigned nw = blockDim.x >> 6;
    const unsigned lane = threadIdx.x & 63, wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned f0 = wg.y * FT, f = f0 + lane;
    const size_t n = N + 1 >= (size_t)m + 1 ? N - m + 1 : 0;      // rows the scan defines; later rows carry bias only
    float acc[5][MT];
#pragma unroll
    for (int l = 0; l < 5; ++l)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[l][t] = 0.0f;
    float db = 0.0f;

    struct pooled_in { float davg, pmax, dmax; unsigned arg; };
    auto load_pooled = [&](size_t r_) -> pooled_in {
        pooled_in q = { 0.0f, 0.0f, 0.0f, 0u };
        if (f < F && r_ < P) {
            const size_t j0 = r_ * F + f;
            if (PT == DBK_PT_AVG) q.davg = dpooled[j0];
            else if (PT == DBK_PT_ALL) { q.davg = dpooled[2 * j0 + 1]; q.pmax = pooled[2 * j0]; q.dmax = dpooled[2 * j0]; q.arg = argmax[j0]; }
            else { q.pmax = pooled[j0]; q.dmax = dpooled[j0]; q.arg = argmax[j0]; }
        }
        return q;
    };
    auto bound = [&](size_t r_, unsigned which) -> size_t { return r_ < P ? (unsigned)__builtin_amdgcn_readfirstlane((int)R[2 * r_ + which]) : 0u; };
    struct raw { unsigned x0, x1; unsigned long long mk; };       // a chunk as loaded: two letters per lane, the row's mask
    auto load_chunk = [&](size_t c0, size_t bend) -> raw {
        raw w = { 254u, 254u, 0ull };
        const size_t g0 = c0 + lane, g1 = g0 + 64;
        if (g0 < N) w.x0 = X[g0];
        if (lane < (unsigned)MT - 1 && g1 < N) w.x1 = X[g1];
        if (DENSE && g0 < bend) w.mk = act[g0 * wg.gy + wg.y];
        return w;
    };

    const size_t step = (size_t)wg.gx * nw;
    size_t r = (size_t)wg.x * nw + wave;
    size_t a = bound(r, 0), b = bound(r, 1), na = bound(r + step, 0), nb = bound(r + step, 1);
    size_t nna = bound(r + 2 * step, 0), nnb = bound(r + 2 * step, 1);
    pooled_in q = load_pooled(r), nq = load_pooled(r + step);
    size_t c0 = a;
    raw cur = r < P ? load_chunk(c0, b) : raw{ 254u, 254u, 0ull };
    float gavg = 0.0f, gmax = 0.0f;
    size_t imax = ~(size_t)0;
    unsigned tm[5] = { 0u, 0u, 0u, 0u, 0u };                        // letters of the taps at the winning row: bit t of tm[l]
    while (r < P) {                                                // uniform over the wave
        // ---- the chunk after this one is requested before this one is worked on
        const bool last = c0 + 64 >= b;
        const size_t nc0 = last ? na : c0 + 64, nend = last ? nb : b;
        const bool more = last ? r + step < P : true;
        raw nxt = { 254u, 254u, 0ull };
        if (more) nxt = load_chunk(nc0, nend);
        if (c0 == a) {
            if (DENSE) gavg = b > a ? q.davg / (float)(b - a) : 0.0f;
            if (PEAK) {
                gmax = 0.0f; imax = ~(size_t)0;
                if (q.pmax > 0.0f) { gmax = q.dmax; imax = q.arg / F; }
#pragma unroll
                for (int l = 0; l < 5; ++l) tm[l] = 0u;
            }
        }
        // ---- one bit per (letter, position) of the chunk: positions c0 .. c0 + 63 and the MT - 1 behind them
        const unsigned v0 = letter_of(cur.x0), v1 = letter_of(cur.x1);
        unsigned long long L0[5], L1[5];
#pragma unroll
        for (int l = 0; l < 5; ++l) { L0[l] = __ballot(v0 == (unsigned)l); L1[l] = __ballot(v1 == (unsigned)l); }
        const size_t nrel = n > c0 ? n - c0 : 0;                   // rows of the chunk the scan defines
        if (DENSE) {
            // ---- one bit per row for this lane's filter: bit i of lane f = bit f of row i's mask
            const unsigned mlo = (unsigned)cur.mk, mhi = (unsigned)(cur.mk >> 32);
            unsigned tlo = mlo, thi = mhi;
            transpose_masks(tlo, thi, lane);
            db += gavg * (float)(__popc(tlo) + __popc(thi));
            const unsigned long long keep = nrel >= 64 ? ~0ull : ((1ull << nrel) - 1ull);
            tlo &= (unsigned)keep;
            thi &= (unsigned)(keep >> 32);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
#pragma unroll
                for (int l = 0; l < 5; ++l) {
                    const unsigned long long sh = t == 0 ? L0[l] : (L0[l] >> t) | (L1[l] << (64 - t));   // is_letter at row + t
                    const unsigned cnt = __popc(tlo & (unsigned)sh) + __popc(thi & (unsigned)(sh >> 32));
                    acc[l][t] = __builtin_fmaf(gavg, (float)cnt, acc[l][t]);
                }
            }
        }
        if (PEAK) {
            // ---- the winning row of this lane's filter, if it lies in the chunk: its taps' letters
            const bool here = imax >= c0 && imax - c0 < 64;
            const unsigned rel = here ? (unsigned)(imax - c0) : 0u;
            if (here) db += gmax;
            const bool counts = here && imax < n;
#pragma unroll
            for (int l = 0; l < 5; ++l) {
                const unsigned long long cut = rel == 0 ? L0[l] : (L0[l] >> rel) | (L1[l] << (64 - rel));
                tm[l] |= counts ? (unsigned)cut : 0u;              // (MT <= 32 taps: the low word is all that is looked at)
            }
            if (last) {
#pragma unroll
                for (int t = 0; t < MT; ++t) {
#pragma unroll
                    for (int l = 0; l < 5; ++l) acc[l][t] = __builtin_fmaf(gmax, (float)((tm[l] >> t) & 1u), acc[l][t]);
                }
            }
        }
        // ---- on to the next chunk / region
        if (last) {
            r += step;
            a = na; b = nb; q = nq;
            na = nna; nb = nnb;
            nna = bound(r + 2 * step, 0); nnb = bound(r + 2 * step, 1);
            nq = load_pooled(r + step);
        }
        c0 = nc0;
        cur = nxt;
    }
    fold_waves_into_slab<MT>(smem, [&](int j, int c) { return acc[c][j] + 0.25f * acc[4][j]; }, db, m, F, f0, slabs + (size_t)wg.x * stride);
}

template <int PT, int MT>
__global__ __launch_bounds__(256) void scanpool_bprop_bits_kernel(unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                                  const uint32_t* __restrict__ R, size_t P,
                                                                  const float* __restrict__ pooled, const uint32_t* __restrict__ argmax,
                                                                  const float* __restrict__ dpooled,
                                                                  const unsigned long long* __restrict__ act,
                                                                  float* __restrict__ slabs, size_t stride)
{
    scanpool_bprop_bits_body<PT, MT>(this_wg(), m, F, X, N, R, P, pooled, argmax, dpooled, act, slabs, stride);
}

// Launch shapes, shared by the single-group launchers and the multi-group ones.
// forward: as many workgroups as are resident at once (three per CU; two with the register planes of 16 taps);
// each sets up its filter tile's weights once and then walks its share of the regions
inline unsigned fprop_grid_x(unsigned mt, unsigned ftiles, size_t P)
{
    unsigned gx = (mt == 16 ? 512u : 768u) / ftiles;
    if (gx < 1) gx = 1;
    if (gx > P) gx = (unsigned)P;
    return gx;
}
inline size_t fprop_smem(unsigned mt, size_t m)
{
    const unsigned nw = 4;
    const size_t taps = mt ? mt : m;
    const bool planes = mt == 8 || mt == 16;                     // weights in registers: no table in LDS
    return (planes ? 0 : taps * NL * FT * sizeof(float)) + nw * 3 * FT * sizeof(float) + ((nw * XCH_SUBS * PSUB + taps - 1 + 7) & ~(size_t)3);
}
// sparse half of the backward pass: ~2048 single-wave workgroups, at least four regions each (more regions per
// workgroup only lengthens its chain of dependent loads)
inline unsigned sparse_grid_x(unsigned ftiles, size_t P)
{
    unsigned gxs = 2048u / ftiles;
    if (gxs > (P + 3) / 4) gxs = (unsigned)((P + 3) / 4);
    if (gxs < 1) gxs = 1;
    return gxs;
}
// dense half: four-wave workgroups, as many as are resident at once (its register planes leave room for two per
// CU, three with 8 taps). A minibatch (a handful of regions per workgroup) takes one workgroup per CU instead:
// alone the kernel runs as fast (half as many partial sums to write and to reduce), and it leaves half of every
// CU's registers to whatever else is running, such as the other architectures of a calibration batch.
inline unsigned dense_grid_x(unsigned mt, unsigned ftiles, size_t P)
{
    unsigned gxd = (mt == 8 ? 768u : 512u) / ftiles;
    if (P < 8 * (size_t)gxd) gxd = 256u / ftiles;
    if (gxd < 1) gxd = 1;
    if (gxd > P) gxd = (unsigned)P;
    return gxd;
}
// The wide forward kernel (four filters per lane, a wave per region) pays off once there are enough (region, tile)
// items to keep every CU's LDS busy; a small batch is latency-bound and better off with four waves per region.
inline bool wide_takes(size_t m, unsigned ftiles, size_t P) { return m > 8 && m <= 24 && P * (size_t)ftiles >= 512; }
inline unsigned wide_tier(size_t m) { return m <= 16 ? 16u : 24u; }
// The matrix-core forward takes those batches (same break-even: it needs enough (region, tile) items to fill the GPU).
inline bool mfma_pays(size_t m, unsigned ftiles, size_t P) { return m > 8 && m <= 32 && P * (size_t)ftiles >= 512; }
inline unsigned wide_grid_x(unsigned ftiles, size_t P)
{
    unsigned gx = 768u / ftiles;                                  // three workgroups per CU are resident (150-160 registers)
    if (gx < 1) gx = 1;
    if (gx > (P + 3) / 4) gx = (unsigned)((P + 3) / 4);           // a workgroup walks four regions at a time
    return gx;
}
inline size_t wide_smem(unsigned mt) { return (size_t)mt * NL * FT * sizeof(float) + 4 * (mt == 16 ? wide_shape<16>::xbytes : wide_shape<24>::xbytes); }
// The bit-count backward: a wave per region, three workgroups per CU resident (its 5 x MT sums and the rest take ~160
// registers at 24 taps: three waves per SIMD);
// the smallest grid that gives every wave the same number of regions as the resident grid would.
inline unsigned bits_grid_x(unsigned ftiles, size_t P)
{
    unsigned gx = 768u / ftiles;
    if (gx < 1) gx = 1;
    // at least two regions per wave: the fold of a workgroup's sums and its slab cost about as much as two regions
    // (measured on a calibration batch of 256 regions x 23 tiles: 26.7 us with two, 29.6 with three, 34.5 with five
    // regions per wave; the reduction of the slabs 7.9 / 7.1 / 6.5 us)
    if (gx > (P + 7) / 8) gx = (unsigned)((P + 7) / 8);
    const size_t per_wave = (P + (size_t)gx * 4 - 1) / ((size_t)gx * 4);
    return (unsigned)((P + 4 * per_wave - 1) / (4 * per_wave));
}
// Max pooling goes through it while the regions are short on average (it visits every 64-row chunk of a region to
// find each filter's winning row; the sparse kernel goes straight to that row).
inline bool bits_takes_max(size_t N, size_t P) { return N <= 128 * P; }
inline size_t bits_smem(unsigned) { return FOLD_BYTES; }
inline size_t sparse_smem(size_t m) { return m * SPARSE_ROWS * FT * sizeof(float); }
inline size_t dense_smem(unsigned mt)
{
    const size_t scan = ((size_t)mt * NL * FT + 4 * FT) * sizeof(float) + ((4 * XCH_SUBS * PSUB + mt - 1 + 7) & ~(size_t)3);
    return scan > FOLD_BYTES ? scan : FOLD_BYTES;                  // (the kernel's last act, the fold of its waves' sums, reuses the memory)
}

template <int PT, int MT>
int launch_fprop_mt(hipStream_t st, unsigned gx, unsigned ftiles, unsigned nw, size_t smem, const float* W, const float* bias, size_t m,
                     size_t F, const uint8_t* X, size_t N, const uint32_t* R, size_t P, float* pooled, uint32_t* argmax,
                     const unsigned* run_if_flag, unsigned long long* act)
{
    if (argmax) {
        auto kern = scanpool_fprop_kernel<PT, true, MT>;
        DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(nw * 64), smem, st, W, bias, (unsigned)m, (unsigned)F, X, N, R, P, pooled, argmax, run_if_flag, act);
    } else {
        auto kern = scanpool_fprop_kernel<PT, false, MT>;
        DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(nw * 64), smem, st, W, bias, (unsigned)m, (unsigned)F, X, N, R, P, pooled, argmax, run_if_flag, act);
    }
    return 0;
}

template <int PT>
int launch_fprop_wide(hipStream_t st, unsigned ftiles, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
                      const uint32_t* R, size_t P, float* pooled, uint32_t* argmax, unsigned long long* act)
{
    const unsigned mt = wide_tier(m);
    const size_t smem = wide_smem(mt);
    DBK_CHECK(smem <= lds_limit(), "ValueError: the wide forward kernel needs %zu bytes of LDS (limit %zu)", smem, lds_limit());
    const unsigned gx = wide_grid_x(ftiles, P);
    auto kern = argmax ? (mt == 16 ? scanpool_fprop_wide_kernel<PT, true, 16> : scanpool_fprop_wide_kernel<PT, true, 24>)
                       : (mt == 16 ? scanpool_fprop_wide_kernel<PT, false, 16> : scanpool_fprop_wide_kernel<PT, false, 24>);
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(256), smem, st, W, bias, (unsigned)m, (unsigned)F, X, N, R, P, pooled, argmax, act);
    DBK_LAUNCH_OK();
}

// The matrix-core forward: a workgroup holds a 64-filter tile (two waves per half) and walks two regions at a time.
inline unsigned mfma_grid_x(unsigned ftiles, size_t P)
{
    unsigned gx = 768u / ftiles;                                  // three workgroups per CU resident
    if (gx < 1) gx = 1;
    if (gx > (P + 1) / 2) gx = (unsigned)((P + 1) / 2);
    return gx;
}

template <int PT, int KS>
int launch_fprop_mfma_ks(hipStream_t st, unsigned ftiles, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
                         const uint32_t* R, size_t P, float* pooled, uint32_t* argmax, unsigned long long* act)
{
    const unsigned gx = mfma_grid_x(ftiles, P);
    auto kern = argmax ? (act ? scanpool_fprop_mfma_kernel<PT, true, true, KS> : scanpool_fprop_mfma_kernel<PT, true, false, KS>)
                       : (act ? scanpool_fprop_mfma_kernel<PT, false, true, KS> : scanpool_fprop_mfma_kernel<PT, false, false, KS>);
    hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(256), MFMA_SMEM, st, W, bias, (unsigned)m, (unsigned)F, X, N, R, P, pooled, argmax, act);
    DBK_LAUNCH_OK();
}

template <int PT>
int launch_fprop_mfma(hipStream_t st, unsigned ftiles, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
                      const uint32_t* R, size_t P, float* pooled, uint32_t* argmax, unsigned long long* act)
{
    switch ((mfma_ksteps(m) + 1) / 2) {
    case 1:  return launch_fprop_mfma_ks<PT, 2>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, argmax, act);
    case 2:  return launch_fprop_mfma_ks<PT, 4>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, argmax, act);
    case 3:  return launch_fprop_mfma_ks<PT, 6>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, argmax, act);
    default: return launch_fprop_mfma_ks<PT, 8>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, argmax, act);
    }
}

template <int PT>
int launch_fprop_pt(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
                    const uint32_t* R, size_t P, float* pooled, uint32_t* argmax, const unsigned* run_if_flag, unsigned long long* act)
{
    const unsigned nw = 4;
    const unsigned mt = m <= 8 ? 8 : (m <= 16 ? 16 : (m <= 24 ? 24 : (m <= 32 ? 32 : 0)));    // 0: any-length kernel
    const size_t smem = fprop_smem(mt, m);
    DBK_CHECK(smem <= lds_limit(), "ValueError: filter length %zu needs %zu bytes of LDS (limit %zu)", m, smem, lds_limit());
    unsigned ftiles = dbk::divup(F, FT);
    DBK_CHECK(ftiles <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
    if (!run_if_flag && mfma_pays(m, ftiles, P)) return launch_fprop_mfma<PT>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, argmax, act);
    const unsigned gx = fprop_grid_x(mt, ftiles, P);
    int rc = 0;
    switch (mt) {
    case 8:  rc = launch_fprop_mt<PT, 8>(st, gx, ftiles, nw, smem, W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag, act); break;
    case 16: rc = launch_fprop_mt<PT, 16>(st, gx, ftiles, nw, smem, W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag, act); break;
    case 24: rc = launch_fprop_mt<PT, 24>(st, gx, ftiles, nw, smem, W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag, act); break;
    case 32: rc = launch_fprop_mt<PT, 32>(st, gx, ftiles, nw, smem, W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag, act); break;
    default: rc = launch_fprop_mt<PT, 0>(st, gx, ftiles, nw, smem, W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag, act); break;
    }
    if (rc) return rc;
    DBK_LAUNCH_OK();
}

template <int PT, int MT>
int launch_dense(hipStream_t st, unsigned gx, unsigned ftiles, size_t smem, const float* W, const float* bias, size_t m, size_t F,
                  const uint8_t* X, size_t N, const uint32_t* R, size_t P, const float* pooled, const uint32_t* argmax,
                  const float* dpooled, const unsigned long long* act, float* slabs, size_t stride)
{
    if (act) {
        auto kern = scanpool_bprop_bits_kernel<PT, MT>;
        DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(256), smem, st, (unsigned)m, (unsigned)F, X, N, R, P, pooled, argmax, dpooled, act, slabs, stride);
        return 0;
    }
    auto kern = scanpool_bprop_dense_kernel<PT, MT>;
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(256), smem, st, W, bias, (unsigned)m, (unsigned)F, X, N, R, P, pooled, argmax, dpooled, slabs, stride);
    return 0;
}

template <int PT>
int launch_bprop_pt(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
                    const uint32_t* R, size_t P, const float* pooled, const uint32_t* argmax, const float* dpooled,
                    float* dW, float* dbias, bool overwrite, const unsigned long long* act)
{
    const unsigned ftiles = dbk::divup(F, FT);
    DBK_CHECK(ftiles <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
    const size_t nW = 4 * m * F, stride = nW + F;
    const unsigned mt = m <= 8 ? 8 : (m <= 16 ? 16 : (m <= 24 ? 24 : 0));    // the register budget of the dense kernel ends at 24 taps
    if (mt == 0) {
        // any filter length: one kernel does both halves through per-wave LDS tables
        unsigned nw = 4;
        const size_t lutb = PT == DBK_PT_MAX ? 0 : m * NL * FT * sizeof(float);
        auto need = [&](unsigned w) { return lutb + (size_t)w * (m * 4 * FT + FT) * sizeof(float) + w * XCH_SUBS * PSUB + m - 1; };
        while (nw > 1 && need(nw) > lds_limit()) nw >>= 1;
        const size_t smem = need(nw);
        DBK_CHECK(smem <= lds_limit(), "ValueError: filter length %zu needs %zu bytes of LDS (limit %zu)", m, smem, lds_limit());
        unsigned gx = 1024u / ftiles;
        if (gx < 1) gx = 1;
        if (gx > P) gx = (unsigned)P;
        float* slabs = (float*)dbk::workspace(stride * gx * sizeof(float), st);
        DBK_CHECK(slabs != nullptr, "MemoryError: could not allocate %zu bytes of scratch (%s)", stride * gx * sizeof(float), dbk::workspace_error());
        auto kern = scanpool_bprop_kernel<PT>;
        DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(nw * 64), smem, st, W, bias, (unsigned)m, (unsigned)F, X, N, R, P,
                           pooled, argmax, dpooled, slabs, stride);
        if (dbk::deferred_sums* later = dbk::deferred()) { later->slabs = slabs; later->slab_stride = stride; later->nslab = gx; }
        else hipLaunchKernelGGL(reduce_slabs_kernel, dim3(dbk::ew_grid(stride)), dim3(256), 0, st, dW, dbias, (const float*)slabs, nW, F, gx, overwrite);
        DBK_LAUNCH_OK();
    }
    // Average pooling without the forward pass's activity masks: the matrix-core forward writes them again (into the
    // stream's second scratch buffer, with its pooled values beside them), and the bit-count kernel takes them from
    // there; less than half the time of recomputing the map through the letter table.
    const size_t mask_bytes = N * ftiles * sizeof(unsigned long long), pooled_bytes = P * F * 2 * sizeof(float);
    if (PT != DBK_PT_MAX && !act && !dbk::deferred() && mfma_pays(m, ftiles, P) && mask_bytes + pooled_bytes <= ((size_t)1 << 30)) {   // (at most 1 GiB of scratch for it)
        unsigned char* scratch = (unsigned char*)dbk::workspace(mask_bytes + pooled_bytes, st, 1);
        DBK_CHECK(scratch != nullptr, "MemoryError: could not allocate %zu bytes of scratch (%s)", mask_bytes + pooled_bytes, dbk::workspace_error());
        unsigned long long* masks = reinterpret_cast<unsigned long long*>(scratch);
        const int rc = launch_fprop_mfma<PT>(st, ftiles, W, bias, m, F, X, N, R, P, reinterpret_cast<float*>(scratch + mask_bytes), nullptr, masks);
        if (rc) return rc;
        act = masks;
    }
    // with max+avg pooling the dense half carries the maxima along
    const bool max_bits = PT == DBK_PT_MAX && bits_takes_max(N, P);
    const unsigned gxs = PT == DBK_PT_MAX ? (max_bits ? bits_grid_x(ftiles, P) : sparse_grid_x(ftiles, P)) : 0u;
    const unsigned gxd = PT == DBK_PT_MAX ? 0u : act ? bits_grid_x(ftiles, P) : dense_grid_x(mt, ftiles, P);
    const size_t smem_s = sparse_smem(m), smem_d = dense_smem(mt);
    DBK_CHECK(smem_s <= lds_limit() && smem_d <= lds_limit(), "ValueError: filter length %zu does not fit in LDS", m);
    float* slabs = (float*)dbk::workspace(stride * (gxs + gxd) * sizeof(float), st);
    DBK_CHECK(slabs != nullptr, "MemoryError: could not allocate %zu bytes of scratch (%s)", stride * (gxs + gxd) * sizeof(float), dbk::workspace_error());
    if (gxs && max_bits) {
        auto kern = mt == 8 ? scanpool_bprop_bits_kernel<DBK_PT_MAX, 8> : mt == 16 ? scanpool_bprop_bits_kernel<DBK_PT_MAX, 16> : scanpool_bprop_bits_kernel<DBK_PT_MAX, 24>;
        const size_t smem_b = bits_smem(mt);
        DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_b));
        hipLaunchKernelGGL(kern, dim3(gxs, ftiles), dim3(256), smem_b, st, (unsigned)m, (unsigned)F, X, N, R, P, pooled, argmax, dpooled,
                           (const unsigned long long*)nullptr, slabs, stride);
    } else if (gxs) {
        constexpr int PS = PT == DBK_PT_AVG ? DBK_PT_MAX : PT;
        auto kern = mt == 8 ? scanpool_bprop_sparse_kernel<PS, 8> : mt == 16 ? scanpool_bprop_sparse_kernel<PS, 16> : scanpool_bprop_sparse_kernel<PS, 24>;
        DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_s));
        hipLaunchKernelGGL(kern, dim3(gxs, ftiles), dim3(64), smem_s, st, (unsigned)m, (unsigned)F, X, N, P, pooled, argmax, dpooled, slabs, stride);
    }
    if (gxd) {
        constexpr int PD = PT == DBK_PT_MAX ? DBK_PT_AVG : PT;
        float* sd = slabs + stride * gxs;
        int rc;
        if (mt == 8) rc = launch_dense<PD, 8>(st, gxd, ftiles, smem_d, W, bias, m, F, X, N, R, P, pooled, argmax, dpooled, act, sd, stride);
        else if (mt == 16) rc = launch_dense<PD, 16>(st, gxd, ftiles, smem_d, W, bias, m, F, X, N, R, P, pooled, argmax, dpooled, act, sd, stride);
        else rc = launch_dense<PD, 24>(st, gxd, ftiles, smem_d, W, bias, m, F, X, N, R, P, pooled, argmax, dpooled, act, sd, stride);
        if (rc) return rc;
    }
    if (dbk::deferred_sums* later = dbk::deferred()) { later->slabs = slabs; later->slab_stride = stride; later->nslab = gxs + gxd; }
    else hipLaunchKernelGGL(reduce_slabs_kernel, dim3(dbk::ew_grid(stride)), dim3(256), 0, st, dW, dbias, (const float*)slabs, nW, F, gxs + gxd, overwrite);
    DBK_LAUNCH_OK();
}

int fprop_mfma(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
               const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax, unsigned long long* act)
{
    const unsigned ftiles = dbk::divup(F, FT);
    DBK_CHECK(ftiles <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
    switch (ptype) {
    case DBK_PT_MAX: return launch_fprop_mfma<DBK_PT_MAX>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, argmax, act);
    case DBK_PT_AVG: return launch_fprop_mfma<DBK_PT_AVG>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, nullptr, act);
    default:         return launch_fprop_mfma<DBK_PT_ALL>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, argmax, act);
    }
}

int fprop_wide(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
               const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax, unsigned long long* act)
{
    const unsigned ftiles = dbk::divup(F, FT);
    DBK_CHECK(ftiles <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
    switch (ptype) {
    case DBK_PT_MAX: return launch_fprop_wide<DBK_PT_MAX>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, argmax, act);
    case DBK_PT_AVG: return launch_fprop_wide<DBK_PT_AVG>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, nullptr, act);
    default:         return launch_fprop_wide<DBK_PT_ALL>(st, ftiles, W, bias, m, F, X, N, R, P, pooled, argmax, act);
    }
}

int fprop(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
          const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax, const unsigned* run_if_flag,
          unsigned long long* act)
{
    switch (ptype) {
    case DBK_PT_MAX: return launch_fprop_pt<DBK_PT_MAX>(st, W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag, act);
    case DBK_PT_AVG: return launch_fprop_pt<DBK_PT_AVG>(st, W, bias, m, F, X, N, R, P, pooled, nullptr, run_if_flag, act);
    default:         return launch_fprop_pt<DBK_PT_ALL>(st, W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag, act);
    }
}

// ---------------------------------------------------------------------------------------------
// several model groups in one launch
// ---------------------------------------------------------------------------------------------
// Workgroups first[g] .. first[g+1]-1 of the launch are group g's grid of gx[g] by ftiles[g], x fastest. The
// argument block travels by value in the kernel-argument segment.
struct multi_args {
    unsigned n, m;
    size_t N, P;
    const uint32_t* R;
    unsigned first[dbk::MULTI_MAX + 1], gx[dbk::MULTI_MAX], ftiles[dbk::MULTI_MAX];
    unsigned wide[dbk::MULTI_MAX];                                 // the group goes through the many-regions kernel body (forward: the matrix-core scan; backward: a wave per region)
    dbk::scan_group g[dbk::MULTI_MAX];
};

__device__ __forceinline__ unsigned multi_locate(const multi_args& a, wg_t& wg)
{
    unsigned g = 0;
    while (g + 1 < a.n && blockIdx.x >= a.first[g + 1]) ++g;
    const unsigned local = blockIdx.x - a.first[g];
    wg = wg_t{local % a.gx[g], local / a.gx[g], a.gx[g], a.ftiles[g]};
    return g;
}

template <int MT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MT == 24 ? 3 : 1))) void scanpool_fprop_multi_kernel(const multi_args a)
{
    wg_t wg;
    const unsigned gi = multi_locate(a, wg);
    const dbk::scan_group& j = a.g[gi];
    if constexpr (MT == 16 || MT == 24) {
        if (a.wide[gi]) {
            if (j.ptype == DBK_PT_MAX)
                scanpool_fprop_mfma_body<DBK_PT_MAX, true, false, MT / 4>(wg, j.W, j.bias, a.m, j.F, j.X, a.N, a.R, a.P, j.pooled, j.argmax, nullptr);
            else if (j.ptype == DBK_PT_ALL)
                scanpool_fprop_mfma_body<DBK_PT_ALL, true, true, MT / 4>(wg, j.W, j.bias, a.m, j.F, j.X, a.N, a.R, a.P, j.pooled, j.argmax, j.act);
            else
                scanpool_fprop_mfma_body<DBK_PT_AVG, false, true, MT / 4>(wg, j.W, j.bias, a.m, j.F, j.X, a.N, a.R, a.P, j.pooled, nullptr, j.act);
            return;
        }
    }
    if (j.ptype == DBK_PT_MAX)
        scanpool_fprop_body<DBK_PT_MAX, true, MT>(wg, j.W, j.bias, a.m, j.F, j.X, a.N, a.R, a.P, j.pooled, j.argmax, nullptr, nullptr);
    else if (j.ptype == DBK_PT_ALL)
        scanpool_fprop_body<DBK_PT_ALL, true, MT>(wg, j.W, j.bias, a.m, j.F, j.X, a.N, a.R, a.P, j.pooled, j.argmax, nullptr, j.act);
    else
        scanpool_fprop_body<DBK_PT_AVG, false, MT>(wg, j.W, j.bias, a.m, j.F, j.X, a.N, a.R, a.P, j.pooled, nullptr, nullptr, j.act);
}

// The bit-count kernel; for max pooling over long regions the one-wave sparse kernel in the first wave of the
// workgroup (the other waves leave at once).
template <int MT>
__global__ __launch_bounds__(256) void scanpool_bprop_multi_kernel(const multi_args a)
{
    wg_t wg;
    const unsigned gi = multi_locate(a, wg);
    const dbk::scan_group& j = a.g[gi];
    if (j.ptype == DBK_PT_MAX) {
        if (a.wide[gi])
            scanpool_bprop_bits_body<DBK_PT_MAX, MT>(wg, a.m, j.F, j.X, a.N, a.R, a.P, j.pooled, j.argmax, j.dpooled, nullptr, j.slabs, j.slab_stride);
        else if (threadIdx.x < 64)
            scanpool_bprop_sparse_body<DBK_PT_MAX, MT>(wg, a.m, j.F, j.X, a.N, a.P, j.pooled, j.argmax, j.dpooled, j.slabs, j.slab_stride);
    } else if (j.ptype == DBK_PT_ALL) {
        scanpool_bprop_bits_body<DBK_PT_ALL, MT>(wg, a.m, j.F, j.X, a.N, a.R, a.P, j.pooled, j.argmax, j.dpooled, j.act, j.slabs, j.slab_stride);
    } else {
        scanpool_bprop_bits_body<DBK_PT_AVG, MT>(wg, a.m, j.F, j.X, a.N, a.R, a.P, j.pooled, j.argmax, j.dpooled, j.act, j.slabs, j.slab_stride);
    }
}

inline unsigned multi_tier(size_t m) { return m <= 8 ? 8u : (m <= 16 ? 16u : (m <= 24 ? 24u : 0u)); }

template <typename K>
int launch_multi(K kern, hipStream_t st, size_t smem, const multi_args& a)
{
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(a.first[a.n]), dim3(256), smem, st, a);
    DBK_LAUNCH_OK();
}

}  // namespace dbk_scanpool_general

namespace dbk_scanpool_kmer {
bool takes(size_t m, size_t F, size_t N, size_t P);
}

namespace dbk {

using namespace dbk_scanpool_general;

bool scan_multi_takes(size_t m, size_t N, size_t P, unsigned n, const scan_group* g)
{
    if (n < 1 || n > MULTI_MAX || multi_tier(m) == 0 || P == 0 || N == 0) return false;
    for (unsigned i = 0; i < n; ++i) {
        if (g[i].F == 0 || dbk::divup(g[i].F, FT) > 65535u) return false;
        if (g[i].ptype != DBK_PT_MAX && g[i].ptype != DBK_PT_AVG && g[i].ptype != DBK_PT_ALL) return false;
        if (g[i].ptype != DBK_PT_MAX && !g[i].act) return false;      // the dense backward kernel here is the mask-driven one
        if (g[i].ptype != DBK_PT_AVG && !g[i].argmax) return false;
        // a max-pooling group on a batch large enough for the k-mer table goes there when stepped alone (other sums, other bits)
        if (g[i].ptype == DBK_PT_MAX && dbk_scanpool_kmer::takes(m, g[i].F, N, P)) return false;
    }
    return fprop_smem(multi_tier(m), m) <= lds_limit() && wide_smem(24) <= lds_limit() && sparse_smem(m) <= lds_limit() && dense_smem(multi_tier(m)) <= lds_limit();
}

int scan_fprop_multi(hipStream_t st, size_t m, size_t N, const uint32_t* R, size_t P, unsigned n, const scan_group* g)
{
    const unsigned mt = multi_tier(m);
    multi_args a;
    a.n = n; a.m = (unsigned)m; a.N = N; a.P = P; a.R = R;
    a.first[0] = 0;
    bool any_wide = false;
    unsigned tiles = 0;
    for (unsigned i = 0; i < n; ++i) tiles += dbk::divup(g[i].F, FT);
    for (unsigned i = 0; i < n; ++i) {
        a.g[i] = g[i];
        a.ftiles[i] = dbk::divup(g[i].F, FT);
        a.wide[i] = mfma_pays(m, a.ftiles[i], P) && m <= 24;      // the kernel body the group's own launch would choose
        // the groups share the GPU: the grids are sized so that all of them are resident together, and a workgroup
        // amortises its filter tile's table over more regions (a region's results do not depend on the grid)
        a.gx[i] = a.wide[i] ? mfma_grid_x(tiles, P) : fprop_grid_x(mt, tiles, P);
        a.first[i + 1] = a.first[i] + a.gx[i] * a.ftiles[i];
        if (a.wide[i]) any_wide = true;
    }
    size_t smem = fprop_smem(mt, m);
    if (any_wide && MFMA_SMEM > smem) smem = MFMA_SMEM;
    if (mt == 8) return launch_multi(scanpool_fprop_multi_kernel<8>, st, smem, a);
    if (mt == 16) return launch_multi(scanpool_fprop_multi_kernel<16>, st, smem, a);
    return launch_multi(scanpool_fprop_multi_kernel<24>, st, smem, a);
}

int scan_bprop_multi(hipStream_t st, size_t m, size_t N, const uint32_t* R, size_t P, unsigned n, scan_group* g)
{
    const unsigned mt = multi_tier(m);
    multi_args a;
    a.n = n; a.m = (unsigned)m; a.N = N; a.P = P; a.R = R;
    a.first[0] = 0;
    size_t total = 0;
    for (unsigned i = 0; i < n; ++i) {
        a.ftiles[i] = dbk::divup(g[i].F, FT);
        // as the group's own launch would choose: the bit-count kernel, or the sparse one for max pooling over long regions
        a.wide[i] = g[i].ptype != DBK_PT_MAX || bits_takes_max(N, P);
        a.gx[i] = a.wide[i] ? bits_grid_x(a.ftiles[i], P) : sparse_grid_x(a.ftiles[i], P);
        a.first[i + 1] = a.first[i] + a.gx[i] * a.ftiles[i];
        g[i].slab_stride = 4 * m * (size_t)g[i].F + g[i].F;
        g[i].nslab = a.gx[i];
        total += g[i].slab_stride * a.gx[i];
    }
    float* slabs = (float*)dbk::workspace(total * sizeof(float), st);
    DBK_CHECK(slabs != nullptr, "MemoryError: could not allocate %zu bytes of scratch (%s)", total * sizeof(float), dbk::workspace_error());
    for (unsigned i = 0; i < n; ++i) {
        g[i].slabs = slabs;
        slabs += g[i].slab_stride * a.gx[i];
        a.g[i] = g[i];
    }
    const size_t ss = sparse_smem(m), sd = dense_smem(mt);
    const size_t smem = ss > sd ? ss : sd;
    if (mt == 8) return launch_multi(scanpool_bprop_multi_kernel<8>, st, smem, a);
    if (mt == 16) return launch_multi(scanpool_bprop_multi_kernel<16>, st, smem, a);
    return launch_multi(scanpool_bprop_multi_kernel<24>, st, smem, a);
}

}  // namespace dbk

namespace dbk_scanpool_kmer {
// Fast path (k-mer lookup table); returns -1 when the shape is outside what it handles.
int fprop(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
          const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax);
}

extern "C" {

int dbk_scanpool_fprop_general(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                               const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                               float* pooled, uint32_t* argmax, uint64_t* act)
{
    // sum pooling has no fused kernel: the operator chain computes it (no activity masks are written)
    if (ptype == DBK_PT_SUM) return dbk_scanpool_fprop_unfused(stream, W, bias, m, nfilter, X, N, regions, nregion, 2, ptype, pooled, argmax);
    DBK_CHECK(ptype == DBK_PT_MAX || ptype == DBK_PT_AVG || ptype == DBK_PT_ALL, "ValueError: unknown pooling type %d", ptype);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    DBK_CHECK(!(argmax && ptype == DBK_PT_AVG), "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    // argmax entries are flat 32-bit indices row*nfilter + f into the (virtual) map, as in the reference (uindex_t)
    DBK_CHECK(!argmax || (double)N * (double)nfilter <= 4294967296.0,
              "ValueError: %zu rows x %zu filters overflow the 32-bit argmax index; score in smaller batches or without argmax", N, nfilter);
    if (nfilter == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && regions && pooled, "ValueError: null pointer argument");
    return dbk_scanpool_general::fprop(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax, nullptr,
                                       reinterpret_cast<unsigned long long*>(act));
}

int dbk_scanpool_fprop_wide(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                            const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                            float* pooled, uint32_t* argmax, uint64_t* act)
{
    DBK_CHECK(ptype == DBK_PT_MAX || ptype == DBK_PT_AVG || ptype == DBK_PT_ALL, "ValueError: fused pooling type must be max, avg or all (got %d)", ptype);
    DBK_CHECK(m > 8 && m <= 24, "NotImplementedError: the wide forward kernel takes filters of 9 to 24 taps (got %zu)", m);
    DBK_CHECK(!(argmax && ptype == DBK_PT_AVG), "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    DBK_CHECK(!argmax || (double)N * (double)nfilter <= 4294967296.0,
              "ValueError: %zu rows x %zu filters overflow the 32-bit argmax index; score in smaller batches or without argmax", N, nfilter);
    if (nfilter == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && regions && pooled, "ValueError: null pointer argument");
    return dbk_scanpool_general::fprop_wide(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax,
                                            reinterpret_cast<unsigned long long*>(act));
}

int dbk_scanpool_fprop_mfma(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                            const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                            float* pooled, uint32_t* argmax, uint64_t* act)
{
    DBK_CHECK(ptype == DBK_PT_MAX || ptype == DBK_PT_AVG || ptype == DBK_PT_ALL, "ValueError: fused pooling type must be max, avg or all (got %d)", ptype);
    DBK_CHECK(dbk_scanpool_general::mfma_takes(m), "NotImplementedError: the matrix-core forward kernel takes filters of 1 to 32 taps (got %zu)", m);
    DBK_CHECK(!(argmax && ptype == DBK_PT_AVG), "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    DBK_CHECK(!argmax || (double)N * (double)nfilter <= 4294967296.0,
              "ValueError: %zu rows x %zu filters overflow the 32-bit argmax index; score in smaller batches or without argmax", N, nfilter);
    if (nfilter == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && regions && pooled, "ValueError: null pointer argument");
    return dbk_scanpool_general::fprop_mfma(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax,
                                            reinterpret_cast<unsigned long long*>(act));
}

int dbk_scanpool_fprop(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                       const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                       float* pooled, uint32_t* argmax, uint64_t* act)
{
    // sum pooling has no fused kernel: the operator chain computes it (no activity masks are written)
    if (ptype == DBK_PT_SUM) return dbk_scanpool_fprop_unfused(stream, W, bias, m, nfilter, X, N, regions, nregion, 2, ptype, pooled, argmax);
    DBK_CHECK(ptype == DBK_PT_MAX || ptype == DBK_PT_AVG || ptype == DBK_PT_ALL, "ValueError: unknown pooling type %d", ptype);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    DBK_CHECK(!(argmax && ptype == DBK_PT_AVG), "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    // argmax entries are flat 32-bit indices row*nfilter + f into the (virtual) map, as in the reference (uindex_t)
    DBK_CHECK(!argmax || (double)N * (double)nfilter <= 4294967296.0,
              "ValueError: %zu rows x %zu filters overflow the 32-bit argmax index; score in smaller batches or without argmax", N, nfilter);
    if (nfilter == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && regions && pooled, "ValueError: null pointer argument");
    // the activity masks are written by the general kernel only (the k-mer table is worth its set-up for bulk scoring,
    // where no backward pass follows)
    if (!act) {
        int rc = dbk_scanpool_kmer::fprop(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax);
        if (rc >= 0) return rc;
    }
    return dbk_scanpool_general::fprop(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax, nullptr,
                                       reinterpret_cast<unsigned long long*>(act));
}

int dbk_scanpool_bprop(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                       const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                       const float* pooled, const uint32_t* argmax, const float* dpooled, float* dW, float* dbias, int overwrite,
                       const uint64_t* act)
{
    using namespace dbk_scanpool_general;
    if (ptype == DBK_PT_SUM && !dbk::deferred())
        return dbk_scanpool_bprop_unfused(stream, W, bias, m, nfilter, X, N, regions, nregion, 2, ptype, argmax, dpooled, dW, dbias, overwrite);
    DBK_CHECK(ptype == DBK_PT_MAX || ptype == DBK_PT_AVG || ptype == DBK_PT_ALL, "ValueError: fused pooling type must be max, avg or all (got %d)", ptype);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    if (nfilter == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && dW && dbias, "ValueError: null pointer argument");
    if (nregion == 0 && dbk::deferred()) {
        dbk::deferred()->slabs = nullptr;                          // zero slabs: the gradient is zero
        dbk::deferred()->slab_stride = 4 * m * nfilter + nfilter;
        dbk::deferred()->nslab = 0;
        dbk::clear_error();
        return 0;
    }
    if (nregion == 0) {
        // no regions: the bias gradient is written as zero by the slab reduction over zero slabs
        // (a kernel rather than a memset, so that the call can sit in a captured graph)
        hipLaunchKernelGGL(reduce_slabs_kernel, dim3(dbk::ew_grid(nfilter)), dim3(256), 0, dbk::as_stream(stream), dW, dbias,
                           (const float*)nullptr, (size_t)(overwrite ? 4 * m * nfilter : 0), nfilter, 0u, overwrite != 0);
        DBK_LAUNCH_OK();
    }
    DBK_CHECK(ptype == DBK_PT_AVG || argmax != nullptr, "ValueError: pooledmaps_argmax must be specified for max pooling.");
    DBK_CHECK(X && regions && pooled && dpooled, "ValueError: null pointer argument");
    hipStream_t st = dbk::as_stream(stream);
    const unsigned long long* am = reinterpret_cast<const unsigned long long*>(act);
    switch (ptype) {
    case DBK_PT_MAX: return launch_bprop_pt<DBK_PT_MAX>(st, W, bias, m, nfilter, X, N, regions, nregion, pooled, argmax, dpooled, dW, dbias, overwrite != 0, am);
    case DBK_PT_AVG: return launch_bprop_pt<DBK_PT_AVG>(st, W, bias, m, nfilter, X, N, regions, nregion, pooled, argmax, dpooled, dW, dbias, overwrite != 0, am);
    default:         return launch_bprop_pt<DBK_PT_ALL>(st, W, bias, m, nfilter, X, N, regions, nregion, pooled, argmax, dpooled, dW, dbias, overwrite != 0, am);
    }
}

}  // extern "C"

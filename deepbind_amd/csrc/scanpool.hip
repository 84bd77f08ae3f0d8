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

// Stages letters for absolute positions [c0, c0+cnt) into xl; past the end of X -> "nothing".
__device__ __forceinline__ void stage(uint8_t* xl, const uint8_t* __restrict__ X, size_t N, size_t c0, unsigned cnt)
{
    for (unsigned t = threadIdx.x; t < cnt; t += blockDim.x) {
        size_t g = c0 + t;
        xl[t] = g < N ? (uint8_t)letter_of(X[g]) : (uint8_t)5;
    }
}

template <int PT, bool WANT_ARGMAX>
__global__ __launch_bounds__(256) void scanpool_fprop_kernel(const float* __restrict__ W, const float* __restrict__ bias,
                                                             unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                             const uint32_t* __restrict__ R, size_t P,
                                                             float* __restrict__ pooled, uint32_t* __restrict__ argmax,
                                                             const unsigned* __restrict__ run_if_flag)
{
    extern __shared__ __align__(16) unsigned char smem[];
    // when given, the launch only does work if the device flag is set (fallback behind the k-mer kernel)
    if (run_if_flag && run_if_flag[0] == 0) return;
    const unsigned nw = blockDim.x >> 6;
    const unsigned chunk = nw * XCH_SUBS * PSUB;
    float* lut = reinterpret_cast<float*>(smem);
    float* red = lut + (size_t)m * NL * FT;                       // [nw][3][FT]: max, index, sum
    uint8_t* xl = reinterpret_cast<uint8_t*>(red + (size_t)nw * 3 * FT);

    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned f0 = blockIdx.y * FT, f = f0 + lane;
    const size_t n = N + 1 >= (size_t)m + 1 ? N - m + 1 : 0;    // rows the scan defines; later rows are relu(bias)
    build_letter_table(lut, W, m, F, f0);
    const float bf = f < F ? bias[f] : 0.0f;

    for (size_t r = blockIdx.x; r < P; r += gridDim.x) {
        const size_t a = R[2 * r], b = R[2 * r + 1];
        float mx = -1.0f, sum = 0.0f;
        size_t xi = a;
        for (size_t c0 = a; c0 < b; c0 += chunk) {
            const unsigned rows = (unsigned)((b - c0) < chunk ? (b - c0) : chunk);
            __syncthreads();
            stage(xl, X, N, c0, rows + m - 1);
            __syncthreads();
            for (unsigned s = 0; s < XCH_SUBS; ++s) {
                const unsigned p0 = (s * nw + wave) * PSUB;
                if (p0 >= rows) break;
                float acc[PSUB];
                scan16(lut, xl, m, p0, lane, acc);
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
                                                             float* __restrict__ slabW, float* __restrict__ slabB)
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
    float* outW = slabW + (size_t)blockIdx.x * (4 * m) * F;
    for (unsigned e = threadIdx.x; e < tab; e += blockDim.x) {
        float s = acc_tab[e];
        for (unsigned w = 1; w < nw; ++w) s += acc_tab[(size_t)w * tab + e];
        const unsigned row = e / FT, fl = e % FT;
        if (f0 + fl < F) outW[(size_t)row * F + f0 + fl] = s;
    }
    if (wave == 0 && f < F) {
        float s = dbacc[lane];
        for (unsigned w = 1; w < nw; ++w) s += dbacc[w * FT + lane];
        slabB[(size_t)blockIdx.x * F + f] = s;
    }
}

// dst[e] (+)= fixed-shape tree sum over slabs
template <bool ACCUMULATE>
__global__ void reduce_slabs_kernel(float* __restrict__ dst, const float* __restrict__ slabs, size_t nelem, unsigned nslab)
{
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < nelem; e += (size_t)gridDim.x * blockDim.x) {
        float total = 0.0f;
        for (unsigned base = 0; base < nslab; base += 8) {
            float buf[8];
            for (unsigned s = 0; s < 8; ++s) buf[s] = base + s < nslab ? slabs[(size_t)(base + s) * nelem + e] : 0.0f;
            total += ((buf[0] + buf[1]) + (buf[2] + buf[3])) + ((buf[4] + buf[5]) + (buf[6] + buf[7]));
        }
        dst[e] = ACCUMULATE ? dst[e] + total : total;
    }
}

template <int PT>
int launch_fprop_pt(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
                    const uint32_t* R, size_t P, float* pooled, uint32_t* argmax, const unsigned* run_if_flag)
{
    const unsigned nw = 4;
    const unsigned chunk = nw * XCH_SUBS * PSUB;
    size_t smem = m * NL * FT * sizeof(float) + nw * 3 * FT * sizeof(float) + chunk + m - 1;
    DBK_CHECK(smem <= lds_limit(), "ValueError: filter length %zu needs %zu bytes of LDS (limit %zu)", m, smem, lds_limit());
    unsigned ftiles = dbk::divup(F, FT);
    DBK_CHECK(ftiles <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
    unsigned gx = 4096u / ftiles;
    if (gx < 1) gx = 1;
    if (gx > P) gx = (unsigned)P;
    if (argmax) {
        auto kern = scanpool_fprop_kernel<PT, true>;
        DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(nw * 64), smem, st, W, bias, (unsigned)m, (unsigned)F, X, N, R, P, pooled, argmax, run_if_flag);
    } else {
        auto kern = scanpool_fprop_kernel<PT, false>;
        DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(nw * 64), smem, st, W, bias, (unsigned)m, (unsigned)F, X, N, R, P, pooled, argmax, run_if_flag);
    }
    DBK_LAUNCH_OK();
}

template <int PT>
int launch_bprop_pt(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
                    const uint32_t* R, size_t P, const float* pooled, const uint32_t* argmax, const float* dpooled,
                    float* dW, float* dbias)
{
    unsigned nw = 4;
    const size_t lutb = PT == DBK_PT_MAX ? 0 : m * NL * FT * sizeof(float);
    auto need = [&](unsigned w) { return lutb + (size_t)w * (m * 4 * FT + FT) * sizeof(float) + w * XCH_SUBS * PSUB + m - 1; };
    while (nw > 1 && need(nw) > lds_limit()) nw >>= 1;
    size_t smem = need(nw);
    DBK_CHECK(smem <= lds_limit(), "ValueError: filter length %zu needs %zu bytes of LDS (limit %zu)", m, smem, lds_limit());
    unsigned ftiles = dbk::divup(F, FT);
    DBK_CHECK(ftiles <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
    unsigned gx = 1024u / ftiles;
    if (gx < 1) gx = 1;
    if (gx > P) gx = (unsigned)P;
    const size_t nW = 4 * m * F;
    float* slabW = (float*)dbk::workspace((nW + F) * gx * sizeof(float));
    DBK_CHECK(slabW != nullptr, "MemoryError: could not allocate %zu bytes of scratch", (nW + F) * gx * sizeof(float));
    float* slabB = slabW + nW * gx;
    auto kern = scanpool_bprop_kernel<PT>;
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(gx, ftiles), dim3(nw * 64), smem, st, W, bias, (unsigned)m, (unsigned)F, X, N, R, P,
                       pooled, argmax, dpooled, slabW, slabB);
    hipLaunchKernelGGL(reduce_slabs_kernel<true>, dim3(dbk::ew_grid(nW)), dim3(256), 0, st, dW, (const float*)slabW, nW, gx);
    hipLaunchKernelGGL(reduce_slabs_kernel<false>, dim3(dbk::ew_grid(F)), dim3(256), 0, st, dbias, (const float*)slabB, F, gx);
    DBK_LAUNCH_OK();
}

int fprop(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
          const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax, const unsigned* run_if_flag)
{
    switch (ptype) {
    case DBK_PT_MAX: return launch_fprop_pt<DBK_PT_MAX>(st, W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag);
    case DBK_PT_AVG: return launch_fprop_pt<DBK_PT_AVG>(st, W, bias, m, F, X, N, R, P, pooled, nullptr, run_if_flag);
    default:         return launch_fprop_pt<DBK_PT_ALL>(st, W, bias, m, F, X, N, R, P, pooled, argmax, run_if_flag);
    }
}

}  // namespace dbk_scanpool_general

namespace dbk_scanpool_kmer {
// Fast path (k-mer lookup table); returns -1 when the shape is outside what it handles.
int fprop(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
          const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax);
}

extern "C" {

int dbk_scanpool_fprop_general(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                               const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                               float* pooled, uint32_t* argmax)
{
    DBK_CHECK(ptype == DBK_PT_MAX || ptype == DBK_PT_AVG || ptype == DBK_PT_ALL, "ValueError: fused pooling type must be max, avg or all (got %d)", ptype);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    DBK_CHECK(!(argmax && ptype == DBK_PT_AVG), "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    if (nfilter == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && regions && pooled, "ValueError: null pointer argument");
    return dbk_scanpool_general::fprop(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax, nullptr);
}

int dbk_scanpool_fprop(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                       const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                       float* pooled, uint32_t* argmax)
{
    DBK_CHECK(ptype == DBK_PT_MAX || ptype == DBK_PT_AVG || ptype == DBK_PT_ALL, "ValueError: fused pooling type must be max, avg or all (got %d)", ptype);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    DBK_CHECK(!(argmax && ptype == DBK_PT_AVG), "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    if (nfilter == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && regions && pooled, "ValueError: null pointer argument");
    int rc = dbk_scanpool_kmer::fprop(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax);
    if (rc >= 0) return rc;
    return dbk_scanpool_general::fprop(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax, nullptr);
}

int dbk_scanpool_bprop(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                       const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                       const float* pooled, const uint32_t* argmax, const float* dpooled, float* dW, float* dbias)
{
    using namespace dbk_scanpool_general;
    DBK_CHECK(ptype == DBK_PT_MAX || ptype == DBK_PT_AVG || ptype == DBK_PT_ALL, "ValueError: fused pooling type must be max, avg or all (got %d)", ptype);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    DBK_CHECK(ptype == DBK_PT_AVG || argmax != nullptr, "ValueError: pooledmaps_argmax must be specified for max pooling.");
    if (nfilter == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && dW && dbias, "ValueError: null pointer argument");
    if (nregion == 0) {
        DBK_HIP(hipMemsetAsync(dbias, 0, nfilter * sizeof(float), dbk::as_stream(stream)));
        dbk::clear_error();
        return 0;
    }
    DBK_CHECK(regions && pooled && dpooled, "ValueError: null pointer argument");
    hipStream_t st = dbk::as_stream(stream);
    switch (ptype) {
    case DBK_PT_MAX: return launch_bprop_pt<DBK_PT_MAX>(st, W, bias, m, nfilter, X, N, regions, nregion, pooled, argmax, dpooled, dW, dbias);
    case DBK_PT_AVG: return launch_bprop_pt<DBK_PT_AVG>(st, W, bias, m, nfilter, X, N, regions, nregion, pooled, argmax, dpooled, dW, dbias);
    default:         return launch_bprop_pt<DBK_PT_ALL>(st, W, bias, m, nfilter, X, N, regions, nregion, pooled, argmax, dpooled, dW, dbias);
    }
}

}  // extern "C"

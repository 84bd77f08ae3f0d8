// Motif scan over an ordinal sequence: forward map, filter gradient, input gradient.
//
// Layout shared by the three kernels: one lane per filter (64 filters per workgroup tile), so a
// wave's 64 lanes read 64 consecutive floats of the [tap][letter][filter] table in LDS and write /
// read 64 consecutive floats of a row of the (N, F) map in HBM. The sequence bytes are mapped to a
// 6-letter alphabet once per tile and kept in LDS: 0..3 = A,C,G,T, 4 = "mean of the four"
// (N, padding and every other code), 5 = "contributes nothing" (code 254).
//
// Reference semantics: kangaroo_smat/corr1ord.cuh:139-157 (forward, taps accumulated in ascending
// order), corr1ord_bprop.cuh:91-137 (filter gradient), corr1ord_bprop.cu:191-201 (input gradient).
#include "dbk_common.h"
#include "scan_common.h"

namespace {

using namespace dbk_scan;

// ---------------------------------------------------------------------------------------------
// forward: Z[i, f] for i in [0, n)
// ---------------------------------------------------------------------------------------------
template <typename T, int NW, int PW>   // NW waves per workgroup, PW positions per wave
__global__ __launch_bounds__(NW * 64) void corr1ord_kernel(const T* __restrict__ W, unsigned m, unsigned F,
                                                           const uint8_t* __restrict__ X, size_t n, T* __restrict__ Z)
{
    extern __shared__ __align__(16) unsigned char smem[];
    T* lut = reinterpret_cast<T*>(smem);
    uint8_t* xl = smem + (size_t)m * NL * FT * sizeof(T);

    const unsigned f0 = blockIdx.y * FT;
    const size_t i0 = (size_t)blockIdx.x * (NW * PW);
    const unsigned span = NW * PW + m - 1;

    build_letter_table(lut, W, m, F, f0);
    for (unsigned t = threadIdx.x; t < span; t += blockDim.x) {
        size_t g = i0 + t;
        xl[t] = (g < n + m - 1) ? (uint8_t)letter_of(X[g]) : (uint8_t)5;
    }
    __syncthreads();

    const unsigned lane = threadIdx.x & 63;
    const unsigned wave = threadIdx.x >> 6;
    const unsigned f = f0 + lane;
    for (unsigned sub = 0; sub < PW; sub += PSUB) {
        const unsigned p0 = wave * PW + sub;
        if (i0 + p0 >= n) break;
        T acc[PSUB];
#pragma unroll
        for (int p = 0; p < PSUB; ++p) acc[p] = (T)0;
        for (unsigned j = 0; j < m; ++j) {
            const T* row = lut + (size_t)j * NL * FT + lane;
            const uint8_t* xs = xl + p0 + j;
#pragma unroll
            for (int p = 0; p < PSUB; ++p) acc[p] += row[(unsigned)xs[p] * FT];
        }
        if (f < F) {
#pragma unroll
            for (int p = 0; p < PSUB; ++p) {
                size_t i = i0 + p0 + p;
                if (i < n) Z[i * F + f] = acc[p];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// filter gradient, pass 1: per-workgroup partial sums in LDS, one private table per wave
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void corr1ord_bprop_W_partial_kernel(T* __restrict__ partial, unsigned m, unsigned F,
                                                const uint8_t* __restrict__ X, size_t n, const T* __restrict__ dZ,
                                                unsigned chunk, unsigned nchunk_total)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const unsigned nw = blockDim.x >> 6;
    const unsigned tab = m * 4 * FT;                       // elements per wave-private table
    T* acc = reinterpret_cast<T*>(smem);
    uint8_t* xl = smem + (size_t)nw * tab * sizeof(T);

    const unsigned lane = threadIdx.x & 63;
    const unsigned wave = threadIdx.x >> 6;
    const unsigned f0 = blockIdx.x * FT;
    const unsigned f = f0 + lane;
    const unsigned span = chunk + m - 1;
    const unsigned per_wave = chunk / nw;

    for (unsigned e = threadIdx.x; e < nw * tab; e += blockDim.x) acc[e] = (T)0;
    T* mine = acc + (size_t)wave * tab + lane;

    // workgroup y walks chunks y, y+gridDim.y, ... in ascending order: fixed summation order
    for (unsigned c = blockIdx.y; c < nchunk_total; c += gridDim.y) {
        const size_t i0 = (size_t)c * chunk;
        __syncthreads();
        for (unsigned t = threadIdx.x; t < span; t += blockDim.x) {
            size_t g = i0 + t;
            xl[t] = (g < n + m - 1) ? (uint8_t)letter_of(X[g]) : (uint8_t)5;
        }
        __syncthreads();
        const unsigned pbeg = wave * per_wave;
        for (unsigned p = pbeg; p < pbeg + per_wave; ++p) {
            const size_t i = i0 + p;
            if (i >= n) break;
            const T dz = (f < F) ? dZ[i * F + f] : (T)0;
            const T dq = dz * (T)0.25;
            for (unsigned j = 0; j < m; ++j) {
                const unsigned l = xl[p + j];
                T* cell = mine + (size_t)j * 4 * FT;
                if (l < 4u) {
                    cell[l * FT] += dz;
                } else if (l == 4u) {
                    cell[0 * FT] += dq;
                    cell[1 * FT] += dq;
                    cell[2 * FT] += dq;
                    cell[3 * FT] += dq;
                }
            }
        }
    }
    __syncthreads();
    // combine the waves' tables in wave order and store this workgroup's partial (4m, F) slab
    T* out = partial + (size_t)blockIdx.y * (4 * m) * F;
    for (unsigned e = threadIdx.x; e < tab; e += blockDim.x) {
        T s = acc[e];
        for (unsigned w = 1; w < nw; ++w) s += acc[(size_t)w * tab + e];
        unsigned row = e / FT, fl = e % FT;
        if (f0 + fl < F) out[(size_t)row * F + f0 + fl] = s;
    }
}

// pass 2: dW[e] += partial[0][e] + partial[1][e] + ... as a balanced tree in a fixed shape
template <typename T>
__global__ void reduce_partials_kernel(T* __restrict__ dW, const T* __restrict__ partial, size_t nelem, unsigned nslab)
{
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < nelem; e += (size_t)gridDim.x * blockDim.x) {
        // pairwise tree over slabs: width halves each round, shape depends on nslab only
        T buf[8];
        T total = (T)0;
        for (unsigned base = 0; base < nslab; base += 8) {
            unsigned cnt = nslab - base < 8 ? nslab - base : 8;
            for (unsigned s = 0; s < 8; ++s) buf[s] = s < cnt ? partial[(size_t)(base + s) * nelem + e] : (T)0;
            T t = ((buf[0] + buf[1]) + (buf[2] + buf[3])) + ((buf[4] + buf[5]) + (buf[6] + buf[7]));
            total += t;
        }
        dW[e] += total;
    }
}

// ---------------------------------------------------------------------------------------------
// input gradient: dX[i, c] += sum_f sum_k dZ[i-k, f] * W[(4k+c), f]
// ---------------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

template <typename T>
__global__ __launch_bounds__(256) void corr1ord_bprop_X_kernel(T* __restrict__ dX, size_t n, const T* __restrict__ W,
                                                               unsigned m, unsigned F, const T* __restrict__ dZ)
{
    const unsigned lane = threadIdx.x & 63;
    const size_t wave_global = (size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const size_t nwaves = (size_t)gridDim.x * (blockDim.x >> 6);
    for (size_t i = wave_global; i < n; i += nwaves) {
        T s0 = 0, s1 = 0, s2 = 0, s3 = 0;
        const unsigned kmax = i + 1 < (size_t)m ? (unsigned)(i + 1) : m;
        for (unsigned f = lane; f < F; f += 64) {
            for (unsigned k = 0; k < kmax; ++k) {
                const T dz = dZ[(i - k) * F + f];
                const T* w = W + (size_t)(4 * k) * F + f;
                s0 += dz * w[0];
                s1 += dz * w[(size_t)F];
                s2 += dz * w[(size_t)2 * F];
                s3 += dz * w[(size_t)3 * F];
            }
        }
        s0 = wave_sum(s0);
        s1 = wave_sum(s1);
        s2 = wave_sum(s2);
        s3 = wave_sum(s3);
        if (lane == 0) {
            dX[i * 4 + 0] += s0;
            dX[i * 4 + 1] += s1;
            dX[i * 4 + 2] += s2;
            dX[i * 4 + 3] += s3;
        }
    }
}

template <typename T>
int launch_fprop(hipStream_t st, const T* W, size_t m, size_t F, const uint8_t* X, size_t n, T* Z)
{
    constexpr int NW = 4, PW = 64;
    size_t smem = m * NL * FT * sizeof(T) + (NW * PW + m - 1);
    DBK_CHECK(smem <= lds_limit(), "ValueError: filter length %zu needs %zu bytes of LDS (limit %zu)", m, smem, lds_limit());
    auto kern = corr1ord_kernel<T, NW, PW>;
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    dim3 grid(dbk::divup(n, NW * PW), dbk::divup(F, FT));
    DBK_CHECK(grid.y <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
    hipLaunchKernelGGL(kern, grid, dim3(NW * 64), smem, st, W, (unsigned)m, (unsigned)F, X, n, Z);
    DBK_LAUNCH_OK();
}

template <typename T>
int launch_bprop_W(hipStream_t st, T* dW, size_t m, size_t F, const uint8_t* X, size_t n, const T* dZ)
{
    const unsigned chunk = 512;
    size_t per_wave = m * 4 * FT * sizeof(T);
    unsigned nw = 4;
    while (nw > 1 && nw * per_wave + chunk + m - 1 > lds_limit()) nw >>= 1;
    size_t smem = nw * per_wave + chunk + m - 1;
    DBK_CHECK(smem <= lds_limit(), "ValueError: filter length %zu needs %zu bytes of LDS (limit %zu)", m, smem, lds_limit());
    unsigned ftiles = dbk::divup(F, FT);
    unsigned nchunk = dbk::divup(n, chunk);
    unsigned gy = 2048u / ftiles;
    if (gy < 1) gy = 1;
    if (gy > nchunk) gy = nchunk;
    size_t nelem = 4 * m * F;
    T* partial = (T*)dbk::workspace(nelem * gy * sizeof(T), st);
    DBK_CHECK(partial != nullptr, "MemoryError: could not allocate %zu bytes of scratch", nelem * gy * sizeof(T));
    auto kern = corr1ord_bprop_W_partial_kernel<T>;
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(ftiles, gy), dim3(nw * 64), smem, st, partial, (unsigned)m, (unsigned)F, X, n, dZ, chunk, nchunk);
    hipLaunchKernelGGL(reduce_partials_kernel<T>, dim3(dbk::ew_grid(nelem)), dim3(256), 0, st, dW, (const T*)partial, nelem, gy);
    DBK_LAUNCH_OK();
}

template <typename T>
int launch_bprop_X(hipStream_t st, T* dX, size_t n, const T* W, size_t m, size_t F, const T* dZ)
{
    unsigned blocks = dbk::divup(n, 4);
    if (blocks > 256u * 32u) blocks = 256u * 32u;
    hipLaunchKernelGGL(corr1ord_bprop_X_kernel<T>, dim3(blocks), dim3(256), 0, st, dX, n, W, (unsigned)m, (unsigned)F, dZ);
    DBK_LAUNCH_OK();
}

}  // namespace

extern "C" {

int dbk_corr1ord(dbk_stream_t stream, int dtype, const void* W, size_t m, size_t nfilter,
                 const uint8_t* X, size_t n, size_t nchannel, void* Z)
{
    DBK_DTYPE_OK(dtype);
    DBK_CHECK(nchannel == 4, "NotImplementedError: The given number of channels (%zu) does not have a matching pre-compiled kernel.", nchannel);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    if (n == 0 || nfilter == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && X && Z, "ValueError: null pointer argument");
    if (dtype == DBK_F32) return launch_fprop<float>(dbk::as_stream(stream), (const float*)W, m, nfilter, X, n, (float*)Z);
    return launch_fprop<double>(dbk::as_stream(stream), (const double*)W, m, nfilter, X, n, (double*)Z);
}

int dbk_corr1ord_bprop_W(dbk_stream_t stream, int dtype, void* dW, size_t m, size_t nfilter,
                         const uint8_t* X, size_t n, size_t nchannel, const void* dZ)
{
    DBK_DTYPE_OK(dtype);
    DBK_CHECK(nchannel == 4, "NotImplementedError: The given number of channels (%zu) does not have a matching pre-compiled kernel.", nchannel);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    if (n == 0 || nfilter == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(dW && X && dZ, "ValueError: null pointer argument");
    if (dtype == DBK_F32) return launch_bprop_W<float>(dbk::as_stream(stream), (float*)dW, m, nfilter, X, n, (const float*)dZ);
    return launch_bprop_W<double>(dbk::as_stream(stream), (double*)dW, m, nfilter, X, n, (const double*)dZ);
}

int dbk_corr1ord_bprop_X(dbk_stream_t stream, int dtype, void* dX, size_t n, size_t nchannel,
                         const void* W, size_t m, size_t nfilter, const void* dZ)
{
    DBK_DTYPE_OK(dtype);
    DBK_CHECK(nchannel == 4, "NotImplementedError: The given number of channels (%zu) does not have a matching pre-compiled kernel.", nchannel);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    if (n == 0 || nfilter == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(dX && W && dZ, "ValueError: null pointer argument");
    if (dtype == DBK_F32) return launch_bprop_X<float>(dbk::as_stream(stream), (float*)dX, n, (const float*)W, m, nfilter, (const float*)dZ);
    return launch_bprop_X<double>(dbk::as_stream(stream), (double*)dX, n, (const double*)W, m, nfilter, (const double*)dZ);
}

}  // extern "C"

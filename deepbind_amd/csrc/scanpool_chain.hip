// The scan + bias + rectifier + pooling chain run operator by operator, with the (N x F) map held in the
// stream's scratch: the path for what the fused kernels do not take (sum pooling, regions with a row step).
// Every step is one of the library's own operator kernels, so the results are those of the reference's chain
// corr1ord -> bias -> relu -> poolrgn (kangaroo/_ext/corr1ord.py:97-138, deepity/std/elemwise.py:71-82,162-180,
// kangaroo/_ext/poolrgn.py:56-82) value for value.
#include "dbk_common.h"

namespace {

// Z[i, f] = max(0, Z[i, f] + b[f]) for rows the scan wrote (i < n), max(0, b[f]) for the rest: the scan leaves rows
// whose window passes the end of the sequence untouched, the bias and the rectifier apply to every row.
template <typename T>
__global__ __launch_bounds__(256) void k_bias_relu_rows(T* Z, const T* __restrict__ b, size_t n, size_t N, size_t F)
{
    const size_t total = N * F;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const size_t i = e / F, f = e - i * F;
        const T z = (i < n ? Z[e] : (T)0) + b[f];
        Z[e] = z > (T)0 ? z : (T)0;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void k_fill_zero(T* p, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = (T)0;
}

template <typename T>
int fill_zero(hipStream_t st, T* p, size_t n)
{
    hipLaunchKernelGGL(k_fill_zero<T>, dim3(dbk::ew_grid(n)), dim3(256), 0, st, p, n);
    DBK_LAUNCH_OK();
}

template <typename T> constexpr int dtype_of() { return sizeof(T) == 4 ? DBK_F32 : DBK_F64; }

// relu(scan(W, X) + bias) for all N rows into `map`.
template <typename T>
int rectified_map(dbk_stream_t stream, const T* W, const T* bias, size_t m, size_t F, const uint8_t* X, size_t N, T* map)
{
    const size_t n = N >= m ? N - m + 1 : 0;
    if (n > 0 && dbk_corr1ord(stream, dtype_of<T>(), W, m, F, X, n, 4, map) != 0) return 1;
    hipLaunchKernelGGL(k_bias_relu_rows<T>, dim3(dbk::ew_grid(N * F)), dim3(256), 0, dbk::as_stream(stream), map, bias, n, N, F);
    DBK_LAUNCH_OK();
    return 0;
}

template <typename T>
T* map_scratch(size_t N, size_t F, dbk_stream_t stream, int which)
{
    return (T*)dbk::workspace(N * F * sizeof(T), dbk::as_stream(stream), which);
}

template <typename T>
int chain_fprop(dbk_stream_t stream, const T* W, const T* bias, size_t m, size_t nfilter,
                const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                T* pooled, uint32_t* argmax)
{
    DBK_CHECK(ptype >= DBK_PT_MAX && ptype <= DBK_PT_ALL, "ValueError: unknown pooling type %d", ptype);
    DBK_CHECK(region_columns == 2 || region_columns == 3, "ValueError: regions have 2 columns, or 3 with a row step (got %d)", region_columns);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    DBK_CHECK(!(argmax && (ptype == DBK_PT_AVG || ptype == DBK_PT_SUM)), "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    DBK_CHECK(!argmax || (double)N * (double)nfilter <= 4294967296.0,
              "ValueError: %zu rows x %zu filters overflow the 32-bit argmax index; score in smaller batches or without argmax", N, nfilter);
    if (nfilter == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && regions && pooled, "ValueError: null pointer argument");
    DBK_CHECK(N > 0, "ValueError: regions over an empty sequence");
    T* map = map_scratch<T>(N, nfilter, stream, 2);
    DBK_CHECK(map, "MemoryError: no scratch for the %zu x %zu map: %s", N, nfilter, dbk::workspace_error());
    if (rectified_map<T>(stream, W, bias, m, nfilter, X, N, map) != 0) return 1;
    return dbk_poolrgn(stream, dtype_of<T>(), map, nfilter, regions, nregion, region_columns == 3, pooled, argmax, ptype);
}

template <typename T>
int chain_bprop(dbk_stream_t stream, const T* W, const T* bias, size_t m, size_t nfilter,
                const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                const uint32_t* argmax, const T* dpooled, T* dW, T* dbias, int overwrite)
{
    DBK_CHECK(ptype >= DBK_PT_MAX && ptype <= DBK_PT_ALL, "ValueError: unknown pooling type %d", ptype);
    DBK_CHECK(region_columns == 2 || region_columns == 3, "ValueError: regions have 2 columns, or 3 with a row step (got %d)", region_columns);
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    const bool peak = ptype == DBK_PT_MAX || ptype == DBK_PT_ALL;
    if (nfilter == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && dW && dbias, "ValueError: null pointer argument");
    hipStream_t st = dbk::as_stream(stream);
    if (overwrite && fill_zero<T>(st, dW, 4 * m * nfilter) != 0) return 2;
    if (nregion == 0 || N == 0) return fill_zero<T>(st, dbias, nfilter);
    DBK_CHECK(!peak || argmax != nullptr, "ValueError: pooledmaps_argmax must be specified for max pooling.");
    DBK_CHECK(X && regions && dpooled, "ValueError: null pointer argument");
    T* map = map_scratch<T>(N, nfilter, stream, 2);
    DBK_CHECK(map, "MemoryError: no scratch for the %zu x %zu map: %s", N, nfilter, dbk::workspace_error());
    T* dmap = map_scratch<T>(N, nfilter, stream, 3);
    DBK_CHECK(dmap, "MemoryError: no scratch for the %zu x %zu map gradient: %s", N, nfilter, dbk::workspace_error());
    const int dt = dtype_of<T>();
    if (rectified_map<T>(stream, W, bias, m, nfilter, X, N, map) != 0) return 1;
    if (fill_zero<T>(st, dmap, N * nfilter) != 0) return 2;
    if (dbk_poolrgn_bprop(stream, dt, dmap, nfilter, regions, nregion, region_columns == 3, dpooled, peak ? argmax : nullptr, ptype) != 0) return 1;
    if (dbk_mul_sign(stream, dt, dmap, map, dmap, N * nfilter) != 0) return 1;
    if (dbk_colsum(stream, dt, dmap, dbias, N, nfilter) != 0) return 1;
    const size_t n = N >= m ? N - m + 1 : 0;
    if (n > 0 && dbk_corr1ord_bprop_W(stream, dt, dW, m, nfilter, X, n, 4, dmap) != 0) return 1;
    dbk::clear_error();
    return 0;
}

}  // namespace

extern "C" {

int dbk_scanpool_fprop_unfused(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                               const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                               float* pooled, uint32_t* argmax)
{
    return chain_fprop<float>(stream, W, bias, m, nfilter, X, N, regions, nregion, region_columns, ptype, pooled, argmax);
}

int dbk_scanpool_bprop_unfused(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                               const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                               const uint32_t* argmax, const float* dpooled, float* dW, float* dbias, int overwrite)
{
    return chain_bprop<float>(stream, W, bias, m, nfilter, X, N, regions, nregion, region_columns, ptype, argmax, dpooled, dW, dbias, overwrite);
}

int dbk_scanpool_fprop_f64(dbk_stream_t stream, const double* W, const double* bias, size_t m, size_t nfilter,
                           const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                           double* pooled, uint32_t* argmax)
{
    return chain_fprop<double>(stream, W, bias, m, nfilter, X, N, regions, nregion, region_columns, ptype, pooled, argmax);
}

int dbk_scanpool_bprop_f64(dbk_stream_t stream, const double* W, const double* bias, size_t m, size_t nfilter,
                           const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                           const uint32_t* argmax, const double* dpooled, double* dW, double* dbias, int overwrite)
{
    return chain_bprop<double>(stream, W, bias, m, nfilter, X, N, regions, nregion, region_columns, ptype, argmax, dpooled, dW, dbias, overwrite);
}

}  // extern "C"

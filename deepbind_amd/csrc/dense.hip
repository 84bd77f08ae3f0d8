// Per-model ("blockwise") small dense products on the model axis, and the fused scoring head.
//
// The products are tiny (k, m <= a few dozen) and there are many of them (one per model), so they
// are not GEMM-shaped work for the matrix cores: one thread owns one output element, the 64 lanes
// of a wave own 64 consecutive output columns of one row, and the inner product runs in a fixed
// order in registers. HBM traffic is one coalesced pass over the operands.
//
// Reference semantics: deepity_smat/blockwise_dot.cu:77-260 (pointer arithmetic per block) and
// deepity/_ext/deepity_smat.py:169-251 (shapes).
#include "dbk_common.h"

namespace {

// Z[r, b*m + c] (beta ? += : =) sum_kk X[r, xb + kk] * W[(b*p + off + kk)*m + c],  xb = bcast ? 0 : b*k
template <typename T>
__global__ __launch_bounds__(256) void k_bdot(int nblock, size_t n, int m, int k, int p, int off, bool bcast, bool accumulate,
                                              const T* __restrict__ X, const T* __restrict__ W, T* __restrict__ Z)
{
    const size_t ldx = (size_t)k * (bcast ? 1 : nblock), ldz = (size_t)m * nblock;
    const size_t total = n * ldz;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const size_t r = e / ldz;
        const unsigned col = (unsigned)(e % ldz);
        const unsigned b = col / m, c = col % m;
        const T* x = X + r * ldx + (bcast ? 0 : (size_t)b * k);
        const T* w = W + ((size_t)b * p + off) * m + c;
        T s = (T)0;
        for (int kk = 0; kk < k; ++kk) s += x[kk] * w[(size_t)kk * m];
        Z[e] = accumulate ? Z[e] + s : s;
    }
}

// dX[r, b*k + kk] = sum_c dZ[r, b*m + c] * W[(b*p + off + kk)*m + c]
template <typename T>
__global__ __launch_bounds__(256) void k_bdot_nt(int nblock, size_t n, int m, int k, int p, int off,
                                                 const T* __restrict__ dZ, const T* __restrict__ W, T* __restrict__ dX)
{
    const size_t ldx = (size_t)k * nblock, ldz = (size_t)m * nblock;
    const size_t total = n * ldx;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const size_t r = e / ldx;
        const unsigned col = (unsigned)(e % ldx);
        const unsigned b = col / k, kk = col % k;
        const T* dz = dZ + r * ldz + (size_t)b * m;
        const T* w = W + ((size_t)b * p + off + kk) * m;
        T s = (T)0;
        for (int c = 0; c < m; ++c) s += dz[c] * w[c];
        dX[e] = s;
    }
}

// dW[(b*p + off + kk)*m + c] = sum_r X[r, xb + kk] * dZ[r, b*m + c]; rows in ascending order.
// One wave per output element group: lanes split the rows, then a fixed-shape butterfly sum.
template <typename T>
__global__ __launch_bounds__(256) void k_bdot_tn(int nblock, size_t n, int m, int k, int p, int off, bool bcast,
                                                 const T* __restrict__ X, const T* __restrict__ dZ, T* __restrict__ dW)
{
    const size_t ldx = (size_t)k * (bcast ? 1 : nblock), ldz = (size_t)m * nblock;
    const size_t total = (size_t)nblock * k * m;
    const unsigned lane = threadIdx.x & 63;
    const size_t wave = (size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const size_t nwave = (size_t)gridDim.x * (blockDim.x >> 6);
    for (size_t e = wave; e < total; e += nwave) {
        const unsigned c = (unsigned)(e % m);
        const unsigned kk = (unsigned)((e / m) % k);
        const unsigned b = (unsigned)(e / ((size_t)m * k));
        const T* x = X + (bcast ? 0 : (size_t)b * k) + kk;
        const T* dz = dZ + (size_t)b * m + c;
        T s = (T)0;
        for (size_t r = lane; r < n; r += 64) s += x[r * ldx] * dz[r * ldz];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) s += __shfl_down(s, o, 64);
        if (lane == 0) dW[((size_t)b * p + off + kk) * m + c] = s;
    }
}

// Scoring head: a workgroup owns one model and a tile of 256 rows. The model's weights (a few KB)
// are staged in LDS once and read back as wave-wide broadcasts; each thread keeps its row's k inputs
// in registers (one contiguous k*4-byte read of HBM per thread) and writes one score.
constexpr int HEAD_MAXK = 64;
template <int KMAX>
__global__ __launch_bounds__(256) void k_head(size_t n, int nblock, int k, int hidden, const float* __restrict__ pooled,
                                              const float* __restrict__ in_scale, const float* __restrict__ W1,
                                              const float* __restrict__ b1, const float* __restrict__ W2,
                                              const float* __restrict__ b2, bool apply_logistic, float* __restrict__ scores)
{
    extern __shared__ float hsm[];
    const unsigned b = blockIdx.y;
    const int h1 = hidden > 0 ? hidden : 1;
    float* w1s = hsm;                       // [k][h1]
    float* b1s = w1s + (size_t)k * h1;      // [h1]
    float* w2s = b1s + h1;                  // [hidden]
    for (int e = threadIdx.x; e < k * h1; e += blockDim.x) w1s[e] = W1[(size_t)b * k * h1 + e];
    for (int e = threadIdx.x; e < h1; e += blockDim.x) b1s[e] = b1[(size_t)b * h1 + e];
    for (int e = threadIdx.x; e < hidden; e += blockDim.x) w2s[e] = W2[(size_t)b * hidden + e];
    __syncthreads();
    const float sc = in_scale ? in_scale[b] : 1.0f;
    const float bias2 = hidden > 0 ? b2[b] : 0.0f;
    for (size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x; r < n; r += (size_t)gridDim.x * blockDim.x) {
        const float* x = pooled + r * (size_t)k * nblock + (size_t)b * k;
        float xr[KMAX];
#pragma unroll
        for (int kk = 0; kk < KMAX; ++kk) xr[kk] = kk < k ? x[kk] * sc : 0.0f;
        float out;
        if (hidden > 0) {
            out = 0.0f;
            for (int h = 0; h < hidden; ++h) {
                float a = 0.0f;
#pragma unroll
                for (int kk = 0; kk < KMAX; ++kk)
                    if (kk < k) a += xr[kk] * w1s[kk * hidden + h];
                a += b1s[h];
                a = a > 0.0f ? a : 0.0f;
                out += a * w2s[h];
            }
            out += bias2;
        } else {
            out = 0.0f;
#pragma unroll
            for (int kk = 0; kk < KMAX; ++kk)
                if (kk < k) out += xr[kk] * w1s[kk];
            out += b1s[0];
        }
        if (apply_logistic) out = 1.0f / (1.0f + expf(-out));
        scores[r * (size_t)nblock + b] = out;
    }
}

int check_dims(int nblock, int n, int m, int k, int p, int off)
{
    DBK_CHECK(nblock >= 1, "ValueError: nblock must be >= 1, got %d", nblock);
    DBK_CHECK(n >= 0 && m >= 0 && k >= 0, "ValueError: negative matrix dimension");
    DBK_CHECK(off >= 0 && off + k <= p, "ValueError: input rows [%d, %d) do not fit in a block of %d weight rows", off, off + k, p);
    return 0;
}

}  // namespace

extern "C" {

int dbk_blockwise_dot_combined(dbk_stream_t stream, int dtype, int nblock, int Xoffset, int Xbroadcast,
                               int n, int m, int k, int p, const void* X, const void* W, void* Z)
{
    DBK_DTYPE_OK(dtype);
    if (check_dims(nblock, n, m, k, p, Xoffset)) return 1;
    if (n == 0 || m == 0 || k == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(X && W && Z, "ValueError: null pointer argument");
    size_t total = (size_t)n * m * nblock;
    if (dtype == DBK_F32)
        hipLaunchKernelGGL(k_bdot<float>, dim3(dbk::ew_grid(total)), dim3(256), 0, dbk::as_stream(stream), nblock, (size_t)n, m, k, p,
                           Xoffset, Xbroadcast != 0, Xoffset != 0, (const float*)X, (const float*)W, (float*)Z);
    else
        hipLaunchKernelGGL(k_bdot<double>, dim3(dbk::ew_grid(total)), dim3(256), 0, dbk::as_stream(stream), nblock, (size_t)n, m, k, p,
                           Xoffset, Xbroadcast != 0, Xoffset != 0, (const double*)X, (const double*)W, (double*)Z);
    DBK_LAUNCH_OK();
}

int dbk_blockwise_dot(dbk_stream_t stream, int dtype, int nblock, int n, int m, int k, int broadcast_x,
                      const void* X, const void* W, void* Z)
{
    return dbk_blockwise_dot_combined(stream, dtype, nblock, 0, broadcast_x, n, m, k, k, X, W, Z);
}

int dbk_blockwise_dot_nt_combined(dbk_stream_t stream, int dtype, int nblock, int Xoffset,
                                  int n, int m, int k, int p, void* dX, const void* W, const void* dZ)
{
    DBK_DTYPE_OK(dtype);
    if (check_dims(nblock, n, m, k, p, Xoffset)) return 1;
    if (n == 0 || m == 0 || k == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(dX && W && dZ, "ValueError: null pointer argument");
    size_t total = (size_t)n * k * nblock;
    if (dtype == DBK_F32)
        hipLaunchKernelGGL(k_bdot_nt<float>, dim3(dbk::ew_grid(total)), dim3(256), 0, dbk::as_stream(stream), nblock, (size_t)n, m, k, p,
                           Xoffset, (const float*)dZ, (const float*)W, (float*)dX);
    else
        hipLaunchKernelGGL(k_bdot_nt<double>, dim3(dbk::ew_grid(total)), dim3(256), 0, dbk::as_stream(stream), nblock, (size_t)n, m, k, p,
                           Xoffset, (const double*)dZ, (const double*)W, (double*)dX);
    DBK_LAUNCH_OK();
}

int dbk_blockwise_dot_nt(dbk_stream_t stream, int dtype, int nblock, int n, int m, int k,
                         const void* dZ, const void* W, void* dX)
{
    return dbk_blockwise_dot_nt_combined(stream, dtype, nblock, 0, n, m, k, k, dX, W, dZ);
}

int dbk_blockwise_dot_tn_combined(dbk_stream_t stream, int dtype, int nblock, int Xoffset, int Xbroadcast,
                                  int n, int m, int k, int p, const void* X, void* dW, const void* dZ)
{
    DBK_DTYPE_OK(dtype);
    if (check_dims(nblock, n, m, k, p, Xoffset)) return 1;
    if (n == 0 || m == 0 || k == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(X && dW && dZ, "ValueError: null pointer argument");
    size_t total = (size_t)nblock * k * m;                 // one wave per element
    unsigned grid = dbk::divup(total, 4);
    if (grid > 256u * 16u) grid = 256u * 16u;
    if (dtype == DBK_F32)
        hipLaunchKernelGGL(k_bdot_tn<float>, dim3(grid), dim3(256), 0, dbk::as_stream(stream), nblock, (size_t)n, m, k, p,
                           Xoffset, Xbroadcast != 0, (const float*)X, (const float*)dZ, (float*)dW);
    else
        hipLaunchKernelGGL(k_bdot_tn<double>, dim3(grid), dim3(256), 0, dbk::as_stream(stream), nblock, (size_t)n, m, k, p,
                           Xoffset, Xbroadcast != 0, (const double*)X, (const double*)dZ, (double*)dW);
    DBK_LAUNCH_OK();
}

int dbk_blockwise_dot_tn(dbk_stream_t stream, int dtype, int nblock, int n, int m, int k, int broadcast_x,
                         const void* X, const void* dZ, void* dW)
{
    return dbk_blockwise_dot_tn_combined(stream, dtype, nblock, 0, broadcast_x, n, m, k, k, X, dW, dZ);
}

int dbk_head_fprop(dbk_stream_t stream, size_t n, int nblock, int k, int hidden,
                   const float* pooled, const float* in_scale,
                   const float* W1, const float* b1, const float* W2, const float* b2,
                   int apply_logistic, float* scores)
{
    DBK_CHECK(nblock >= 1 && k >= 1 && hidden >= 0, "ValueError: bad head shape (nblock=%d, k=%d, hidden=%d)", nblock, k, hidden);
    if (n == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(pooled && W1 && b1 && scores, "ValueError: null pointer argument");
    DBK_CHECK(hidden == 0 || (W2 && b2), "ValueError: hidden layer requested but W2/b2 are null");
    DBK_CHECK(k <= HEAD_MAXK, "ValueError: the fused head takes at most %d inputs per model (got %d)", HEAD_MAXK, k);
    DBK_CHECK(nblock <= 65535, "ValueError: too many models (%d) for one launch", nblock);
    const int h1 = hidden > 0 ? hidden : 1;
    size_t smem = ((size_t)k * h1 + h1 + hidden) * sizeof(float);
    DBK_CHECK(smem <= 65536, "ValueError: head weights (%zu bytes per model) do not fit in LDS", smem);
    unsigned gx = dbk::divup(n, 256);
    if (gx > 2048u) gx = 2048u;
    auto kern = k <= 16 ? k_head<16> : (k <= 32 ? k_head<32> : k_head<64>);
    hipLaunchKernelGGL(kern, dim3(gx, nblock), dim3(256), smem, dbk::as_stream(stream), n, nblock, k, hidden, pooled, in_scale,
                       W1, b1, W2, b2, apply_logistic != 0, scores);
    DBK_LAUNCH_OK();
}

}  // extern "C"

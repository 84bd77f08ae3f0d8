// Per-model ("blockwise") small dense products on the model axis, and the fused scoring head.
//
// The products are tiny (k, m <= a few dozen) and there are many of them (one per model). The vector kernels: one
// thread owns one output element (or four), the lanes of a wave own consecutive output columns of one row, the
// inner product runs in a fixed order in registers. At bulk row counts, float32 products whose widths are multiples
// of 16 run on the matrix cores instead (k_bdot_mfma): the vector kernels spend their time on LDS reads of the
// weights (one per multiply-add), the matrix-core kernel moves at the rate of its one pass over the operands.
//
// Reference semantics: deepity_smat/blockwise_dot.cu:77-260 (pointer arithmetic per block) and
// deepity/_ext/deepity_smat.py:169-251 (shapes).
#include "dbk_common.h"
#include "mfma_common.h"

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

// ---------------------------------------------------------------------------------------------
// Bulk variants (many rows). A workgroup takes TG = 16 consecutive models; lane = (row, model) with the
// model fastest, so a wave reads and writes contiguous row segments spanning 16 models, and the 16
// models' weights sit in LDS as [input][output/4][model][4]: one aligned 256-byte line per 16 lanes and
// ds_read_b128. Multiply-adds are fused (as in the reference's GEMM library); inputs ascending.
// ---------------------------------------------------------------------------------------------
constexpr int TG = 16;

template <typename T> struct alignas(4 * sizeof(T)) vec4 { T x, y, z, w; };

__device__ __forceinline__ float fma_t(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_t(double a, double b, double c) { return __builtin_fma(a, b, c); }

template <typename T>
__device__ void stage_weights16(T* ws, const T* __restrict__ W, int nblock, unsigned m0, int k, int m, int p, int off)
{
    const int mq = m >> 2;
    for (int e = threadIdx.x; e < k * m * TG; e += blockDim.x) {
        // destination order: e = ((kk*mq + c4)*TG + g)*4 + c
        const int c = e & 3, g = (e >> 2) & (TG - 1), rest = e >> 6, c4 = rest % mq, kk = rest / mq;
        const unsigned mdl = m0 + g;
        ws[e] = mdl < (unsigned)nblock ? W[((size_t)mdl * p + off + kk) * m + c4 * 4 + c] : (T)0;
    }
}

// Z[r, b*m + c] (accumulate ? += : =) sum_kk X[r, xb + kk] * W[(b*p + off + kk)*m + c]
template <typename T, int KMAX, int MMAX>
__global__ __launch_bounds__(256) void k_bdot_tile(int nblock, size_t n, int m, int k, int p, int off, bool bcast, bool accumulate,
                                                   const T* __restrict__ X, const T* __restrict__ W, T* __restrict__ Z)
{
    extern __shared__ __align__(16) unsigned char tsm[];
    T* ws = reinterpret_cast<T*>(tsm);
    const unsigned g = threadIdx.x & (TG - 1), rl = threadIdx.x >> 4, m0 = blockIdx.x * TG, mdl = m0 + g;
    stage_weights16(ws, W, nblock, m0, k, m, p, off);
    __syncthreads();
    if (mdl >= (unsigned)nblock) return;
    const int mq = m >> 2;
    const size_t ldx = (size_t)k * (bcast ? 1 : nblock), ldz = (size_t)m * nblock;
    const vec4<T>* wv = reinterpret_cast<const vec4<T>*>(ws) + g;
    const size_t rstep = (size_t)gridDim.y * 16, xoff = bcast ? 0 : (size_t)mdl * k;
    size_t r = (size_t)blockIdx.y * 16 + rl;
    T xn[KMAX];                                          // next row's inputs, fetched while this row is computed
#pragma unroll
    for (int kk = 0; kk < KMAX; ++kk) xn[kk] = (kk < k && r < n) ? X[r * ldx + xoff + kk] : (T)0;
    for (; r < n; r += rstep) {
        T xr[KMAX];
#pragma unroll
        for (int kk = 0; kk < KMAX; ++kk) xr[kk] = xn[kk];
        const size_t rn = r + rstep;
#pragma unroll
        for (int kk = 0; kk < KMAX; ++kk) xn[kk] = (kk < k && rn < n) ? X[rn * ldx + xoff + kk] : (T)0;
        T* z = Z + r * ldz + (size_t)mdl * m;
#pragma unroll
        for (int c4 = 0; c4 < MMAX / 4; ++c4) {
            if (c4 < mq) {
                T a0 = 0, a1 = 0, a2 = 0, a3 = 0;
#pragma unroll
                for (int kk = 0; kk < KMAX; ++kk)
                    if (kk < k) {
                        const vec4<T> w = wv[(kk * mq + c4) * TG];
                        a0 = fma_t(xr[kk], w.x, a0);
                        a1 = fma_t(xr[kk], w.y, a1);
                        a2 = fma_t(xr[kk], w.z, a2);
                        a3 = fma_t(xr[kk], w.w, a3);
                    }
                vec4<T>* zo = reinterpret_cast<vec4<T>*>(z) + c4;
                if (accumulate) { const vec4<T> o = *zo; a0 += o.x; a1 += o.y; a2 += o.z; a3 += o.w; }
                *zo = vec4<T>{a0, a1, a2, a3};
            }
        }
    }
}

// dX[r, b*k + kk] = sum_c dZ[r, b*m + c] * W[(b*p + off + kk)*m + c]
template <typename T, int KMAX, int MMAX>
__global__ __launch_bounds__(256) void k_bdot_nt_tile(int nblock, size_t n, int m, int k, int p, int off,
                                                      const T* __restrict__ dZ, const T* __restrict__ W, T* __restrict__ dX)
{
    extern __shared__ __align__(16) unsigned char tsm[];
    T* ws = reinterpret_cast<T*>(tsm);
    const unsigned g = threadIdx.x & (TG - 1), rl = threadIdx.x >> 4, m0 = blockIdx.x * TG, mdl = m0 + g;
    stage_weights16(ws, W, nblock, m0, k, m, p, off);
    __syncthreads();
    if (mdl >= (unsigned)nblock) return;
    const int mq = m >> 2;
    const size_t ldx = (size_t)k * nblock, ldz = (size_t)m * nblock;
    const vec4<T>* wv = reinterpret_cast<const vec4<T>*>(ws) + g;
    const size_t rstep = (size_t)gridDim.y * 16;
    size_t r = (size_t)blockIdx.y * 16 + rl;
    vec4<T> dn[MMAX / 4];                                // next row's gradient, fetched while this row is computed
#pragma unroll
    for (int c4 = 0; c4 < MMAX / 4; ++c4)
        dn[c4] = (c4 < mq && r < n) ? reinterpret_cast<const vec4<T>*>(dZ + r * ldz + (size_t)mdl * m)[c4] : vec4<T>{0, 0, 0, 0};
    for (; r < n; r += rstep) {
        vec4<T> d[MMAX / 4];
#pragma unroll
        for (int c4 = 0; c4 < MMAX / 4; ++c4) d[c4] = dn[c4];
        const size_t rn = r + rstep;
#pragma unroll
        for (int c4 = 0; c4 < MMAX / 4; ++c4)
            dn[c4] = (c4 < mq && rn < n) ? reinterpret_cast<const vec4<T>*>(dZ + rn * ldz + (size_t)mdl * m)[c4] : vec4<T>{0, 0, 0, 0};
        T* dx = dX + r * ldx + (size_t)mdl * k;
#pragma unroll
        for (int kk = 0; kk < KMAX; ++kk) {
            if (kk < k) {
                T s0 = 0, s1 = 0, s2 = 0, s3 = 0;
#pragma unroll
                for (int c4 = 0; c4 < MMAX / 4; ++c4)
                    if (c4 < mq) {
                        const vec4<T> w = wv[(kk * mq + c4) * TG];
                        s0 = fma_t(d[c4].x, w.x, s0);
                        s1 = fma_t(d[c4].y, w.y, s1);
                        s2 = fma_t(d[c4].z, w.z, s2);
                        s3 = fma_t(d[c4].w, w.w, s3);
                    }
                dx[kk] = (s0 + s1) + (s2 + s3);
            }
        }
    }
}

// Row-tile kernel shared by dot and dot_nt when the output width per model `no` is 4, 8, 16, 32 or 64:
// out[r, b*no + o] (+)= sum_i in[r, inbase(b) + i] * w_b[i][o]. no/4 adjacent lanes share one (row, model)
// and own four outputs each, so a wave stores whole contiguous row segments (16 bytes per lane, lanes
// adjacent) and the 16 lanes of a quarter-wave read one aligned 256-byte line of the weights, which sit
// in LDS as [input][model][output]. `transpose` stages w_b[i][o] = W_b[o][i] (the dot_nt case).
template <typename T, int IMAX>
__global__ __launch_bounds__(256) void k_bdot_rowtile(int nblock, size_t n, int ni, int no, bool bcast, bool accumulate, bool transpose,
                                                      int m, int p, int off,
                                                      const T* __restrict__ in, const T* __restrict__ W, T* __restrict__ out)
{
    extern __shared__ __align__(16) unsigned char tsm[];
    T* ws = reinterpret_cast<T*>(tsm);                                     // [ni][TG][no]
    const unsigned m0 = blockIdx.x * TG;
    for (int e = threadIdx.x; e < ni * TG * no; e += blockDim.x) {
        const int o = e % no, g = (e / no) % TG, i = e / (no * TG);
        const unsigned mdl = m0 + g;
        // W_b is (k rows = inputs of dot, m columns); dot: (i, o) = (row, col); dot_nt: (i, o) = (col, row)
        const size_t src = transpose ? ((size_t)mdl * p + off + o) * m + i : ((size_t)mdl * p + off + i) * m + o;
        ws[e] = mdl < (unsigned)nblock ? W[src] : (T)0;
    }
    __syncthreads();
    const int lpm = no >> 2;                                               // lanes per (row, model)
    const unsigned j = threadIdx.x % lpm, pm = threadIdx.x / lpm, g = pm % TG, rl = pm / TG;
    const unsigned rpp = 256 / (lpm * TG);                                 // rows per pass
    const unsigned mdl = m0 + g;
    if (mdl >= (unsigned)nblock) return;
    const size_t ldin = (size_t)ni * (bcast ? 1 : nblock), ldout = (size_t)no * nblock;
    const size_t inoff = bcast ? 0 : (size_t)mdl * ni;
    const vec4<T>* wv = reinterpret_cast<const vec4<T>*>(ws + (size_t)g * no) + j;
    const int wstep = TG * no / 4;                                         // vec4 stride between inputs
    for (size_t r = (size_t)blockIdx.y * rpp + rl; r < n; r += (size_t)gridDim.y * rpp) {
        const T* x = in + r * ldin + inoff;
        T xr[IMAX];
#pragma unroll
        for (int i = 0; i < IMAX; ++i) xr[i] = i < ni ? x[i] : (T)0;
        T a0 = 0, a1 = 0, a2 = 0, a3 = 0;
#pragma unroll
        for (int i = 0; i < IMAX; ++i)
            if (i < ni) {
                const vec4<T> w = wv[i * wstep];
                a0 = fma_t(xr[i], w.x, a0);
                a1 = fma_t(xr[i], w.y, a1);
                a2 = fma_t(xr[i], w.z, a2);
                a3 = fma_t(xr[i], w.w, a3);
            }
        vec4<T>* zo = reinterpret_cast<vec4<T>*>(out + r * ldout + (size_t)mdl * no) + j;
        if (accumulate) { const vec4<T> o = *zo; a0 += o.x; a1 += o.y; a2 += o.z; a3 += o.w; }
        *zo = vec4<T>{a0, a1, a2, a3};
    }
}

// dW partial sums: workgroup (b, y) takes model b and row chunk y, stages 64 rows of the model's
// X (64 x k) and dZ (64 x m) columns in LDS at a time, and thread e owns output elements e, e+256, ...
// (rows ascending). k_bdot_tn_fold adds the chunks in ascending order.
constexpr int TN_ROWS = 64, TN_CHUNK = 1024, TN_OWN = 16;
template <typename T>
__global__ __launch_bounds__(256) void k_bdot_tn_tile(int nblock, size_t n, int m, int k, bool bcast,
                                                      const T* __restrict__ X, const T* __restrict__ dZ, T* __restrict__ partial)
{
    extern __shared__ __align__(16) unsigned char tsm[];
    const int ks = k | 1, ms = m | 1;                        // odd strides: no bank conflicts while staging
    T* xs = reinterpret_cast<T*>(tsm);                       // [TN_ROWS][ks]
    T* ds_ = xs + TN_ROWS * ks;                              // [TN_ROWS][ms]
    const unsigned b = blockIdx.x;
    const size_t ldx = (size_t)k * (bcast ? 1 : nblock), ldz = (size_t)m * nblock;
    const size_t r0 = (size_t)blockIdx.y * TN_CHUNK;
    const size_t r1 = r0 + TN_CHUNK < n ? r0 + TN_CHUNK : n;
    const int nout = k * m;
    T acc[TN_OWN];
#pragma unroll
    for (int i = 0; i < TN_OWN; ++i) acc[i] = (T)0;
    for (size_t t0 = r0; t0 < r1; t0 += TN_ROWS) {
        const int rows = (int)(r1 - t0 < (size_t)TN_ROWS ? r1 - t0 : (size_t)TN_ROWS);
        __syncthreads();
        for (int e = threadIdx.x; e < TN_ROWS * k; e += blockDim.x) {
            const int rr = e / k, kk = e % k;
            xs[rr * ks + kk] = rr < rows ? X[(t0 + rr) * ldx + (bcast ? 0 : (size_t)b * k) + kk] : (T)0;
        }
        for (int e = threadIdx.x; e < TN_ROWS * m; e += blockDim.x) {
            const int rr = e / m, c = e % m;
            ds_[rr * ms + c] = rr < rows ? dZ[(t0 + rr) * ldz + (size_t)b * m + c] : (T)0;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < TN_OWN; ++i) {
            const int e = threadIdx.x + i * 256;
            if (e < nout) {
                const int kk = e / m, c = e % m;
                T s = acc[i];
#pragma unroll 8
                for (int rr = 0; rr < TN_ROWS; ++rr) s = fma_t(xs[rr * ks + kk], ds_[rr * ms + c], s);
                acc[i] = s;
            }
        }
    }
    T* out = partial + ((size_t)blockIdx.y * nblock + b) * nout;
#pragma unroll
    for (int i = 0; i < TN_OWN; ++i) {
        const int e = threadIdx.x + i * 256;
        if (e < nout) out[e] = acc[i];
    }
}
// The weight gradient for 16 consecutive models per workgroup (float32, K = 16 or 32 inputs, 32 outputs per model,
// 16-byte aligned operands): a row of X then holds 16*K contiguous floats for the workgroup and a row of dZ 16*32, so
// the rows are read as full 1-4 KB segments (the kernel above reads 64-byte pieces at a 4 KB stride: ~20 % of the HBM
// rate). Eight rows at a time are staged in LDS (the next eight are requested before these are used); a thread owns a
// (K/4 x 8) block of one model's K x 32 gradient in registers and reads its row values as three or four 16-byte words
// (same address within a quarter wave's groups: broadcasts). Rows are added in ascending order within a chunk; the
// chunks are added in ascending order by k_bdot_tn_fold, as above.
constexpr int TN16_ROWS = 8, TN16_G = 16;
template <int K>
__global__ __launch_bounds__(256) void k_bdot_tn16(int nblock, size_t n, const float* __restrict__ X, const float* __restrict__ dZ,
                                                  float* __restrict__ partial)
{
    constexpr int M = 32, TK = K / 4, XW = TN16_G * K, ZW = TN16_G * M;    // floats of X / dZ per row and workgroup
    constexpr int XV = TN16_ROWS * XW / 4 / 256, ZV = TN16_ROWS * ZW / 4 / 256;   // 16-byte words per thread and tile
    __shared__ __align__(16) float xs[2][TN16_ROWS * XW];
    __shared__ __align__(16) float zs[2][TN16_ROWS * ZW];
    const unsigned tid = threadIdx.x, g = tid >> 4, kq = (tid >> 2) & 3, cq = tid & 3;
    const unsigned m0 = blockIdx.x * TN16_G;                            // first model of this workgroup
    const unsigned nlive = m0 + TN16_G <= (unsigned)nblock ? TN16_G : (unsigned)nblock - m0;
    const size_t ldx = (size_t)K * nblock, ldz = (size_t)M * nblock;
    const size_t r0 = (size_t)blockIdx.y * TN_CHUNK, r1 = r0 + TN_CHUNK < n ? r0 + TN_CHUNK : n;
    float acc[TK][8];
#pragma unroll
    for (int i = 0; i < TK; ++i)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[i][c] = 0.0f;
    float4 xv[XV], zv[ZV];
    auto fetch = [&](size_t t0) {
#pragma unroll
        for (int i = 0; i < XV; ++i) {
            const unsigned e = tid + i * 256, rr = e / (XW / 4), w = e % (XW / 4);      // word w of row rr
            const bool in = t0 + rr < r1 && w * 4 < nlive * K;
            xv[i] = in ? *reinterpret_cast<const float4*>(X + (t0 + rr) * ldx + (size_t)m0 * K + w * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < ZV; ++i) {
            const unsigned e = tid + i * 256, rr = e / (ZW / 4), w = e % (ZW / 4);
            const bool in = t0 + rr < r1 && w * 4 < nlive * M;
            zv[i] = in ? *reinterpret_cast<const float4*>(dZ + (t0 + rr) * ldz + (size_t)m0 * M + w * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto park = [&](int buf) {
#pragma unroll
        for (int i = 0; i < XV; ++i) reinterpret_cast<float4*>(xs[buf])[tid + i * 256] = xv[i];
#pragma unroll
        for (int i = 0; i < ZV; ++i) reinterpret_cast<float4*>(zs[buf])[tid + i * 256] = zv[i];
    };
    fetch(r0);
    park(0);
    int buf = 0;
    for (size_t t0 = r0; t0 < r1; t0 += TN16_ROWS, buf ^= 1) {
        __syncthreads();                                            // tile `buf` is complete; the other one is free again
        const bool more = t0 + TN16_ROWS < r1;
        if (more) fetch(t0 + TN16_ROWS);
        const float* xrow = xs[buf] + g * K + kq * TK;
        const float* zrow = zs[buf] + g * M + cq * 8;
#pragma unroll
        for (int rr = 0; rr < TN16_ROWS; ++rr) {
            float x[TK], z[8];
#pragma unroll
            for (int i = 0; i < TK; i += 4) {
                const float4 v = *reinterpret_cast<const float4*>(xrow + rr * XW + i);
                x[i] = v.x; x[i + 1] = v.y; x[i + 2] = v.z; x[i + 3] = v.w;
            }
            const float4 z0 = *reinterpret_cast<const float4*>(zrow + rr * ZW), z1 = *reinterpret_cast<const float4*>(zrow + rr * ZW + 4);
            z[0] = z0.x; z[1] = z0.y; z[2] = z0.z; z[3] = z0.w; z[4] = z1.x; z[5] = z1.y; z[6] = z1.z; z[7] = z1.w;
#pragma unroll
            for (int i = 0; i < TK; ++i)
#pragma unroll
                for (int c = 0; c < 8; ++c) acc[i][c] = __builtin_fmaf(x[i], z[c], acc[i][c]);
        }
        if (more) park(buf ^ 1);
    }
    if (g < nlive) {
        float* out = partial + ((size_t)blockIdx.y * nblock + m0 + g) * (K * M);
#pragma unroll
        for (int i = 0; i < TK; ++i) {
            float* row = out + (kq * TK + i) * M + cq * 8;
            *reinterpret_cast<float4*>(row) = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
            *reinterpret_cast<float4*>(row + 4) = make_float4(acc[i][4], acc[i][5], acc[i][6], acc[i][7]);
        }
    }
}
template <typename T>
__global__ void k_bdot_tn_fold(int nblock, int m, int k, int p, int off, unsigned nchunk, const T* __restrict__ partial, T* __restrict__ dW)
{
    const size_t nout = (size_t)k * m, total = nout * nblock;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const unsigned b = (unsigned)(e / nout), idx = (unsigned)(e % nout), kk = idx / m, c = idx % m;
        T s = partial[e];
#pragma unroll 8
        for (unsigned y = 1; y < nchunk; ++y) s += partial[(size_t)y * total + e];
        dW[((size_t)b * p + off + kk) * m + c] = s;
    }
}

// Scoring head: a workgroup owns one model and a tile of 256 rows. The model's weights (a few KB)
// are staged in LDS once and read back as wave-wide broadcasts; each thread keeps its row's k inputs
// in registers (one contiguous k*4-byte read of HBM per thread) and writes one score.
constexpr int HEAD_MAXK = 64;
template <int KMAX>
__global__ __launch_bounds__(256) void k_head(size_t n, int nblock, int k, int kf, int kw, int hidden, const float* __restrict__ pooled,
                                              const float* __restrict__ feats,
                                              const float* __restrict__ in_scale, const float* __restrict__ W1,
                                              const float* __restrict__ b1, const float* __restrict__ W2,
                                              const float* __restrict__ b2, bool apply_logistic, float* __restrict__ scores)
{
    extern __shared__ __align__(16) float hsm[];
    // models vary fastest over the grid: the workgroups that share a tile of rows run together, so each
    // 4 KB row of the feature matrix is pulled from HBM once and served to its 64 models from L2
    const unsigned b = blockIdx.x;
    // a model's block of W1 has kw rows: k for its own inputs, then the shared feature columns, of which the
    // first kf are read here (kf = 0 when the features are all zeros: their weights then play no part)
    const int h1 = hidden > 0 ? hidden : 1, kt = k + kf;
    float* w1s = hsm;                       // [kt][h1]
    float* b1s = w1s + (size_t)kt * h1;     // [h1]
    float* w2s = b1s + h1;                  // [hidden]
    for (int e = threadIdx.x; e < kt * h1; e += blockDim.x) w1s[e] = W1[(size_t)b * kw * h1 + e];
    for (int e = threadIdx.x; e < h1; e += blockDim.x) b1s[e] = b1[(size_t)b * h1 + e];
    for (int e = threadIdx.x; e < hidden; e += blockDim.x) w2s[e] = W2[(size_t)b * hidden + e];
    __syncthreads();
    const float sc = in_scale ? in_scale[b] : 1.0f;
    const float bias2 = hidden > 0 ? b2[b] : 0.0f;
    for (size_t r = (size_t)blockIdx.y * blockDim.x + threadIdx.x; r < n; r += (size_t)gridDim.y * blockDim.x) {
        const float* x = pooled + r * (size_t)k * nblock + (size_t)b * k;
        const float* xf = feats + r * (size_t)kf;                    // (only read when kf > 0)
        float xr[KMAX];
#pragma unroll
        for (int kk = 0; kk < KMAX; ++kk) xr[kk] = kk < k ? x[kk] * sc : (kk < kt ? xf[kk - k] : 0.0f);
        float out;
        if (hidden > 0) {
            out = 0.0f;
            int h = 0;
            // four hidden units at a time: one 16-byte broadcast read of LDS feeds four multiply-adds
            // (hidden % 4 == 0 keeps the reads aligned; taps ascending per unit, units ascending in the output sum)
            if ((hidden & 3) == 0) {
                for (; h < hidden; h += 4) {
                    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
#pragma unroll
                    for (int kk = 0; kk < KMAX; ++kk)
                        if (kk < kt) {
                            const float4 w = *reinterpret_cast<const float4*>(w1s + kk * hidden + h);
                            // fused multiply-add, as the reference's GEMM library issues them
                            a0 = __builtin_fmaf(xr[kk], w.x, a0);
                            a1 = __builtin_fmaf(xr[kk], w.y, a1);
                            a2 = __builtin_fmaf(xr[kk], w.z, a2);
                            a3 = __builtin_fmaf(xr[kk], w.w, a3);
                        }
                    const float4 bb = *reinterpret_cast<const float4*>(b1s + h);
                    const float4 ww = *reinterpret_cast<const float4*>(w2s + h);
                    a0 += bb.x; a1 += bb.y; a2 += bb.z; a3 += bb.w;
                    out += (a0 > 0.0f ? a0 : 0.0f) * ww.x;
                    out += (a1 > 0.0f ? a1 : 0.0f) * ww.y;
                    out += (a2 > 0.0f ? a2 : 0.0f) * ww.z;
                    out += (a3 > 0.0f ? a3 : 0.0f) * ww.w;
                }
            }
            for (; h < hidden; ++h) {
                float a = 0.0f;
#pragma unroll
                for (int kk = 0; kk < KMAX; ++kk)
                    if (kk < kt) a += xr[kk] * w1s[kk * hidden + h];
                a += b1s[h];
                a = a > 0.0f ? a : 0.0f;
                out += a * w2s[h];
            }
            out += bias2;
        } else {
            out = 0.0f;
#pragma unroll
            for (int kk = 0; kk < KMAX; ++kk)
                if (kk < kt) out += xr[kk] * w1s[kk];
            out += b1s[0];
        }
        if (apply_logistic) out = 1.0f / (1.0f + expf(-out));
        scores[r * (size_t)nblock + b] = out;
    }
}

// Scoring head, coalesced variant for hidden % 4 == 0: a workgroup owns 16 consecutive models and a tile of
// 16 rows (x 4, 2 or 1 rows per lane) per pass; lane = (row, model) with the model fastest, so a wave's reads of the
// feature matrix cover four contiguous 16*k*4-byte row segments. The 16 models' first-layer weights sit in LDS as
// [input][hidden/4][model][4]: the 16 lanes of a row read one aligned 256-byte line per ds_read_b128,
// and the four rows of a wave read the same line.
constexpr int HG = 16;
template <int KMAX>
__global__ __launch_bounds__(256) void k_head16(size_t n, int nblock, int k, int kf, int kw, int hidden, const float* __restrict__ pooled,
                                                const float* __restrict__ feats,
                                                const float* __restrict__ in_scale, const float* __restrict__ W1,
                                                const float* __restrict__ b1, const float* __restrict__ W2,
                                                const float* __restrict__ b2, bool apply_logistic, float* __restrict__ scores)
{
    extern __shared__ __align__(16) float hsm[];
    const int hq = hidden >> 2, kt = k + kf;            // inputs read: the model's own k, then kf shared feature columns
    float* w1s = hsm;                                   // [kt][hq][HG][4]
    float* b1s = w1s + (size_t)kt * hidden * HG;        // [hq][HG][4]
    float* w2s = b1s + (size_t)hidden * HG;             // [hq][HG][4]
    const unsigned g = threadIdx.x & (HG - 1), rl = threadIdx.x >> 4;
    const unsigned m0 = blockIdx.x * HG;                // first model of this workgroup
    for (int e = threadIdx.x; e < kt * hidden * HG; e += blockDim.x) {
        // destination order: e = ((kk*hq + h4)*HG + gg)*4 + c
        const int c = e & 3, gg = (e >> 2) & (HG - 1), rest = e >> 6, h4 = rest % hq, kk = rest / hq;
        const unsigned mdl = m0 + gg;
        w1s[e] = mdl < (unsigned)nblock ? W1[((size_t)mdl * kw + kk) * hidden + h4 * 4 + c] : 0.0f;
    }
    for (int e = threadIdx.x; e < hidden * HG; e += blockDim.x) {
        const int c = e & 3, gg = (e >> 2) & (HG - 1), h4 = e >> 6;
        const unsigned mdl = m0 + gg;
        b1s[e] = mdl < (unsigned)nblock ? b1[(size_t)mdl * hidden + h4 * 4 + c] : 0.0f;
        w2s[e] = mdl < (unsigned)nblock ? W2[(size_t)mdl * hidden + h4 * 4 + c] : 0.0f;
    }
    __syncthreads();
    const unsigned mdl = m0 + g;
    const bool live = mdl < (unsigned)nblock;
    const float sc = (in_scale && live) ? in_scale[mdl] : 1.0f;
    const float bias2 = live ? b2[mdl] : 0.0f;
    const float4* w1v = reinterpret_cast<const float4*>(w1s) + g;
    const float4* b1v = reinterpret_cast<const float4*>(b1s) + g;
    const float4* w2v = reinterpret_cast<const float4*>(w2s) + g;
    if (!live) return;                                   // (after the only barrier)
    // A pass takes 16 * HR rows: this lane rows base + rl + 16 j, j < HR, of its model. Every weight read from LDS serves
    // the HR rows (one ds_read_b128 per 4 * HR multiply-adds), each row's sums are formed as for a single row; a row's
    // inputs arrive as 16-byte loads where a model's k inputs are whole packs.
    constexpr int HR = KMAX <= 16 ? 4 : (KMAX <= 32 ? 2 : 1);      // (the rows' inputs stay in registers: 64 of them)
    const size_t rowlen = (size_t)k * nblock;
    const bool packs = k == KMAX && kf == 0 && (reinterpret_cast<uintptr_t>(pooled) & 15u) == 0;
    for (size_t base = (size_t)blockIdx.y * (16 * HR); base < n; base += (size_t)gridDim.y * (16 * HR)) {
        float xr[HR][KMAX];
#pragma unroll
        for (int j = 0; j < HR; ++j) {
            const size_t r = base + rl + 16 * j;
            if (packs) {
                const float4* src = reinterpret_cast<const float4*>(pooled + (r < n ? r : n - 1) * rowlen + (size_t)mdl * k);
#pragma unroll
                for (int q = 0; q < KMAX / 4; ++q) {
                    const float4 v = src[q];
                    xr[j][4 * q] = v.x * sc; xr[j][4 * q + 1] = v.y * sc; xr[j][4 * q + 2] = v.z * sc; xr[j][4 * q + 3] = v.w * sc;
                }
            } else {
#pragma unroll
                for (int kk = 0; kk < KMAX; ++kk) {
                    const float v = r < n ? (kk < k ? pooled[r * rowlen + (size_t)mdl * k + kk] : (kk < kt ? feats[r * (size_t)kf + (kk - k)] : 0.0f)) : 0.0f;
                    xr[j][kk] = kk < k ? v * sc : v;
                }
            }
        }
        float out[HR];
#pragma unroll
        for (int j = 0; j < HR; ++j) out[j] = 0.0f;
        for (int h4 = 0; h4 < hq; ++h4) {
            float a[HR][4];
#pragma unroll
            for (int j = 0; j < HR; ++j) a[j][0] = a[j][1] = a[j][2] = a[j][3] = 0.0f;
#pragma unroll
            for (int kk = 0; kk < KMAX; ++kk)
                if (kk < kt) {
                    const float4 w = w1v[(kk * hq + h4) * HG];
#pragma unroll
                    for (int j = 0; j < HR; ++j) {
                        a[j][0] = __builtin_fmaf(xr[j][kk], w.x, a[j][0]);
                        a[j][1] = __builtin_fmaf(xr[j][kk], w.y, a[j][1]);
                        a[j][2] = __builtin_fmaf(xr[j][kk], w.z, a[j][2]);
                        a[j][3] = __builtin_fmaf(xr[j][kk], w.w, a[j][3]);
                    }
                }
            const float4 bb = b1v[h4 * HG], ww = w2v[h4 * HG];
#pragma unroll
            for (int j = 0; j < HR; ++j) {
                const float a0 = a[j][0] + bb.x, a1 = a[j][1] + bb.y, a2 = a[j][2] + bb.z, a3 = a[j][3] + bb.w;
                out[j] += (a0 > 0.0f ? a0 : 0.0f) * ww.x;
                out[j] += (a1 > 0.0f ? a1 : 0.0f) * ww.y;
                out[j] += (a2 > 0.0f ? a2 : 0.0f) * ww.z;
                out[j] += (a3 > 0.0f ? a3 : 0.0f) * ww.w;
            }
        }
#pragma unroll
        for (int j = 0; j < HR; ++j) {
            const size_t r = base + rl + 16 * j;
            float o = out[j] + bias2;
            if (apply_logistic) o = 1.0f / (1.0f + expf(-o));
            if (r < n) scores[r * (size_t)nblock + mdl] = o;
        }
    }
}

// Row-slice count for the kernels that stage 16 models' weights per workgroup: about 1024 workgroups in all
// (a few per CU), so that staging is paid once per many rows.
inline unsigned row_slices(size_t n, unsigned rows_per_pass, unsigned ngroups)
{
    unsigned cap = 1024u / (ngroups ? ngroups : 1u);
    if (cap < 1) cap = 1;
    unsigned gy = dbk::divup(n, rows_per_pass);
    if (gy > cap) gy = cap;
    if (gy > 65535u) gy = 65535u;
    return gy < 1 ? 1 : gy;
}

inline bool bulk_ok(int n, int m, int k) { return n >= 2048 && (m & 3) == 0 && m <= 64 && k <= 64; }

// returns -1 when the shape does not fit the bulk kernel (the caller falls back), else the launch status
template <typename T>
int launch_rowtile(hipStream_t st, int nblock, int n, int ni, int no, bool bcast, bool accumulate, bool transpose, int m, int p, int off,
                   const T* in, const T* W, T* out)
{
    if (!(no == 4 || no == 8 || no == 16 || no == 32 || no == 64) || ni > 64) return -1;
    const size_t smem = (size_t)ni * no * TG * sizeof(T);
    if (smem > 65536) return -1;
    const unsigned rpp = 256 / ((no / 4) * TG);
    const unsigned gy = row_slices((size_t)n, rpp, dbk::divup(nblock, TG));
    const dim3 grid(dbk::divup(nblock, TG), gy);
    auto kern = ni <= 16 ? k_bdot_rowtile<T, 16> : (ni <= 32 ? k_bdot_rowtile<T, 32> : k_bdot_rowtile<T, 64>);
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) return -1;
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, nblock, (size_t)n, ni, no, bcast, accumulate, transpose, m, p, off, in, W, out);
    return 0;
}

// The per-model products at bulk row counts on the matrix cores: out[r, b*no + o] = sum_i in[r, b*ni + i] * w_b[i][o]
// for ni = 16 * KS inputs and no <= 32 * NT outputs per model, both operands split into three bf16 pieces that add up
// to the float32 value exactly (six piece products, the small ones first, float32 accumulation: float32 results, the
// sums in another order than the vector kernels'). A wave owns one model and walks blocks of 32 rows; the model's
// weight pieces stay in its registers; a lane reads 8 consecutive inputs of its row (the matrix instruction's operand
// layout), the next block's while this block is multiplied (two blocks ahead: no faster). The four waves of a workgroup take four adjacent models,
// so the rows' segments they read and write lie side by side. `transpose`: w_b[i][o] = W_b[o][i] (the dot_nt case).
template <int KS, int NT>
__global__ __launch_bounds__(256) void k_bdot_mfma(int nblock, size_t n, int ni, int no, bool transpose, int m, int p, int off,
                                                   const float* __restrict__ in, const float* __restrict__ W, float* __restrict__ out)
{
    using namespace dbk_mfma;
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, col = lane & 31u, half = lane >> 5;
    const unsigned b = blockIdx.x * 4u + wave;
    if (b >= (unsigned)nblock) return;
    // weight pieces: lane = output column `col` of tile nt, inputs 16 ks + 8 half .. + 7
    uint4 B[KS][NT][3];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const unsigned o = nt * 32 + col, i0 = ks * 16 + 8 * half;
            unsigned lo[8], mid[8], hi[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float w = 0.0f;
                if (o < (unsigned)no)
                    w = transpose ? W[((size_t)b * p + off + o) * m + i0 + j] : W[((size_t)b * p + off + i0 + j) * m + o];
                split3(w, lo[j], mid[j], hi[j]);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                (&B[ks][nt][0].x)[q] = pack_upper_halves(lo[2 * q], lo[2 * q + 1]);
                (&B[ks][nt][1].x)[q] = pack_upper_halves(mid[2 * q], mid[2 * q + 1]);
                (&B[ks][nt][2].x)[q] = pack_upper_halves(hi[2 * q], hi[2 * q + 1]);
            }
        }
    const size_t ldin = (size_t)ni * nblock, ldout = (size_t)no * nblock;
    const float* src = in + (size_t)b * ni + 8 * half;
    float* dst = out + (size_t)b * no + col;
    const size_t nblk = (n + 31) / 32;
    auto request = [&](size_t blk, float4 (&x)[KS][2]) {
        size_t r = blk * 32 + col;
        if (r >= n) r = n - 1;                                     // (a row past the end: a valid address, its results are not stored)
        const float4* q = reinterpret_cast<const float4*>(src + r * ldin);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) { x[ks][0] = q[4 * ks]; x[ks][1] = q[4 * ks + 1]; }
    };
    float4 xn[KS][2];
    size_t blk = blockIdx.y;
    if (blk < nblk) request(blk, xn);
    for (; blk < nblk; blk += gridDim.y) {
        uint4 A[KS][3];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const float v[8] = {xn[ks][0].x, xn[ks][0].y, xn[ks][0].z, xn[ks][0].w, xn[ks][1].x, xn[ks][1].y, xn[ks][1].z, xn[ks][1].w};
            unsigned lo[8], mid[8], hi[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) split3(v[j], lo[j], mid[j], hi[j]);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                (&A[ks][0].x)[q] = pack_upper_halves(lo[2 * q], lo[2 * q + 1]);
                (&A[ks][1].x)[q] = pack_upper_halves(mid[2 * q], mid[2 * q + 1]);
                (&A[ks][2].x)[q] = pack_upper_halves(hi[2 * q], hi[2 * q + 1]);
            }
        }
        if (blk + gridDim.y < nblk) request(blk + gridDim.y, xn);
        const size_t r0 = blk * 32 + 4 * half;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            f32x16_t acc;
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                acc = mfma_bf16(A[ks][0], B[ks][nt][2], acc);     // lo . hi
                acc = mfma_bf16(A[ks][2], B[ks][nt][0], acc);     // hi . lo
                acc = mfma_bf16(A[ks][1], B[ks][nt][1], acc);     // mid . mid
                acc = mfma_bf16(A[ks][1], B[ks][nt][2], acc);     // mid . hi
                acc = mfma_bf16(A[ks][2], B[ks][nt][1], acc);     // hi . mid
                acc = mfma_bf16(A[ks][2], B[ks][nt][2], acc);     // hi . hi
            }
            if (nt * 32 + col < (unsigned)no) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const size_t r = r0 + (i & 3) + 8 * (i >> 2);
                    if (r < n) dst[r * ldout + nt * 32] = acc[i];
                }
            }
        }
    }
}

// returns -1 when the shape is not the matrix-core kernel's (the caller goes on to the vector kernels)
inline int launch_bdot_mfma(hipStream_t st, int nblock, int n, int ni, int no, bool transpose, int m, int p, int off,
                            const float* in, const float* W, float* out)
{
    if (n < 2048 || ni % 16 != 0 || ni > 64 || no % 16 != 0 || no > 64 || ((uintptr_t)in & 15) != 0) return -1;
    const int ks = ni / 16, nt = (no + 31) / 32;
    if (ks * nt > 4) return -1;
    const unsigned groups = dbk::divup(nblock, 4);
    unsigned gy = 2048u / groups;                                  // ~2 workgroups per SIMD in all
    const unsigned nblk = dbk::divup((size_t)n, 32);
    if (gy < 1) gy = 1;
    if (gy > nblk) gy = nblk;
    if (gy > 65535u) gy = 65535u;
    const dim3 grid(groups, gy);
#define DBK_BDOT_MFMA(KSV, NTV)                                                                                       \
    if (ks == KSV && nt == NTV) {                                                                                     \
        hipLaunchKernelGGL((k_bdot_mfma<KSV, NTV>), grid, dim3(256), 0, st, nblock, (size_t)n, ni, no, transpose, m, p, off, in, W, out); \
        return 0;                                                                                                     \
    }
    DBK_BDOT_MFMA(1, 1) DBK_BDOT_MFMA(2, 1) DBK_BDOT_MFMA(3, 1) DBK_BDOT_MFMA(4, 1) DBK_BDOT_MFMA(1, 2) DBK_BDOT_MFMA(2, 2)
#undef DBK_BDOT_MFMA
    return -1;
}

template <typename T>
int launch_bdot_tile(hipStream_t st, int nblock, int n, int m, int k, int p, int off, bool bcast, bool accumulate,
                     const T* X, const T* W, T* Z)
{
    if constexpr (sizeof(T) == 4)
        if (!bcast && !accumulate && launch_bdot_mfma(st, nblock, n, k, m, false, m, p, off, X, W, Z) == 0) return 0;
    if (launch_rowtile<T>(st, nblock, n, k, m, bcast, accumulate, false, m, p, off, X, W, Z) == 0) return 0;
    const size_t smem = (size_t)k * m * TG * sizeof(T);
    if (smem > 65536) return -1;
    const unsigned gy = row_slices((size_t)n, 16, dbk::divup(nblock, TG));
    const dim3 grid(dbk::divup(nblock, TG), gy);
#define DBK_BDOT_CASE(KM, MM)                                                                                         \
    if (k <= KM && m <= MM) {                                                                                         \
        auto kern = k_bdot_tile<T, KM, MM>;                                                                           \
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) return -1; \
        hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, nblock, (size_t)n, m, k, p, off, bcast, accumulate, X, W, Z); \
        return 0;                                                                                                     \
    }
    DBK_BDOT_CASE(16, 32) DBK_BDOT_CASE(32, 32) DBK_BDOT_CASE(64, 32) DBK_BDOT_CASE(16, 64) DBK_BDOT_CASE(32, 64) DBK_BDOT_CASE(64, 64)
#undef DBK_BDOT_CASE
    return -1;
}

template <typename T>
int launch_bdot_nt_tile(hipStream_t st, int nblock, int n, int m, int k, int p, int off, const T* dZ, const T* W, T* dX)
{
    if constexpr (sizeof(T) == 4)
        if (launch_bdot_mfma(st, nblock, n, m, k, true, m, p, off, dZ, W, dX) == 0) return 0;
    if (launch_rowtile<T>(st, nblock, n, m, k, false, false, true, m, p, off, dZ, W, dX) == 0) return 0;
    const size_t smem = (size_t)k * m * TG * sizeof(T);
    if (smem > 65536) return -1;
    const unsigned gy = row_slices((size_t)n, 16, dbk::divup(nblock, TG));
    const dim3 grid(dbk::divup(nblock, TG), gy);
#define DBK_BDOT_CASE(KM, MM)                                                                                         \
    if (k <= KM && m <= MM) {                                                                                         \
        auto kern = k_bdot_nt_tile<T, KM, MM>;                                                                        \
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) return -1; \
        hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, nblock, (size_t)n, m, k, p, off, dZ, W, dX);             \
        return 0;                                                                                                     \
    }
    DBK_BDOT_CASE(16, 32) DBK_BDOT_CASE(32, 32) DBK_BDOT_CASE(64, 32) DBK_BDOT_CASE(16, 64) DBK_BDOT_CASE(32, 64) DBK_BDOT_CASE(64, 64)
#undef DBK_BDOT_CASE
    return -1;
}

template <typename T>
int launch_bdot_tn_tile(hipStream_t st, int nblock, int n, int m, int k, int p, int off, bool bcast, const T* X, const T* dZ, T* dW)
{
    const unsigned nchunk = dbk::divup((size_t)n, TN_CHUNK);
    const size_t nout = (size_t)k * m * nblock;
    T* partial = (T*)dbk::workspace(nout * nchunk * sizeof(T), st);
    if (!partial) { dbk::set_error("MemoryError: could not allocate %zu bytes of scratch (%s)", nout * nchunk * sizeof(T), dbk::workspace_error()); return 1; }
    if constexpr (sizeof(T) == 4) {
        // 16 models per workgroup, rows read as whole segments
        if (!bcast && m == 32 && (k == 16 || k == 32) && nblock >= 2 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)dZ & 15) == 0 &&
            ((size_t)k * nblock) % 4 == 0) {
            const dim3 grid(dbk::divup(nblock, TN16_G), nchunk);
            if (k == 16) hipLaunchKernelGGL(k_bdot_tn16<16>, grid, dim3(256), 0, st, nblock, (size_t)n, (const float*)X, (const float*)dZ, (float*)partial);
            else hipLaunchKernelGGL(k_bdot_tn16<32>, grid, dim3(256), 0, st, nblock, (size_t)n, (const float*)X, (const float*)dZ, (float*)partial);
            hipLaunchKernelGGL(k_bdot_tn_fold<T>, dim3(dbk::ew_grid(nout)), dim3(256), 0, st, nblock, m, k, p, off, nchunk, (const T*)partial, dW);
            return 0;
        }
    }
    const size_t smem = (size_t)TN_ROWS * ((k | 1) + (m | 1)) * sizeof(T);
    auto kern = k_bdot_tn_tile<T>;
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(nblock, nchunk), dim3(256), smem, st, nblock, (size_t)n, m, k, bcast, X, dZ, partial);
    hipLaunchKernelGGL(k_bdot_tn_fold<T>, dim3(dbk::ew_grid(nout)), dim3(256), 0, st, nblock, m, k, p, off, nchunk, (const T*)partial, dW);
    return 0;
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
    if (bulk_ok(n, m, k)) {
        const int rc = dtype == DBK_F32
            ? launch_bdot_tile<float>(dbk::as_stream(stream), nblock, n, m, k, p, Xoffset, Xbroadcast != 0, Xoffset != 0, (const float*)X, (const float*)W, (float*)Z)
            : launch_bdot_tile<double>(dbk::as_stream(stream), nblock, n, m, k, p, Xoffset, Xbroadcast != 0, Xoffset != 0, (const double*)X, (const double*)W, (double*)Z);
        if (rc >= 0) { if (rc) return rc; DBK_LAUNCH_OK(); }
    }
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
    if (bulk_ok(n, m, k)) {
        const int rc = dtype == DBK_F32
            ? launch_bdot_nt_tile<float>(dbk::as_stream(stream), nblock, n, m, k, p, Xoffset, (const float*)dZ, (const float*)W, (float*)dX)
            : launch_bdot_nt_tile<double>(dbk::as_stream(stream), nblock, n, m, k, p, Xoffset, (const double*)dZ, (const double*)W, (double*)dX);
        if (rc >= 0) { if (rc) return rc; DBK_LAUNCH_OK(); }
    }
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
    if (n >= 2048 && k * m <= 256 * TN_OWN) {
        const int rc = dtype == DBK_F32
            ? launch_bdot_tn_tile<float>(dbk::as_stream(stream), nblock, n, m, k, p, Xoffset, Xbroadcast != 0, (const float*)X, (const float*)dZ, (float*)dW)
            : launch_bdot_tn_tile<double>(dbk::as_stream(stream), nblock, n, m, k, p, Xoffset, Xbroadcast != 0, (const double*)X, (const double*)dZ, (double*)dW);
        if (rc) return rc;
        DBK_LAUNCH_OK();
    }
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
                   const float* pooled, int nfeat, const float* feats, const float* in_scale,
                   const float* W1, const float* b1, const float* W2, const float* b2,
                   int apply_logistic, float* scores)
{
    DBK_CHECK(nblock >= 1 && k >= 1 && nfeat >= 0 && hidden >= 0, "ValueError: bad head shape (nblock=%d, k=%d, nfeat=%d, hidden=%d)", nblock, k, nfeat, hidden);
    if (n == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(pooled && W1 && b1 && scores, "ValueError: null pointer argument");
    DBK_CHECK(hidden == 0 || (W2 && b2), "ValueError: hidden layer requested but W2/b2 are null");
    // all-zero feature columns (feats == NULL) add nothing: their weight rows are stepped over, not read
    const int kw = k + nfeat, kf = feats ? nfeat : 0, kk_all = k + kf;
    DBK_CHECK(kk_all <= HEAD_MAXK, "ValueError: the fused head takes at most %d inputs per model (got %d)", HEAD_MAXK, kk_all);
    const int h1 = hidden > 0 ? hidden : 1;
    size_t smem = ((size_t)kk_all * h1 + h1 + hidden) * sizeof(float);
    DBK_CHECK(smem <= 65536, "ValueError: head weights (%zu bytes per model) do not fit in LDS", smem);
    unsigned gx = dbk::divup(n, 256);
    if (gx > 2048u) gx = 2048u;
    const size_t smem16 = ((size_t)kk_all * hidden + 2 * (size_t)hidden) * HG * sizeof(float);
    if (hidden > 0 && (hidden & 3) == 0 && smem16 <= 65536 && n >= 4096) {
        // bulk scoring: 16 models per workgroup, coalesced reads of the feature matrix
        const unsigned gy = row_slices(n, kk_all <= 16 ? 64 : (kk_all <= 32 ? 32 : 16), dbk::divup(nblock, HG));
        auto kern16 = kk_all <= 16 ? k_head16<16> : (kk_all <= 32 ? k_head16<32> : k_head16<64>);
        DBK_HIP(hipFuncSetAttribute((const void*)kern16, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem16));
        hipLaunchKernelGGL(kern16, dim3(dbk::divup(nblock, HG), gy), dim3(256), smem16, dbk::as_stream(stream), n, nblock, k, kf, kw, hidden, pooled,
                           feats, in_scale, W1, b1, W2, b2, apply_logistic != 0, scores);
        DBK_LAUNCH_OK();
    }
    auto kern = kk_all <= 16 ? k_head<16> : (kk_all <= 32 ? k_head<32> : k_head<64>);
    hipLaunchKernelGGL(kern, dim3(nblock, gx), dim3(256), smem, dbk::as_stream(stream), n, nblock, k, kf, kw, hidden, pooled, feats, in_scale,
                       W1, b1, W2, b2, apply_logistic != 0, scores);
    DBK_LAUNCH_OK();
}

}  // extern "C"

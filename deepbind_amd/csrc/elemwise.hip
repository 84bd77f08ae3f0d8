// Elementwise and small reduction kernels around the dense head: optimiser steps, per-model
// broadcast multiply-add, masks, dropout, and the handful of array ops the bias / ReLU / loss
// nodes are made of. All are grid-stride loops over flat arrays: consecutive lanes touch
// consecutive elements, so each wave moves whole 256-byte lines of HBM.
//
// Reference semantics: deepity_smat/gradstep.cu:41-72, madd_bcast.cu:41-47, maskout.cu:41-67,
// dropout.cu:41-109, kangaroo_smat/dropoutord.cu:41-52, smat_cuda/elemwise2.cu:42-77, elemwise3.cu:57-62.
#include "dbk_common.h"
#include "rng.h"

namespace {

using dbk_rng::philox4x32_10;
using dbk_rng::uniform_at;

#define GRID_STRIDE(i, n) for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < (n); i += (size_t)gridDim.x * blockDim.x)

// Z[i] = f(X[i]) and Z[i] = f(X[i], Y[i]) over flat arrays, launched through EWV: ONE access of 16 bytes per lane (four
// floats, two doubles) where every pointer is 16-byte aligned, thread t taking pack t; the threads after the last whole
// pack take the remaining elements one each. (A 1 GB map streams at 6.2 TB/s this way; grid-stride loops, whatever their
// grid and however many accesses they keep in flight, reached 4.6-5.5: the workgroups of a one-shot grid sweep the
// arrays in launch order.) Arrays that are not aligned go element by element in a grid-stride loop.
// Z may be X or Y itself: a lane writes only what it has read.
template <typename T> struct pack16 {
    static constexpr int V = 16 / sizeof(T);
    typedef T type __attribute__((ext_vector_type(16 / sizeof(T))));
};
template <typename T> __device__ __forceinline__ bool aligned16(const void* a, const void* b, const void* c = nullptr)
{
    return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15u) == 0;
}
template <typename T, typename F> __device__ __forceinline__ void map1(const T* X, T* Z, size_t n, F f)
{
    using P = typename pack16<T>::type;
    constexpr int V = pack16<T>::V;
    if (aligned16<T>(X, Z)) {
        const size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x, np = n / V;
        if (p < np) {
            const P a = reinterpret_cast<const P*>(X)[p];
            P z;
#pragma unroll
            for (int k = 0; k < V; ++k) z[k] = f(a[k]);
            reinterpret_cast<P*>(Z)[p] = z;
        } else if (np * V + (p - np) < n) {
            const size_t i = np * V + (p - np);
            Z[i] = f(X[i]);
        }
        return;
    }
    GRID_STRIDE(i, n) Z[i] = f(X[i]);
}
template <typename T, typename F> __device__ __forceinline__ void map2(const T* X, const T* Y, T* Z, size_t n, F f)
{
    using P = typename pack16<T>::type;
    constexpr int V = pack16<T>::V;
    if (aligned16<T>(X, Y, Z)) {
        const size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x, np = n / V;
        if (p < np) {
            const P a = reinterpret_cast<const P*>(X)[p], c = reinterpret_cast<const P*>(Y)[p];
            P z;
#pragma unroll
            for (int k = 0; k < V; ++k) z[k] = f(a[k], c[k]);
            reinterpret_cast<P*>(Z)[p] = z;
        } else if (np * V + (p - np) < n) {
            const size_t i = np * V + (p - np);
            Z[i] = f(X[i], Y[i]);
        }
        return;
    }
    GRID_STRIDE(i, n) Z[i] = f(X[i], Y[i]);
}
template <typename T> __global__ void k_gradstep(T* P, const T* dP, const T* drate, T* mP, const T* mrate, size_t n)
{
    GRID_STRIDE(i, n) {
        T delta = mP[i] * mrate[i] - dP[i] * drate[i];
        mP[i] = delta;
        P[i] += delta;
    }
}
template <typename T> __global__ void k_nesterov1(T* P, const T* mP, const T* mrate, size_t n)
{
    GRID_STRIDE(i, n) P[i] = P[i] + mrate[i] * mP[i];
}
template <typename T> __global__ void k_nesterov2(T* P, const T* dP, const T* drate, T* mP, const T* mrate, size_t n)
{
    GRID_STRIDE(i, n) {
        T delta = dP[i] * drate[i];
        mP[i] = mP[i] * mrate[i] - delta;
        P[i] -= delta;
    }
}
// Look-ahead kept beside the parameters: L = P + mrate*mP (the value nesterov1 leaves in P).
template <typename T> __global__ void k_lookahead(T* L, const T* P, const T* mP, const T* mrate, size_t n)
{
    GRID_STRIDE(i, n) L[i] = P[i] + mrate[i] * mP[i];
}
// nesterov2 on the look-ahead L, leaving the new parameters in P and the NEXT step's look-ahead in L:
// the same operations, in the same order, as nesterov2 followed by the next step's nesterov1.
template <typename T> __global__ void k_nesterov2_lookahead(T* P, T* L, const T* dP, const T* drate, T* mP, const T* mrate, size_t n)
{
    GRID_STRIDE(i, n) {
        const T delta = dP[i] * drate[i];
        const T mom = mP[i] * mrate[i] - delta;
        const T pn = L[i] - delta;
        mP[i] = mom;
        P[i] = pn;
        L[i] = pn + mrate[i] * mom;
    }
}
template <typename T> __global__ void k_madd_bcast(const T* A, const T* b, T* dst, size_t n, size_t m, size_t k)
{
    GRID_STRIDE(i, n) dst[i] += A[i] * b[(i / k) % m];
}
template <typename T> __global__ void k_maskout(const uint8_t* M, T* A, size_t n)
{
    GRID_STRIDE(i, n) if (!M[i]) A[i] = (T)0;
}
template <typename T> __global__ void k_calc_zmask(const T* Z, uint8_t* M, size_t n, size_t m)
{
    GRID_STRIDE(i, (n * m) / 2) {
        size_t row = (i / m) * 2, col = i % m, idx = m * row + col;
        if (Z[idx] >= Z[idx + m]) M[idx] = 1;
        else M[idx + m] = 1;
    }
}
// dropout on pooled features; U may be null (then the generator supplies the uniforms)
template <typename T> __global__ void k_dropout_fp_tr(const T* X, const T* rate, T* Z, uint8_t* M, size_t n, size_t m, size_t k,
                                                      const float* U, uint64_t seed, uint64_t offset)
{
    // a thread takes four consecutive elements: they share one call of the generator, and (when the arrays
    // allow it) one 16-byte load, one 16-byte store and one 4-byte mask store
    const bool vec = sizeof(T) == 4 && (n & 3) == 0 && ((reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(Z)) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(M) & 3) == 0 && (!U || (reinterpret_cast<uintptr_t>(U) & 15) == 0);
    GRID_STRIDE(q, (n + 3) / 4) {
        float u4[4];
        if (!U) dbk_rng::uniform4_at(seed, offset, q, u4);
        if (vec) {
            if (U) { const float4 uu = reinterpret_cast<const float4*>(U)[q]; u4[0] = uu.x; u4[1] = uu.y; u4[2] = uu.z; u4[3] = uu.w; }
            const float4 x = reinterpret_cast<const float4*>(X)[q];
            const float xs[4] = {x.x, x.y, x.z, x.w};
            float zs[4];
            unsigned mk = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const size_t i = 4 * q + j;
                const bool keep = (T)u4[j] >= rate[(i / k) % m];
                mk |= (unsigned)keep << (8 * j);
                zs[j] = xs[j] * (float)keep;
            }
            reinterpret_cast<float4*>(Z)[q] = make_float4(zs[0], zs[1], zs[2], zs[3]);
            reinterpret_cast<unsigned*>(M)[q] = mk;
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const size_t i = 4 * q + j;
            if (i < n) {
                T p = rate[(i / k) % m];
                float u = U ? U[i] : u4[j];
                bool keep = (T)u >= p;
                M[i] = keep;
                Z[i] = X[i] * (T)keep;
            }
        }
    }
}
template <typename T> __global__ void k_dropout_fp_tr_match(const T* X, const T* rate, T* Z, uint8_t* M, size_t nrow, size_t ncol,
                                                            size_t k, const float* U, uint64_t seed, uint64_t offset)
{
    const size_t npair = nrow * ncol / 2;
    const bool vec = sizeof(T) == 4 && (ncol & 3) == 0 && ((reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(Z)) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(M) & 3) == 0;
    GRID_STRIDE(q, (npair + 3) / 4) {
        float u4[4];
        if (!U) dbk_rng::uniform4_at(seed, offset, q, u4);
        if (vec) {
            // four consecutive pair indices are four consecutive columns of one row pair
            const size_t i = 4 * q, row = (i / ncol) * 2, col = i % ncol, i0 = row * ncol + col, i1 = i0 + ncol;
            if (U) { u4[0] = U[i0]; u4[1] = U[i0 + 1]; u4[2] = U[i0 + 2]; u4[3] = U[i0 + 3]; }
            const float4 a = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(X) + i0);
            const float4 b = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(X) + i1);
            const float as[4] = {a.x, a.y, a.z, a.w}, bs[4] = {b.x, b.y, b.z, b.w};
            float za[4], zb[4];
            unsigned mk = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool keep = (T)u4[j] >= rate[(col + j) / k];
                mk |= (unsigned)keep << (8 * j);
                za[j] = as[j] * (float)keep;
                zb[j] = bs[j] * (float)keep;
            }
            *reinterpret_cast<float4*>(reinterpret_cast<float*>(Z) + i0) = make_float4(za[0], za[1], za[2], za[3]);
            *reinterpret_cast<float4*>(reinterpret_cast<float*>(Z) + i1) = make_float4(zb[0], zb[1], zb[2], zb[3]);
            *reinterpret_cast<unsigned*>(M + i0) = mk;
            *reinterpret_cast<unsigned*>(M + i1) = mk;
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const size_t i = 4 * q + j;                    // pair index: the draw both rows of a pair share
            if (i < npair) {
                size_t row = (i / ncol) * 2, col = i % ncol;
                T p = rate[col / k];
                size_t i0 = row * ncol + col, i1 = i0 + ncol;
                float u = U ? U[i0] : u4[j];
                bool keep = (T)u >= p;
                M[i0] = keep; M[i1] = keep;
                Z[i0] = X[i0] * (T)keep;
                Z[i1] = X[i1] * (T)keep;
            }
        }
    }
}
template <typename T> __global__ void k_dropout_scale(const T* X, const T* rate, T* Z, size_t n, size_t m, size_t k)
{
    GRID_STRIDE(i, n) Z[i] = X[i] * ((T)1 - rate[(i / k) % m]);
}
template <typename T> __global__ void k_dropout_bp_tr(const T* dZ, const uint8_t* M, T* dX, size_t n)
{
    GRID_STRIDE(i, n) dX[i] = dZ[i] * (T)(M[i] != 0);
}
__global__ void k_dropoutord(const uint8_t* X, uint8_t* Z, uint8_t* M, size_t n, float rate, const float* U, uint64_t seed, uint64_t offset,
                             const unsigned long long* counter)
{
    if (counter) offset = counter[0];
    GRID_STRIDE(q, (n + 3) / 4) {
        float u4[4];
        if (!U) dbk_rng::uniform4_at(seed, offset, q, u4);
        if (4 * q + 3 < n && ((reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(Z) | reinterpret_cast<uintptr_t>(M)) & 3) == 0) {
            // four letters per 32-bit word
            const unsigned xw = reinterpret_cast<const unsigned*>(X)[q];
            unsigned zw = 0, mw = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const unsigned x = (xw >> (8 * j)) & 0xffu;
                const float u = U ? U[4 * q + j] : u4[j];
                const bool mask = x == 255u || u >= rate;
                mw |= (unsigned)mask << (8 * j);
                zw |= (mask ? x : 254u) << (8 * j);
            }
            reinterpret_cast<unsigned*>(Z)[q] = zw;
            reinterpret_cast<unsigned*>(M)[q] = mw;
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const size_t i = 4 * q + j;
            if (i < n) {
                float u = U ? U[i] : u4[j];
                uint8_t x = X[i];
                bool mask = x == 255 || u >= rate;          // padding always passes (and reports "kept")
                M[i] = mask;
                Z[i] = mask ? x : (uint8_t)254;
            }
        }
    }
}
// One workgroup per (fwd, rev) pair of regions: the reverse strand drops the mirrored letters of the
// forward strand. Regions are [leading pad | sequence]; letter t of the forward sequence pairs with
// letter len-1-t of the reverse one.
__global__ void k_dropoutord_mirror(const uint8_t* X, uint8_t* Z, uint8_t* M, const uint32_t* R, size_t npair, unsigned pad)
{
    for (size_t p = blockIdx.x; p < npair; p += gridDim.x) {
        const size_t a = R[4 * p], b = R[4 * p + 1], c = R[4 * p + 2], d = R[4 * p + 3];
        const size_t lf = b - a, lr = d - c;
        const size_t len = (lf < lr ? lf : lr);
        for (size_t t = threadIdx.x; t + pad < len; t += blockDim.x) {
            const size_t src = a + pad + t, dst = d - 1 - t;
            const uint8_t mk = M[src];
            M[dst] = mk;
            Z[dst] = mk ? X[dst] : (uint8_t)254;
        }
    }
}
template <typename T> __global__ void k_pair_max(const T* Z, T* out, size_t npair, size_t m)
{
    GRID_STRIDE(i, npair * m) {
        size_t r = i / m, c = i % m;
        T a = Z[(2 * r) * m + c], b = Z[(2 * r + 1) * m + c];
        out[i] = a >= b ? a : b;
    }
}
// Z (n x m) = X + b, b added to every row. One pack of 16 bytes per thread (launched through EWV) when the rows are
// whole packs (then a pack never straddles two rows and b's pack is aligned too) and the array has fewer than 2^32
// elements (32-bit index arithmetic).
template <typename T> __global__ void k_add_rowvec(const T* X, const T* b, T* Z, size_t n, size_t m)
{
    using P = typename pack16<T>::type;
    constexpr int V = pack16<T>::V;
    const size_t total = n * m;
    if (m % V == 0 && aligned16<T>(X, b, Z) && total < 0xffffffffull) {
        const size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (p < total / V) reinterpret_cast<P*>(Z)[p] = reinterpret_cast<const P*>(X)[p] + reinterpret_cast<const P*>(b)[(unsigned)p % (unsigned)(m / V)];
        return;
    }
    GRID_STRIDE(i, total) Z[i] = X[i] + b[i % m];
}
// Column sums in a fixed order. Workgroup (x, y) takes 64 columns and row slice y; wave w sums rows
// w, w+4, ... of the slice in ascending order (four rows in flight), the four waves are combined in
// wave order, and k_colsum_fold adds the slices in ascending order: the summation order depends only
// on the shape.
template <typename T> __global__ __launch_bounds__(256) void k_colsum(const T* __restrict__ X, T* __restrict__ out, size_t n, size_t m,
                                                                      size_t rows_per_slice)
{
    __shared__ T part[4][64];
    const unsigned lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const size_t c = (size_t)blockIdx.x * 64 + lane;
    const size_t r0 = (size_t)blockIdx.y * rows_per_slice;
    const size_t r1 = r0 + rows_per_slice < n ? r0 + rows_per_slice : n;
    T s = (T)0;
    if (c < m) {
        size_t r = r0 + w;
        for (; r + 12 < r1; r += 16) {
            const T a0 = X[r * m + c], a1 = X[(r + 4) * m + c], a2 = X[(r + 8) * m + c], a3 = X[(r + 12) * m + c];
            s += a0;
            s += a1;
            s += a2;
            s += a3;
        }
        for (; r < r1; r += 4) s += X[r * m + c];
    }
    part[w][lane] = s;
    __syncthreads();
    if (w == 0 && c < m) out[(size_t)blockIdx.y * m + c] = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
}
template <typename T> __global__ void k_colsum_fold(const T* __restrict__ partial, T* __restrict__ out, size_t m, unsigned nslice)
{
    GRID_STRIDE(c, m) {
        T s = partial[c];
#pragma unroll 8
        for (unsigned y = 1; y < nslice; ++y) s += partial[(size_t)y * m + c];
        out[c] = s;
    }
}
template <typename T> __global__ void k_relu(const T* X, T* Z, size_t n)
{
    map1(X, Z, n, [](T x) { return x > (T)0 ? x : (T)0; });   // NaN -> 0, as fmax(0, x)
}
template <typename T> __global__ void k_mul_sign(const T* dZ, const T* Z, T* dX, size_t n)
{
    map2(dZ, Z, dX, n, [](T g, T z) { return g * ((T)(z > (T)0) - (T)(z < (T)0)); });
}
template <typename T> __global__ void k_sign(const T* X, T* Z, size_t n)
{
    map1(X, Z, n, [](T x) { return (T)(x > (T)0) - (T)(x < (T)0); });
}
template <typename T> __global__ void k_logistic(const T* X, T* Z, size_t n)
{
    map1(X, Z, n, [](T x) { return (T)1 / ((T)1 + exp(-x)); });
}
template <typename T> __global__ void k_loss_terms(int kind, const T* Z, const T* Y, T* L, size_t n)
{
    GRID_STRIDE(i, n) {
        T z = Z[i], y = Y[i];
        if (kind == 0) {
            T a = z > (T)1e-15 ? z : (T)1e-15;
            T b = ((T)1 - z) > (T)1e-15 ? ((T)1 - z) : (T)1e-15;
            L[i] = log(a) * y + log(b) * ((T)1 - y);
        } else if (kind == 3) {                                    // bidirectional hinge (deepity/std/loss.py:162-163)
            T l = ((T)1 - y) * z + y * ((T)1 - z);
            L[i] = l > (T)0 ? l : (T)0;
        } else if (kind == 2) {                                    // several columns per output: multiclass term
            T a = z > (T)1e-15 ? z : (T)1e-15;
            L[i] = log(a) * y;
        } else {
            T d = z - y;
            L[i] = d * d;
        }
    }
}
// Softmax over groups of g consecutive elements (a row of a (rows x ncol) matrix holds ncol/g groups):
// z = exp(x - max) / sum(exp(x - max)), maximum and sum taken left to right. One thread per group.
template <typename T> __global__ void k_softmax_groups(const T* X, T* Z, size_t ngroups, size_t g)
{
    GRID_STRIDE(i, ngroups) {
        const T* x = X + i * g;
        T* z = Z + i * g;
        T mx = x[0];
        for (size_t c = 1; c < g; ++c) mx = x[c] > mx ? x[c] : mx;
        T s = (T)0;
        for (size_t c = 0; c < g; ++c) { const T e = exp(x[c] - mx); z[c] = e; s += e; }
        for (size_t c = 0; c < g; ++c) z[c] = z[c] / s;
    }
}
__global__ void k_uniform_fill(float* U, size_t n, uint64_t seed, uint64_t offset)
{
    GRID_STRIDE(q, (n + 3) / 4) {
        float u4[4];
        dbk_rng::uniform4_at(seed, offset, q, u4);
        if (4 * q + 3 < n && (reinterpret_cast<uintptr_t>(U) & 15) == 0) {
            reinterpret_cast<float4*>(U)[q] = make_float4(u4[0], u4[1], u4[2], u4[3]);
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (4 * q + j < n) U[4 * q + j] = u4[j];
    }
}
// Standard normals by Box-Muller from two independent Philox streams (third counter word 0 / 1), one value
// per element so that element i depends only on (seed, offset, i).
template <typename T> __global__ void k_l1_decay(const T* P, const T* decay, T* dP, size_t n)
{
    GRID_STRIDE(i, n) {
        const T w = P[i];
        const T sg = (T)((w > (T)0) - (w < (T)0));
        dP[i] += sg * decay[i];
    }
}
template <typename T> __global__ void k_normal_fill(T* Z, size_t n, uint64_t seed, uint64_t offset)
{
    GRID_STRIDE(q, (n + 3) / 4) {
        const uint64_t ctr = offset + (uint64_t)q;
        uint32_t a[4] = {(uint32_t)ctr, (uint32_t)(ctr >> 32), 0u, 0u};
        uint32_t b[4] = {(uint32_t)ctr, (uint32_t)(ctr >> 32), 1u, 0u};
        philox4x32_10(a, (uint32_t)seed, (uint32_t)(seed >> 32));
        philox4x32_10(b, (uint32_t)seed, (uint32_t)(seed >> 32));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const size_t i = 4 * q + j;
            const float u1 = ((float)(a[j] >> 8) + 1.0f) * (1.0f / 16777216.0f);      // (0, 1]
            const float u2 = (float)(b[j] >> 8) * (1.0f / 16777216.0f);               // [0, 1)
            if (i < n) Z[i] = (T)(sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2));
        }
    }
}
__global__ void k_counter_add(unsigned long long* ctr, unsigned long long delta) { if (threadIdx.x == 0 && blockIdx.x == 0) ctr[0] += delta; }
template <typename T> __global__ void k_sub_scale(const T* Z, const T* Y, T scale, T* dZ, size_t n)
{
    map2(Z, Y, dZ, n, [scale](T z, T y) { return (z - y) * scale; });
}
template <typename T> __global__ void k_hinge_grad(const T* Z, const T* Y, T scale, T* dZ, size_t n)
{
    GRID_STRIDE(i, n) {
        const T z = Z[i], y = Y[i];
        const T l = ((T)1 - y) * z + y * ((T)1 - z);
        dZ[i] = l > (T)0 ? ((T)1 - (T)2 * y) * scale : (T)0;
    }
}

}  // namespace

#define F32(p) ((float*)(p))
#define CF32(p) ((const float*)(p))
#define F64(p) ((double*)(p))
#define CF64(p) ((const double*)(p))

// The typed pointer casts differ per dtype, so each entry point spells out both launches.
// The scan filters' constraint, applied to W (4m, F) in place after every update (kangaroo/_ext/corr1ord.py:60-77):
// kind 0 "pfm": each filter tap's four letter weights become log(e / sum(e)), e = exp(w), letters added A,C,G,T;
// kind 1 "psam": log(e / max(e)); kind 2: clipped to [lo, hi] (minimum with hi first, then maximum with lo).
// One thread per (tap, filter); a wave reads four 256-byte row segments.
template <typename T> __global__ void k_scan_constraint(T* W, size_t m, size_t F, int kind, T lo, T hi)
{
    GRID_STRIDE(i, m * F) {
        const size_t tap = i / F, f = i % F;
        T* w = W + tap * 4 * F + f;
        T v[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = w[(size_t)c * F];
        if (kind == 2) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const T a = v[c] < hi ? v[c] : hi;
                w[(size_t)c * F] = a > lo ? a : lo;
            }
        } else {
            T e[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) e[c] = exp(v[c]);
            T d;
            if (kind == 0) { d = e[0]; d += e[1]; d += e[2]; d += e[3]; }
            else { d = e[0]; d = e[1] > d ? e[1] : d; d = e[2] > d ? e[2] : d; d = e[3] > d ? e[3] : d; }
#pragma unroll
            for (int c = 0; c < 4; ++c) w[(size_t)c * F] = log(e[c] / d);
        }
    }
}

#define EW2(kernel, n, ARGS32, ARGS64)                                                                     \
    do {                                                                                                   \
        DBK_DTYPE_OK(dtype);                                                                               \
        if ((n) == 0) { dbk::clear_error(); return 0; }                                                    \
        if (dtype == DBK_F32) hipLaunchKernelGGL(kernel<float>, dim3(dbk::ew_grid(n)), dim3(256), 0, dbk::as_stream(stream), ARGS32); \
        else hipLaunchKernelGGL(kernel<double>, dim3(dbk::ew_grid(n)), dim3(256), 0, dbk::as_stream(stream), ARGS64);                  \
        DBK_LAUNCH_OK();                                                                                   \
    } while (0)
// The launch of a kernel built on map1 / map2: one thread per pack of 16 bytes, plus the few that take the elements after
// the last whole pack (at most 2^31 - 1 workgroups: 2^41 bytes per array).
inline unsigned pack_grid(size_t n, size_t per_pack) { return (unsigned)dbk::divup(n / per_pack + per_pack, (size_t)256); }
#define EWV(kernel, n, ARGS32, ARGS64)                                                                     \
    do {                                                                                                   \
        DBK_DTYPE_OK(dtype);                                                                               \
        if ((n) == 0) { dbk::clear_error(); return 0; }                                                    \
        DBK_CHECK((n) < ((size_t)1 << 39), "ValueError: %zu elements are more than one launch takes", (size_t)(n)); \
        if (dtype == DBK_F32) hipLaunchKernelGGL(kernel<float>, dim3(pack_grid(n, 4)), dim3(256), 0, dbk::as_stream(stream), ARGS32); \
        else hipLaunchKernelGGL(kernel<double>, dim3(pack_grid(n, 2)), dim3(256), 0, dbk::as_stream(stream), ARGS64);                  \
        DBK_LAUNCH_OK();                                                                                   \
    } while (0)
#define A(...) __VA_ARGS__

template <typename T>
int launch_colsum(hipStream_t st, const T* X, T* out, size_t n, size_t m)
{
    const unsigned tiles = dbk::divup(m, 64);
    // slices of at least 256 rows, about 2048 workgroups in all
    size_t nslice = (n + 255) / 256;
    const size_t cap = 2048u / tiles > 0 ? 2048u / tiles : 1;
    if (nslice > cap) nslice = cap;
    if (nslice < 1) nslice = 1;
    const size_t rows_per = (n + nslice - 1) / nslice;
    if (nslice == 1) {
        hipLaunchKernelGGL(k_colsum<T>, dim3(tiles, 1), dim3(256), 0, st, X, out, n, m, rows_per);
        return 0;
    }
    T* partial = (T*)dbk::workspace(nslice * m * sizeof(T), st);
    if (!partial) { dbk::set_error("MemoryError: could not allocate %zu bytes of scratch (%s)", nslice * m * sizeof(T), dbk::workspace_error()); return 1; }
    hipLaunchKernelGGL(k_colsum<T>, dim3(tiles, (unsigned)nslice), dim3(256), 0, st, X, partial, n, m, rows_per);
    hipLaunchKernelGGL(k_colsum_fold<T>, dim3(dbk::ew_grid(m)), dim3(256), 0, st, (const T*)partial, out, m, (unsigned)nslice);
    return 0;
}

extern "C" {

int dbk_gradstep(dbk_stream_t stream, int dtype, size_t n, void* P, const void* dP, const void* drate, void* mP, const void* mrate)
{
    EW2(k_gradstep, n, A(F32(P), CF32(dP), CF32(drate), F32(mP), CF32(mrate), n), A(F64(P), CF64(dP), CF64(drate), F64(mP), CF64(mrate), n));
}
int dbk_gradstep_nesterov1(dbk_stream_t stream, int dtype, size_t n, void* P, const void* mP, const void* mrate)
{
    EW2(k_nesterov1, n, A(F32(P), CF32(mP), CF32(mrate), n), A(F64(P), CF64(mP), CF64(mrate), n));
}
int dbk_gradstep_nesterov2(dbk_stream_t stream, int dtype, size_t n, void* P, const void* dP, const void* drate, void* mP, const void* mrate)
{
    EW2(k_nesterov2, n, A(F32(P), CF32(dP), CF32(drate), F32(mP), CF32(mrate), n), A(F64(P), CF64(dP), CF64(drate), F64(mP), CF64(mrate), n));
}
int dbk_gradstep_lookahead(dbk_stream_t stream, int dtype, size_t n, void* L, const void* P, const void* mP, const void* mrate)
{
    EW2(k_lookahead, n, A(F32(L), CF32(P), CF32(mP), CF32(mrate), n), A(F64(L), CF64(P), CF64(mP), CF64(mrate), n));
}
int dbk_gradstep_nesterov2_lookahead(dbk_stream_t stream, int dtype, size_t n, void* P, void* L, const void* dP, const void* drate,
                                     void* mP, const void* mrate)
{
    EW2(k_nesterov2_lookahead, n, A(F32(P), F32(L), CF32(dP), CF32(drate), F32(mP), CF32(mrate), n),
        A(F64(P), F64(L), CF64(dP), CF64(drate), F64(mP), CF64(mrate), n));
}
int dbk_madd_bcast(dbk_stream_t stream, int dtype, const void* A_, const void* b, void* dst, size_t n, size_t m, size_t k)
{
    DBK_CHECK(m >= 1 && k >= 1, "ValueError: madd_bcast needs m >= 1 and k >= 1");
    EW2(k_madd_bcast, n, A(CF32(A_), CF32(b), F32(dst), n, m, k), A(CF64(A_), CF64(b), F64(dst), n, m, k));
}
int dbk_maskout(dbk_stream_t stream, int dtype, const uint8_t* M, void* A_, size_t n)
{
    EW2(k_maskout, n, A(M, F32(A_), n), A(M, F64(A_), n));
}
int dbk_calc_zmask(dbk_stream_t stream, int dtype, const void* Z, uint8_t* M, size_t n, size_t m)
{
    size_t half = (n * m) / 2;
    EW2(k_calc_zmask, half, A(CF32(Z), M, n, m), A(CF64(Z), M, n, m));
}

static int dropout_fp_tr_impl(dbk_stream_t stream, int dtype, const void* X, const void* rate, void* Z, uint8_t* M,
                              size_t n, size_t m, size_t k, int matchrows, const float* U, uint64_t seed, uint64_t offset)
{
    DBK_CHECK(m >= 1 && k >= 1, "ValueError: dropout needs at least one rate and one column per rate");
    if (matchrows) {
        size_t ncol = m * k, nrow = n / ncol, half = n / 2;
        DBK_CHECK(nrow % 2 == 0, "ValueError: matchrows needs an even number of rows, got %zu", nrow);
        EW2(k_dropout_fp_tr_match, half, A(CF32(X), CF32(rate), F32(Z), M, nrow, ncol, k, U, seed, offset),
            A(CF64(X), CF64(rate), F64(Z), M, nrow, ncol, k, U, seed, offset));
    }
    EW2(k_dropout_fp_tr, n, A(CF32(X), CF32(rate), F32(Z), M, n, m, k, U, seed, offset),
        A(CF64(X), CF64(rate), F64(Z), M, n, m, k, U, seed, offset));
}
int dbk_dropout_fp_tr(dbk_stream_t stream, int dtype, const void* X, const void* rate, void* Z, uint8_t* M,
                      size_t n, size_t m, size_t k, int matchrows, uint64_t seed, uint64_t offset)
{
    return dropout_fp_tr_impl(stream, dtype, X, rate, Z, M, n, m, k, matchrows, nullptr, seed, offset);
}
int dbk_dropout_fp_tr_u(dbk_stream_t stream, int dtype, const void* X, const void* rate, void* Z, uint8_t* M,
                        size_t n, size_t m, size_t k, int matchrows, const float* U)
{
    DBK_CHECK(U != nullptr, "ValueError: U must not be null");
    return dropout_fp_tr_impl(stream, dtype, X, rate, Z, M, n, m, k, matchrows, U, 0, 0);
}
int dbk_dropout_fp_te(dbk_stream_t stream, int dtype, const void* X, const void* rate, void* Z, size_t n, size_t m, size_t k)
{
    DBK_CHECK(m >= 1 && k >= 1, "ValueError: dropout needs at least one rate and one column per rate");
    EW2(k_dropout_scale, n, A(CF32(X), CF32(rate), F32(Z), n, m, k), A(CF64(X), CF64(rate), F64(Z), n, m, k));
}
int dbk_dropout_bp_tr(dbk_stream_t stream, int dtype, const void* dZ, const uint8_t* M, void* dX, size_t n)
{
    EW2(k_dropout_bp_tr, n, A(CF32(dZ), M, F32(dX), n), A(CF64(dZ), M, F64(dX), n));
}
int dbk_dropout_bp_te(dbk_stream_t stream, int dtype, const void* dZ, const void* rate, void* dX, size_t n, size_t m, size_t k)
{
    DBK_CHECK(m >= 1 && k >= 1, "ValueError: dropout needs at least one rate and one column per rate");
    EW2(k_dropout_scale, n, A(CF32(dZ), CF32(rate), F32(dX), n, m, k), A(CF64(dZ), CF64(rate), F64(dX), n, m, k));
}
int dbk_dropoutord_fp_tr(dbk_stream_t stream, const uint8_t* X, uint8_t* Z, uint8_t* M, size_t n, float rate, uint64_t seed, uint64_t offset,
                         const uint64_t* counter)
{
    if (n == 0) { dbk::clear_error(); return 0; }
    hipLaunchKernelGGL(k_dropoutord, dim3(dbk::ew_grid(n)), dim3(256), 0, dbk::as_stream(stream), X, Z, M, n, rate, (const float*)nullptr, seed, offset,
                       (const unsigned long long*)counter);
    DBK_LAUNCH_OK();
}
int dbk_dropoutord_mirror(dbk_stream_t stream, const uint8_t* X, uint8_t* Z, uint8_t* M, const uint32_t* regions, size_t nregion, size_t padding)
{
    DBK_CHECK(nregion % 2 == 0, "ValueError: reverse-complement regions come in pairs, got %zu", nregion);
    if (nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(X && Z && M && regions, "ValueError: null pointer argument");
    const size_t npair = nregion / 2;
    hipLaunchKernelGGL(k_dropoutord_mirror, dim3(npair < 4096 ? (unsigned)npair : 4096u), dim3(64), 0, dbk::as_stream(stream), X, Z, M, regions, npair,
                       (unsigned)padding);
    DBK_LAUNCH_OK();
}
int dbk_dropoutord_fp_tr_u(dbk_stream_t stream, const uint8_t* X, uint8_t* Z, uint8_t* M, size_t n, float rate, const float* U)
{
    DBK_CHECK(U != nullptr, "ValueError: U must not be null");
    if (n == 0) { dbk::clear_error(); return 0; }
    hipLaunchKernelGGL(k_dropoutord, dim3(dbk::ew_grid(n)), dim3(256), 0, dbk::as_stream(stream), X, Z, M, n, rate, U, (uint64_t)0, (uint64_t)0,
                       (const unsigned long long*)nullptr);
    DBK_LAUNCH_OK();
}
int dbk_pair_max(dbk_stream_t stream, int dtype, const void* Z, void* out, size_t n, size_t m)
{
    DBK_CHECK(n % 2 == 0, "ValueError: pair_max needs an even number of rows, got %zu", n);
    size_t total = (n / 2) * m;
    EW2(k_pair_max, total, A(CF32(Z), F32(out), n / 2, m), A(CF64(Z), F64(out), n / 2, m));
}
int dbk_add_rowvec(dbk_stream_t stream, int dtype, const void* X, const void* b, void* Z, size_t n, size_t m)
{
    size_t total = n * m;
    EWV(k_add_rowvec, total, A(CF32(X), CF32(b), F32(Z), n, m), A(CF64(X), CF64(b), F64(Z), n, m));
}
int dbk_colsum(dbk_stream_t stream, int dtype, const void* X, void* out, size_t n, size_t m)
{
    DBK_DTYPE_OK(dtype);
    if (m == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(dbk::divup(m, 64) <= 65535u, "ValueError: too many columns");
    DBK_CHECK(out && (X || n == 0), "ValueError: null pointer argument");
    int rc = dtype == DBK_F32 ? launch_colsum<float>(dbk::as_stream(stream), CF32(X), F32(out), n, m)
                              : launch_colsum<double>(dbk::as_stream(stream), CF64(X), F64(out), n, m);
    if (rc) return rc;
    DBK_LAUNCH_OK();
}
int dbk_corr1ord_constraint(dbk_stream_t stream, int dtype, void* W, size_t m, size_t nfilter, int kind, double lo, double hi)
{
    DBK_CHECK(kind >= 0 && kind <= 2, "NotImplementedError: constraint kind %d (0 = pfm, 1 = psam, 2 = clip to [lo, hi])", kind);
    DBK_CHECK(W || m * nfilter == 0, "ValueError: null pointer argument");
    EW2(k_scan_constraint, m * nfilter, A(F32(W), m, nfilter, kind, (float)lo, (float)hi), A(F64(W), m, nfilter, kind, lo, hi));
}
int dbk_relu(dbk_stream_t stream, int dtype, const void* X, void* Z, size_t n)
{
    EWV(k_relu, n, A(CF32(X), F32(Z), n), A(CF64(X), F64(Z), n));
}
int dbk_mul_sign(dbk_stream_t stream, int dtype, const void* dZ, const void* Z, void* dX, size_t n)
{
    EWV(k_mul_sign, n, A(CF32(dZ), CF32(Z), F32(dX), n), A(CF64(dZ), CF64(Z), F64(dX), n));
}
int dbk_sign(dbk_stream_t stream, int dtype, const void* X, void* Z, size_t n)
{
    EWV(k_sign, n, A(CF32(X), F32(Z), n), A(CF64(X), F64(Z), n));
}
int dbk_logistic(dbk_stream_t stream, int dtype, const void* X, void* Z, size_t n)
{
    EWV(k_logistic, n, A(CF32(X), F32(Z), n), A(CF64(X), F64(Z), n));
}
int dbk_loss_terms(dbk_stream_t stream, int dtype, int kind, const void* Z, const void* Y, void* L, size_t n)
{
    DBK_CHECK(kind >= 0 && kind <= 3, "ValueError: loss kind must be 0 (nll), 1 (mse), 2 (multiclass nll) or 3 (hinge), got %d", kind);
    EW2(k_loss_terms, n, A(kind, CF32(Z), CF32(Y), F32(L), n), A(kind, CF64(Z), CF64(Y), F64(L), n));
}
int dbk_softmax(dbk_stream_t stream, int dtype, const void* X, void* Z, size_t n, size_t group)
{
    DBK_CHECK(group >= 1 && n % group == 0, "ValueError: %zu elements do not split into groups of %zu", n, group);
    const size_t ngroups = n / group;
    EW2(k_softmax_groups, ngroups, A(CF32(X), F32(Z), ngroups, group), A(CF64(X), F64(Z), ngroups, group));
}
int dbk_sub_scale(dbk_stream_t stream, int dtype, const void* Z, const void* Y, double scale, void* dZ, size_t n)
{
    EWV(k_sub_scale, n, A(CF32(Z), CF32(Y), (float)scale, F32(dZ), n), A(CF64(Z), CF64(Y), scale, F64(dZ), n));
}
int dbk_hinge_grad(dbk_stream_t stream, int dtype, const void* Z, const void* Y, double scale, void* dZ, size_t n)
{
    EW2(k_hinge_grad, n, A(CF32(Z), CF32(Y), (float)scale, F32(dZ), n), A(CF64(Z), CF64(Y), scale, F64(dZ), n));
}

int dbk_uniform_fill(dbk_stream_t stream, float* U, size_t n, uint64_t seed, uint64_t offset)
{
    if (n == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(U != nullptr, "ValueError: U must not be null");
    hipLaunchKernelGGL(k_uniform_fill, dim3(dbk::ew_grid(n)), dim3(256), 0, dbk::as_stream(stream), U, n, seed, offset);
    DBK_LAUNCH_OK();
}

int dbk_l1_decay(dbk_stream_t stream, int dtype, const void* P, const void* decay, void* dP, size_t n)
{
    DBK_CHECK(dtype == DBK_F32 || dtype == DBK_F64, "TypeError: dtype must be float32 or float64");
    if (n == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(P && decay && dP, "ValueError: null pointer argument");
    if (dtype == DBK_F32)
        hipLaunchKernelGGL(k_l1_decay<float>, dim3(dbk::ew_grid(n)), dim3(256), 0, dbk::as_stream(stream), (const float*)P, (const float*)decay, (float*)dP, n);
    else
        hipLaunchKernelGGL(k_l1_decay<double>, dim3(dbk::ew_grid(n)), dim3(256), 0, dbk::as_stream(stream), (const double*)P, (const double*)decay, (double*)dP, n);
    DBK_LAUNCH_OK();
}

int dbk_normal_fill(dbk_stream_t stream, int dtype, void* Z, size_t n, uint64_t seed, uint64_t offset)
{
    DBK_CHECK(dtype == DBK_F32 || dtype == DBK_F64, "TypeError: dtype must be float32 or float64");
    if (n == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(Z != nullptr, "ValueError: Z must not be null");
    if (dtype == DBK_F32)
        hipLaunchKernelGGL(k_normal_fill<float>, dim3(dbk::ew_grid(n)), dim3(256), 0, dbk::as_stream(stream), (float*)Z, n, seed, offset);
    else
        hipLaunchKernelGGL(k_normal_fill<double>, dim3(dbk::ew_grid(n)), dim3(256), 0, dbk::as_stream(stream), (double*)Z, n, seed, offset);
    DBK_LAUNCH_OK();
}

int dbk_counter_add(dbk_stream_t stream, uint64_t* counter, uint64_t delta)
{
    DBK_CHECK(counter != nullptr, "ValueError: counter must not be null");
    hipLaunchKernelGGL(k_counter_add, dim3(1), dim3(64), 0, dbk::as_stream(stream), (unsigned long long*)counter, (unsigned long long)delta);
    DBK_LAUNCH_OK();
}

// Test hook: the raw Philox block function, so the host can check it against published vectors.
int dbk_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c[4] = {ctr[0], ctr[1], ctr[2], ctr[3]};
    philox4x32_10(c, key[0], key[1]);
    for (int i = 0; i < 4; ++i) out[i] = c[i];
    return 0;
}

}  // extern "C"

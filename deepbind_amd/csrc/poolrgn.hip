// Region pooling over the rows of an (N, F) feature map and its gradient.
//
// One thread per (region, column): the 64 lanes of a wave take 64 consecutive columns, so every
// row visit is one coalesced 256-byte read (or read-modify-write) of HBM. Rows are visited in
// ascending order, which fixes both the argmax tie rule (first strict maximum) and the order of
// the running sum.
//
// Reference semantics: kangaroo_smat/poolrgn.cuh:44-160 (forward), poolrgn_bprop.cuh:45-127 (gradient).
#include "dbk_common.h"

namespace {

struct region_t { size_t a, b, step, count; };

__device__ __forceinline__ region_t load_region(const uint32_t* __restrict__ R, size_t r, bool per_step)
{
    const uint32_t* p = R + r * (per_step ? 3 : 2);
    region_t g;
    g.a = p[0];
    g.b = p[1];
    g.step = per_step ? p[2] : 1;
    if (g.step == 0) g.step = 1;
    g.count = (g.b - g.a + g.step - 1) / g.step;
    return g;
}

template <typename T, int PT>
__global__ __launch_bounds__(256) void poolrgn_kernel(const T* __restrict__ U, size_t F, const uint32_t* __restrict__ R,
                                                      size_t P, bool per_step, T* __restrict__ pooled,
                                                      uint32_t* __restrict__ argmax)
{
    const size_t f = (size_t)blockIdx.y * 64 + (threadIdx.x & 63);
    const size_t r = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (f >= F || r >= P) return;
    const region_t g = load_region(R, r, per_step);
    size_t xi = g.a * F + f;
    T x = U[xi];
    T y = x;
    auto take = [&](size_t i, T v) {
        if (PT == DBK_PT_MAX || PT == DBK_PT_ALL) {
            if (v > x) { x = v; xi = i * F + f; }
        }
        if (PT != DBK_PT_MAX) y += v;
    };
    // eight rows per round: the loads of a round are in flight together, the rows are still taken in ascending order
    size_t i = g.a + g.step;
    for (; i + 7 * g.step < g.b; i += 8 * g.step) {
        T v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = U[(i + t * g.step) * F + f];
#pragma unroll
        for (int t = 0; t < 8; ++t) take(i + t * g.step, v[t]);
    }
    for (; i < g.b; i += g.step) take(i, U[i * F + f]);
    const size_t j = r * F + f;
    if (PT == DBK_PT_MAX) {
        pooled[j] = x;
    } else if (PT == DBK_PT_SUM) {
        pooled[j] = y;
    } else if (PT == DBK_PT_AVG) {
        pooled[j] = y / (T)g.count;
    } else {
        pooled[2 * j] = x;
        pooled[2 * j + 1] = y / (T)g.count;
    }
    if ((PT == DBK_PT_MAX || PT == DBK_PT_ALL) && argmax) argmax[j] = (uint32_t)xi;
}

// ---- sixteen bytes per lane -----------------------------------------------------------------------------------
// When a row is a whole number of 16-byte packs (four floats, two doubles) a lane takes one pack of one region: V
// neighbouring columns, each pooled exactly as poolrgn_kernel pools it. Thread t owns pack t % (F / V) of region
// t / (F / V), so the lanes of a wave read consecutive packs - whole rows when the map has 256 columns, 16 short
// regions side by side when it has 16 (where the one-column kernel leaves 48 of its 64 lanes idle) - and the map streams
// at 6 TB/s instead of 5.
template <typename T> struct pack_t {
    static constexpr int V = 16 / sizeof(T);
    typedef T type __attribute__((ext_vector_type(16 / sizeof(T))));
    typedef uint32_t index_type __attribute__((ext_vector_type(16 / sizeof(T))));
};

template <typename T, int PT>
__global__ __launch_bounds__(256) void poolrgn_pack_kernel(const T* __restrict__ U, unsigned F, const uint32_t* __restrict__ R,
                                                           unsigned P, bool per_step, T* __restrict__ pooled,
                                                           uint32_t* __restrict__ argmax)
{
    using V4 = typename pack_t<T>::type;
    using I4 = typename pack_t<T>::index_type;
    constexpr int V = pack_t<T>::V;
    const unsigned Fp = F / V;
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (size_t)P * Fp) return;
    const unsigned r = (unsigned)(t / Fp), f = (unsigned)(t - (size_t)r * Fp) * V;      // region; first of this lane's columns
    const region_t g = load_region(R, r, per_step);
    const V4* Up = reinterpret_cast<const V4*>(U + f);               // row i of the lane's pack: Up[i * Fp]
    V4 x = Up[g.a * Fp], y = x;
    I4 xr;                                                           // row of each column's maximum
#pragma unroll
    for (int k = 0; k < V; ++k) xr[k] = (uint32_t)g.a;
    auto take = [&](size_t i, const V4& v) {
#pragma unroll
        for (int k = 0; k < V; ++k) {
            if (PT == DBK_PT_MAX || PT == DBK_PT_ALL) {
                const bool gt = v[k] > x[k];
                x[k] = gt ? v[k] : x[k];
                xr[k] = gt ? (uint32_t)i : xr[k];
            }
            if (PT != DBK_PT_MAX) y[k] += v[k];
        }
    };
    // ROUND rows per round: the loads of a round are in flight together, the rows are still taken in ascending order
    constexpr int ROUND = 8;
    size_t i = g.a + g.step;
    for (; i + (ROUND - 1) * g.step < g.b; i += ROUND * g.step) {
        V4 v[ROUND];
#pragma unroll
        for (int q = 0; q < ROUND; ++q) v[q] = Up[(i + q * g.step) * Fp];
#pragma unroll
        for (int q = 0; q < ROUND; ++q) take(i + q * g.step, v[q]);
    }
    for (; i < g.b; i += g.step) take(i, Up[i * Fp]);
    I4 xi;
#pragma unroll
    for (int k = 0; k < V; ++k) xi[k] = (uint32_t)((size_t)xr[k] * F + f + k);
    const size_t j = (size_t)r * F + f;
    if (PT == DBK_PT_MAX) {
        *reinterpret_cast<V4*>(pooled + j) = x;
    } else if (PT == DBK_PT_SUM) {
        *reinterpret_cast<V4*>(pooled + j) = y;
    } else if (PT == DBK_PT_AVG) {
        V4 o;
#pragma unroll
        for (int k = 0; k < V; ++k) o[k] = y[k] / (T)g.count;
        *reinterpret_cast<V4*>(pooled + j) = o;
    } else {
        V4 o[2];
#pragma unroll
        for (int k = 0; k < V; ++k) {
            o[(2 * k) / V][(2 * k) % V] = x[k];
            o[(2 * k + 1) / V][(2 * k + 1) % V] = y[k] / (T)g.count;
        }
        reinterpret_cast<V4*>(pooled + 2 * j)[0] = o[0];
        reinterpret_cast<V4*>(pooled + 2 * j)[1] = o[1];
    }
    if ((PT == DBK_PT_MAX || PT == DBK_PT_ALL) && argmax) *reinterpret_cast<I4*>(argmax + j) = xi;
}

// LDS the packed forward asks for without using it: 40 KB leave four workgroups per CU instead of eight, and with fewer
// regions being read at the same time the map streams ~6 % faster (5.3 -> 5.6 TB/s at 8192 regions x 124 rows x 256).
constexpr size_t PACK_LDS_CAP = 40 * 1024;
template <typename T>
bool pack_shape(const void* U, size_t F, size_t P, const void* pooled, const void* index)
{
    constexpr size_t V = 16 / sizeof(T);
    return F % V == 0 && (double)P * (double)(F / V) < 2147483648.0 * 256.0 && F < 0x80000000u && P < 0x80000000u &&
           ((reinterpret_cast<uintptr_t>(U) | reinterpret_cast<uintptr_t>(pooled)) & 15u) == 0 &&
           (reinterpret_cast<uintptr_t>(index) & (4 * V - 1)) == 0;
}

// flag[0] = 1 when regions are sorted, unit-step and non-overlapping (each map element then has a
// single writer in the gradient kernel), else 0.
__global__ void regions_disjoint_kernel(const uint32_t* __restrict__ R, size_t P, bool per_step, unsigned* flag)
{
    __shared__ unsigned bad;
    if (threadIdx.x == 0) bad = 0;
    __syncthreads();
    unsigned mine = 0;
    const unsigned rc = per_step ? 3 : 2;
    for (size_t r = threadIdx.x; r < P; r += blockDim.x) {
        if (R[r * rc + 1] < R[r * rc]) mine = 1;
        if (per_step && R[r * rc + 2] != 1) mine = 1;
        if (r + 1 < P && R[(r + 1) * rc] < R[r * rc + 1]) mine = 1;
    }
    if (mine) atomicOr(&bad, 1u);
    __syncthreads();
    if (threadIdx.x == 0) flag[0] = bad ? 0u : 1u;
}

template <bool ATOMIC, typename T>
__device__ __forceinline__ void accumulate(T* p, T v)
{
    if (ATOMIC) atomicAdd(p, v);
    else *p += v;
}

// ATOMIC=false runs when flag says "disjoint" (plain read-modify-write, reproducible);
// ATOMIC=true runs otherwise (overlapping regions: same accumulation races as any scatter-add).
template <typename T, int PT, bool ATOMIC>
__global__ __launch_bounds__(256) void poolrgn_bprop_kernel(T* __restrict__ dU, size_t F, size_t nelem_map,
                                                            const uint32_t* __restrict__ R, size_t P, bool per_step,
                                                            const T* __restrict__ dP, const uint32_t* __restrict__ argmax,
                                                            const unsigned* __restrict__ flag)
{
    const bool disjoint = flag[0] != 0;
    if (disjoint == ATOMIC) return;
    const size_t f = (size_t)blockIdx.y * 64 + (threadIdx.x & 63);
    const size_t r = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (f >= F || r >= P) return;
    const region_t g = load_region(R, r, per_step);
    const size_t j = r * F + f;
    // The argmax index is caller data. One that lies in this thread's own column and region (what the forward
    // pass produces) has this thread as its only writer when regions are disjoint: a plain add. Any other index
    // may point anywhere in the map and is added atomically.
    auto scatter = [&](T v) {
        const size_t ai = argmax[j], row = ai / F;
        if (!ATOMIC && ai - row * F == f && row >= g.a && row < g.b) dU[ai] += v;
        else atomicAdd(&dU[ai], v);
    };
    if (PT == DBK_PT_MAX) {
        scatter(dP[j]);
        return;
    }
    T dy;
    if (PT == DBK_PT_ALL) dy = dP[2 * j + 1] / (T)g.count;
    else if (PT == DBK_PT_AVG) dy = dP[j] / (T)g.count;
    else dy = dP[j];
    size_t i = g.a;
    if (!ATOMIC) {
        // eight rows per round: read, add, write, with the eight reads in flight together
        for (; i + 7 * g.step < g.b; i += 8 * g.step) {
            T v[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) v[t] = dU[(i + t * g.step) * F + f];
#pragma unroll
            for (int t = 0; t < 8; ++t) dU[(i + t * g.step) * F + f] = v[t] + dy;
        }
    }
    for (; i < g.b; i += g.step) accumulate<ATOMIC>(&dU[i * F + f], dy);
    if (PT == DBK_PT_ALL) scatter(dP[2 * j]);
}

// The gradient of average / sum / max+average pooling with sixteen bytes per lane (regions disjoint, rows whole packs):
// thread t adds to pack t % (F / V) of every row of region t / (F / V), as poolrgn_pack_kernel reads them; every column
// receives what poolrgn_bprop_kernel<.., false> gives it, in the same order (the share of the average first, then the
// maximum's).
template <typename T, int PT>
__global__ __launch_bounds__(256) void poolrgn_bprop_pack_kernel(T* __restrict__ dU, unsigned F, const uint32_t* __restrict__ R, unsigned P,
                                                                 bool per_step, const T* __restrict__ dP,
                                                                 const uint32_t* __restrict__ argmax, const unsigned* __restrict__ flag)
{
    using V4 = typename pack_t<T>::type;
    constexpr int V = pack_t<T>::V;
    if (flag[0] == 0) return;                                        // overlapping regions: the atomic kernel runs instead
    const unsigned Fp = F / V;
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (size_t)P * Fp) return;
    const unsigned r = (unsigned)(t / Fp), f = (unsigned)(t - (size_t)r * Fp) * V;
    const region_t g = load_region(R, r, per_step);
    const size_t j = (size_t)r * F + f;
    V4 dy;
    if (PT == DBK_PT_ALL) {
        const V4 a = reinterpret_cast<const V4*>(dP + 2 * j)[0], b = reinterpret_cast<const V4*>(dP + 2 * j)[1];
#pragma unroll
        for (int k = 0; k < V; ++k) dy[k] = ((2 * k + 1) / V ? b : a)[(2 * k + 1) % V] / (T)g.count;
    } else {
        dy = *reinterpret_cast<const V4*>(dP + j);
        if (PT == DBK_PT_AVG) {
#pragma unroll
            for (int k = 0; k < V; ++k) dy[k] = dy[k] / (T)g.count;
        }
    }
    V4* Dp = reinterpret_cast<V4*>(dU + f);                          // row i of the lane's pack: Dp[i * Fp]
    size_t i = g.a;
    for (; i + 7 * g.step < g.b; i += 8 * g.step) {
        V4 v[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) v[q] = Dp[(i + q * g.step) * Fp];
#pragma unroll
        for (int q = 0; q < 8; ++q) Dp[(i + q * g.step) * Fp] = v[q] + dy;
    }
    for (; i < g.b; i += g.step) Dp[i * Fp] = Dp[i * Fp] + dy;
    if (PT == DBK_PT_ALL) {
        // the maximum's share: a plain add where the index lies in this lane's own column and region, else atomic
#pragma unroll
        for (int k = 0; k < V; ++k) {
            const size_t ai = argmax[j + k], row = ai / F;
            const T v = dP[2 * (j + k)];
            if (ai - row * F == f + k && row >= g.a && row < g.b) dU[ai] += v;
            else atomicAdd(&dU[ai], v);
        }
    }
}

template <typename T>
int launch_fwd(hipStream_t st, const T* U, size_t F, const uint32_t* R, size_t P, bool per_step, T* pooled,
               uint32_t* argmax, int ptype)
{
    if (pack_shape<T>(U, F, P, pooled, argmax)) {
        const dim3 grid(dbk::divup(P * (F / (16 / sizeof(T))), 256)), block(256);
        const unsigned F32 = (unsigned)F, P32 = (unsigned)P;
        switch (ptype) {
        case DBK_PT_MAX: hipLaunchKernelGGL((poolrgn_pack_kernel<T, DBK_PT_MAX>), grid, block, PACK_LDS_CAP, st, U, F32, R, P32, per_step, pooled, argmax); break;
        case DBK_PT_AVG: hipLaunchKernelGGL((poolrgn_pack_kernel<T, DBK_PT_AVG>), grid, block, PACK_LDS_CAP, st, U, F32, R, P32, per_step, pooled, argmax); break;
        case DBK_PT_SUM: hipLaunchKernelGGL((poolrgn_pack_kernel<T, DBK_PT_SUM>), grid, block, PACK_LDS_CAP, st, U, F32, R, P32, per_step, pooled, argmax); break;
        default:         hipLaunchKernelGGL((poolrgn_pack_kernel<T, DBK_PT_ALL>), grid, block, PACK_LDS_CAP, st, U, F32, R, P32, per_step, pooled, argmax); break;
        }
        DBK_LAUNCH_OK();
    }
    dim3 grid(dbk::divup(P, 4), dbk::divup(F, 64)), block(256);
    DBK_CHECK(grid.y <= 65535u, "ValueError: too many feature maps (%zu) for one launch", F);
    switch (ptype) {
    case DBK_PT_MAX: hipLaunchKernelGGL((poolrgn_kernel<T, DBK_PT_MAX>), grid, block, 0, st, U, F, R, P, per_step, pooled, argmax); break;
    case DBK_PT_AVG: hipLaunchKernelGGL((poolrgn_kernel<T, DBK_PT_AVG>), grid, block, 0, st, U, F, R, P, per_step, pooled, argmax); break;
    case DBK_PT_SUM: hipLaunchKernelGGL((poolrgn_kernel<T, DBK_PT_SUM>), grid, block, 0, st, U, F, R, P, per_step, pooled, argmax); break;
    default:         hipLaunchKernelGGL((poolrgn_kernel<T, DBK_PT_ALL>), grid, block, 0, st, U, F, R, P, per_step, pooled, argmax); break;
    }
    DBK_LAUNCH_OK();
}

template <typename T, int PT>
void launch_bwd_pt(hipStream_t st, T* dU, size_t F, const uint32_t* R, size_t P, bool per_step, const T* dP,
                   const uint32_t* argmax, const unsigned* flag)
{
    dim3 grid(dbk::divup(P, 4), dbk::divup(F, 64)), block(256);
    if (PT != DBK_PT_MAX && pack_shape<T>(dU, F, P, dP, nullptr))
        hipLaunchKernelGGL((poolrgn_bprop_pack_kernel<T, PT>), dim3(dbk::divup(P * (F / (16 / sizeof(T))), 256)), block, PACK_LDS_CAP, st, dU, (unsigned)F, R,
                           (unsigned)P, per_step, dP, argmax, flag);
    else
        hipLaunchKernelGGL((poolrgn_bprop_kernel<T, PT, false>), grid, block, 0, st, dU, F, (size_t)0, R, P, per_step, dP, argmax, flag);
    hipLaunchKernelGGL((poolrgn_bprop_kernel<T, PT, true>), grid, block, 0, st, dU, F, (size_t)0, R, P, per_step, dP, argmax, flag);
}

template <typename T>
int launch_bwd(hipStream_t st, T* dU, size_t F, const uint32_t* R, size_t P, bool per_step, const T* dP,
               const uint32_t* argmax, int ptype)
{
    DBK_CHECK(dbk::divup(F, 64) <= 65535u, "ValueError: too many feature maps (%zu) for one launch", F);
    unsigned* flag = (unsigned*)dbk::workspace(256, st);
    DBK_CHECK(flag != nullptr, "MemoryError: could not allocate scratch (%s)", dbk::workspace_error());
    hipLaunchKernelGGL(regions_disjoint_kernel, dim3(1), dim3(1024), 0, st, R, P, per_step, flag);
    switch (ptype) {
    case DBK_PT_MAX: launch_bwd_pt<T, DBK_PT_MAX>(st, dU, F, R, P, per_step, dP, argmax, flag); break;
    case DBK_PT_AVG: launch_bwd_pt<T, DBK_PT_AVG>(st, dU, F, R, P, per_step, dP, argmax, flag); break;
    case DBK_PT_SUM: launch_bwd_pt<T, DBK_PT_SUM>(st, dU, F, R, P, per_step, dP, argmax, flag); break;
    default:         launch_bwd_pt<T, DBK_PT_ALL>(st, dU, F, R, P, per_step, dP, argmax, flag); break;
    }
    DBK_LAUNCH_OK();
}

}  // namespace

extern "C" {

int dbk_poolrgn(dbk_stream_t stream, int dtype, const void* unpooledmaps, size_t nfeaturemap,
                const uint32_t* regions, size_t nregion, int per_region_step,
                void* pooledmaps, uint32_t* pooledmaps_argmax, int ptype)
{
    DBK_DTYPE_OK(dtype);
    DBK_CHECK(ptype >= DBK_PT_MAX && ptype <= DBK_PT_ALL, "ValueError: unknown pooling type %d", ptype);
    DBK_CHECK(!pooledmaps_argmax || ptype == DBK_PT_MAX || ptype == DBK_PT_ALL,
              "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    if (nfeaturemap == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(unpooledmaps && regions && pooledmaps, "ValueError: null pointer argument");
    if (dtype == DBK_F32)
        return launch_fwd<float>(dbk::as_stream(stream), (const float*)unpooledmaps, nfeaturemap, regions, nregion,
                                 per_region_step != 0, (float*)pooledmaps, pooledmaps_argmax, ptype);
    return launch_fwd<double>(dbk::as_stream(stream), (const double*)unpooledmaps, nfeaturemap, regions, nregion,
                              per_region_step != 0, (double*)pooledmaps, pooledmaps_argmax, ptype);
}

int dbk_poolrgn_bprop(dbk_stream_t stream, int dtype, void* unpooledmaps, size_t nfeaturemap,
                      const uint32_t* regions, size_t nregion, int per_region_step,
                      const void* pooledmaps, const uint32_t* pooledmaps_argmax, int ptype)
{
    DBK_DTYPE_OK(dtype);
    DBK_CHECK(ptype >= DBK_PT_MAX && ptype <= DBK_PT_ALL, "ValueError: unknown pooling type %d", ptype);
    if (ptype == DBK_PT_MAX || ptype == DBK_PT_ALL)
        DBK_CHECK(pooledmaps_argmax != nullptr, "ValueError: pooledmaps_argmax must be specified for max pooling.");
    else
        DBK_CHECK(pooledmaps_argmax == nullptr, "ValueError: pooledmaps_argmax can only be specified for max pooling.");
    if (nfeaturemap == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(unpooledmaps && regions && pooledmaps, "ValueError: null pointer argument");
    if (dtype == DBK_F32)
        return launch_bwd<float>(dbk::as_stream(stream), (float*)unpooledmaps, nfeaturemap, regions, nregion,
                                 per_region_step != 0, (const float*)pooledmaps, pooledmaps_argmax, ptype);
    return launch_bwd<double>(dbk::as_stream(stream), (double*)unpooledmaps, nfeaturemap, regions, nregion,
                              per_region_step != 0, (const double*)pooledmaps, pooledmaps_argmax, ptype);
}

}  // extern "C"

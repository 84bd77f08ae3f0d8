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
#include "mfma_common.h"
#include <type_traits>

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

// ---------------------------------------------------------------------------------------------
// Kernels for filters of at most MT taps (MT = 8, 16, 24, 32). All lanes of a wave look at the same
// positions, so the letters of a 16-position window are read once into scalar registers.
// ---------------------------------------------------------------------------------------------
constexpr unsigned WSUBS = 4;             // windows of PSUB positions per wave and staging round
constexpr unsigned WSUBS_W = 8;           // the same for the filter-gradient kernel

// forward: every (position, tap) is one LDS read with an immediate offset; taps in ascending order,
// so the sums are bit-identical to the any-length kernel's. A workgroup builds its filter tile's
// table once and walks chunks of 256 positions.
template <typename T, int MT>
__global__ __launch_bounds__(256) void corr1ord_window_kernel(const T* __restrict__ W, unsigned m, unsigned F,
                                                              const uint8_t* __restrict__ X, size_t n, T* __restrict__ Z)
{
    extern __shared__ __align__(16) unsigned char smem[];
    T* lut = reinterpret_cast<T*>(smem);                                   // [MT][NL][FT], zero rows past m
    uint8_t* xl = smem + (size_t)MT * NL * FT * sizeof(T);                 // 4-byte aligned
    const unsigned nw = blockDim.x >> 6, chunk = nw * WSUBS * PSUB;
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned f0 = blockIdx.y * FT, f = f0 + lane;
    const size_t N = n + m - 1;
    build_letter_table(lut, W, m, F, f0, MT);
    for (size_t c0 = (size_t)blockIdx.x * chunk; c0 < n; c0 += (size_t)gridDim.x * chunk) {
        const unsigned rows = (unsigned)((n - c0) < chunk ? (n - c0) : chunk);
        __syncthreads();
        stage(xl, X, N, c0, window_span<MT>(rows));
        __syncthreads();
#pragma unroll 1
        for (unsigned s = 0; s < WSUBS; ++s) {
            const unsigned p0 = (s * nw + wave) * PSUB;
            if (p0 >= rows) break;
            unsigned wq[window<MT>::words];
            load_window<MT>(xl, p0, wq);
            T acc[PSUB];
            scan16_window<MT>(lut, wq, lane, acc);
            if (f < F) {
#pragma unroll
                for (int p = 0; p < PSUB; ++p)
                    if (p0 + p < rows) Z[(c0 + p0 + p) * F + f] = acc[p];
            }
        }
    }
}

// forward, float32 and at most 24 taps: the lane's filter weights sit in register planes and the scan needs
// no table in LDS (one index-mode v_add_f32 per position and tap). Same additions in the same order as above.
template <int MT>
__global__ __launch_bounds__(256) void corr1ord_planes_kernel(const float* __restrict__ W, unsigned m, unsigned F,
                                                              const uint8_t* __restrict__ X, size_t n, float* __restrict__ Z)
{
    extern __shared__ __align__(16) unsigned char smem[];
    uint8_t* xl = smem;
    const unsigned nw = blockDim.x >> 6, chunk = nw * WSUBS_W * PSUB;
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned f0 = blockIdx.y * FT, f = f0 + lane;
    const size_t N = n + m - 1;
    grad_planes<MT> planes;
    weight_planes_load<MT>(planes, W, m, F, f);
    for (size_t c0 = (size_t)blockIdx.x * chunk; c0 < n; c0 += (size_t)gridDim.x * chunk) {
        const unsigned rows = (unsigned)((n - c0) < chunk ? (n - c0) : chunk);
        __syncthreads();
        stage(xl, X, N, c0, window_span<MT>(rows));
        __syncthreads();
#pragma unroll 1
        for (unsigned s = 0; s < WSUBS_W; ++s) {
            const unsigned p0 = (s * nw + wave) * PSUB;
            if (p0 >= rows) break;
            unsigned wq[window<MT>::words];
            load_window<MT>(xl, p0, wq);
            float acc[PSUB];
            scan16_planes<MT>(planes, wq, acc);
            if (f < F) {
#pragma unroll
                for (int p = 0; p < PSUB; ++p)
                    if (p0 + p < rows) Z[(c0 + p0 + p) * F + f] = acc[p];
            }
        }
    }
}

// forward, float32, 9 to 24 taps, many rows: four filters per lane (4l .. 4l+3: the table's ordinary row layout read
// as float4), ds_read_b128 on aligned 256-byte lines, a wave on its own 64 rows per round (no workgroup barrier after
// the table is built), one 16-byte store per lane and row: a quarter wave writes a whole 256-byte row segment.
// The register-plane kernel above is bound by the half-rate index-mode adds (0.36 ms for 6.24e9 adds); here the
// adds are plain and the LDS delivers twice the bytes per clock of the one-filter-per-lane table kernel.
// Same additions in the same order as above.
template <int MT>
__global__ __launch_bounds__(256) void corr1ord_wide_kernel(const float* __restrict__ W, unsigned m, unsigned F,
                                                            const uint8_t* __restrict__ X, size_t n, float* __restrict__ Z)
{
    extern __shared__ __align__(16) unsigned char smem[];
    float* lut = reinterpret_cast<float*>(smem);                   // [MT*NL][FT]
    const unsigned nw = blockDim.x >> 6;
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned qd = lane >> 4, l = lane & 15;
    uint8_t* xw = smem + (size_t)MT * NL * FT * sizeof(float) + (size_t)wave * wide_shape<MT>::xbytes;
    const unsigned f0 = blockIdx.y * FT, f = f0 + 4 * l;
    const size_t N = n + m - 1;
    build_letter_table(lut, W, m, F, f0, MT);
    __syncthreads();
    const float4* lut4 = reinterpret_cast<const float4*>(lut) + l;
    const bool vec = (F & 3u) == 0 && (reinterpret_cast<uintptr_t>(Z) & 15u) == 0;   // 16-byte stores allowed
    const size_t span = 4 * PSUB;
    for (size_t c0 = ((size_t)blockIdx.x * nw + wave) * span; c0 < n; c0 += (size_t)gridDim.x * nw * span) {
        unsigned wq[wide_shape<MT>::words];
        wide_stage<MT>(xw, X, N, c0, lane, wq);
        float4 acc[PSUB];
        scan16_wide<MT>(lut4, wq, acc);
        const size_t i0 = c0 + PSUB * qd;
#pragma unroll
        for (int p = 0; p < PSUB; ++p) {
            const size_t i = i0 + p;
            if (i >= n) break;
            float* dst = Z + i * F + f;
            if (vec) {
                if (f < F) *reinterpret_cast<float4*>(dst) = acc[p];
            } else {
                if (f + 0 < F) dst[0] = acc[p].x;
                if (f + 1 < F) dst[1] = acc[p].y;
                if (f + 2 < F) dst[2] = acc[p].z;
                if (f + 3 < F) dst[3] = acc[p].w;
            }
        }
    }
}

// filter gradient, pass 1: a lane keeps its filter's whole [letter][tap] column in registers; the window's
// letters (scalars) pick the register plane each gradient value is added into through the register index
// mode: one addition per (position, tap). "Mean of the four" letters collect in a plane of their own that
// is spread over the four channels (x 1/4) at the end.
// Workgroup y walks chunks y, y+gridDim.y, ... in ascending order; its waves are folded in wave order.
template <int MT>
__global__ __launch_bounds__(256) void corr1ord_bprop_W_window_kernel(float* __restrict__ partial, unsigned m, unsigned F,
                                                                      const uint8_t* __restrict__ X, size_t n,
                                                                      const float* __restrict__ dZ)
{
    extern __shared__ __align__(16) unsigned char smem[];
    float* fold = reinterpret_cast<float*>(smem);                          // [MT*4][FT]
    uint8_t* xl = smem + (size_t)MT * 4 * FT * sizeof(float);
    const unsigned nw = blockDim.x >> 6, chunk = nw * WSUBS_W * PSUB;
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned f0 = blockIdx.x * FT, f = f0 + lane;
    const size_t N = n + m - 1;
    grad_planes<MT> planes;                                                // [letter][tap] accumulators in fixed registers
    planes.clear();
    for (size_t c0 = (size_t)blockIdx.y * chunk; c0 < n; c0 += (size_t)gridDim.y * chunk) {
        const unsigned rows = (unsigned)((n - c0) < chunk ? (n - c0) : chunk);
        __syncthreads();
        stage(xl, X, N, c0, window_span<MT>(rows));
        __syncthreads();
        // the next window's gradient rows are requested before this window's additions start
        float g[PSUB], gn[PSUB];
        auto fetch = [&](unsigned p0, float (&dst)[PSUB]) {
#pragma unroll
            for (int p = 0; p < PSUB; ++p) dst[p] = (f < F && p0 + p < rows) ? dZ[(c0 + p0 + p) * F + f] : 0.0f;
        };
        fetch(wave * PSUB, g);
#pragma unroll 1
        for (unsigned s = 0; s < WSUBS_W; ++s) {
            const unsigned p0 = (s * nw + wave) * PSUB;
            if (p0 >= rows) break;
            fetch(p0 + nw * PSUB, gn);                                     // all zero past the chunk's rows
            unsigned wq[window<MT>::words];
            load_window<MT>(xl, p0, wq);
            grad_planes_window<MT>(planes, wq, g);                         // one add per (position, tap)
#pragma unroll
            for (int p = 0; p < PSUB; ++p) g[p] = gn[p];
        }
    }
    float aw[MT][4];
    grad_planes_read<MT>(planes, aw);
    float* mine = fold + lane;
    for (unsigned w = 0; w < nw; ++w) {
        __syncthreads();
        if (wave == w) {
#pragma unroll
            for (int j = 0; j < MT; ++j)
                if ((unsigned)j < m) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float* cell = mine + (j * 4 + c) * FT;
                        *cell = w == 0 ? aw[j][c] : *cell + aw[j][c];
                    }
                }
        }
    }
    __syncthreads();
    float* out = partial + (size_t)blockIdx.y * (4 * m) * F;
    for (unsigned e = threadIdx.x; e < m * 4 * FT; e += blockDim.x) {
        const unsigned row = e / FT, fl = e % FT;
        if (f0 + fl < F) out[(size_t)row * F + f0 + fl] = fold[e];
    }
}

// input gradient: a wave owns RPW consecutive rows and walks the filter tiles; a lane holds its filter's
// [tap][channel] weights in registers and a ring of the last MT gradient rows, so each row of dZ is read
// once per tile and each (row, tap, channel) is one multiply-add. Row sums over the 64 filters of a tile
// go through LDS eight rows at a time: every lane parks its 32 partial sums, then lane v < 32 adds up
// value v over the 64 lanes in lane order (a fixed order); tiles are added in ascending order into the
// wave's rows in LDS.
constexpr int XR_STRIDE = 65;             // odd row stride: the 32 column sums read 32 different banks
constexpr int XR_AHEAD = 4;               // rows of dZ in flight per lane

template <int MT, int RPW>
__global__ __launch_bounds__(256) void corr1ord_bprop_X_ring_kernel(float* __restrict__ dX, size_t n, const float* __restrict__ W,
                                                                    unsigned m, unsigned F, const float* __restrict__ dZ)
{
    static_assert(RPW % MT == 0 && MT % 8 == 0 && MT % XR_AHEAD == 0, "a wave's rows are walked in blocks of MT, reduced eight at a time");
    __shared__ float rows_acc[4][RPW * 4];
    __shared__ float parts[4][32 * XR_STRIDE];
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t i0 = ((size_t)blockIdx.x * 4 + wave) * RPW;
    if (i0 >= n) return;                                                   // (no barriers in this kernel)
    float* acc = rows_acc[wave];
    float* part = parts[wave];
    for (unsigned e = lane; e < RPW * 4; e += 64) acc[e] = 0.0f;
    const unsigned ftiles = (F + FT - 1) / FT;
    for (unsigned t = 0; t < ftiles; ++t) {
        const unsigned f = t * FT + lane;
        const bool live = f < F;
        float w[MT][4];
#pragma unroll
        for (int k = 0; k < MT; ++k) {
#pragma unroll
            for (int c = 0; c < 4; ++c) w[k][c] = (live && (unsigned)k < m) ? W[(size_t)(4 * k + c) * F + f] : 0.0f;
        }
        // ring slot r holds row i with i % MT == r (i0 is a multiple of MT); start with the MT-1 rows before i0
        float ring[MT];
        ring[0] = 0.0f;
#pragma unroll
        for (int r = 1; r < MT; ++r) {
            const bool have = i0 + r >= (size_t)MT;                         // row i0 - MT + r exists
            ring[r] = (live && have) ? dZ[(i0 - MT + r) * F + f] : 0.0f;
        }
        // rows are fetched XR_AHEAD positions before they are used (MT is a multiple of XR_AHEAD, so the
        // slot of a row is a compile-time index)
        float pre[XR_AHEAD];
#pragma unroll
        for (int d = 0; d < XR_AHEAD; ++d) pre[d] = (live && i0 + d < n) ? dZ[(i0 + d) * F + f] : 0.0f;
#pragma unroll 1
        for (unsigned b0 = 0; b0 < RPW; b0 += MT) {
            if (i0 + b0 >= n) break;
#pragma unroll
            for (int u = 0; u < MT; ++u) {
                ring[u] = pre[u % XR_AHEAD];
                {
                    const size_t i = i0 + b0 + u + XR_AHEAD;
                    pre[u % XR_AHEAD] = (live && i < n) ? dZ[i * F + f] : 0.0f;
                }
                float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
#pragma unroll
                for (int k = 0; k < MT; ++k) {
                    const float dz = ring[(u - k + MT) % MT];              // row i - k
                    s0 = __builtin_fmaf(dz, w[k][0], s0);
                    s1 = __builtin_fmaf(dz, w[k][1], s1);
                    s2 = __builtin_fmaf(dz, w[k][2], s2);
                    s3 = __builtin_fmaf(dz, w[k][3], s3);
                }
                float* mine = part + ((u & 7) * 4) * XR_STRIDE + lane;
                mine[0 * XR_STRIDE] = s0;
                mine[1 * XR_STRIDE] = s1;
                mine[2 * XR_STRIDE] = s2;
                mine[3 * XR_STRIDE] = s3;
                if ((u & 7) == 7) {
                    // the wave's own LDS accesses execute in program order; no other wave touches `part`
                    __builtin_amdgcn_wave_barrier();
                    if (lane < 32) {
                        const float* col = part + lane * XR_STRIDE;
                        float tot = 0.0f;
#pragma unroll 16
                        for (int l = 0; l < 64; ++l) tot += col[l];
                        acc[(b0 + u - 7) * 4 + lane] += tot;
                    }
                    __builtin_amdgcn_wave_barrier();
                }
            }
        }
    }
    for (unsigned e = lane; e < RPW * 4; e += 64) {
        const size_t i = i0 + e / 4;
        if (i < n) dX[i * 4 + (e & 3)] += acc[e];
    }
}

template <typename T>
int launch_fprop(hipStream_t st, const T* W, size_t m, size_t F, const uint8_t* X, size_t n, T* Z)
{
    const unsigned mt = m <= 8 ? 8 : (m <= 16 ? 16 : (m <= 24 ? 24 : (m <= 32 ? 32 : 0)));
    if constexpr (sizeof(T) == 4) {
        // many rows of 9-24 taps: four filters per lane (enough waves of 64 rows to fill the GPU's 3072 wave slots)
        if ((mt == 16 || mt == 24) && (n + 63) / 64 * dbk::divup(F, FT) >= 4096) {
            const unsigned ftiles = dbk::divup(F, FT);
            DBK_CHECK(ftiles <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
            const size_t smem_q = (size_t)mt * NL * FT * sizeof(float) + 4 * (mt == 16 ? wide_shape<16>::xbytes : wide_shape<24>::xbytes);
            if (smem_q <= lds_limit()) {
                unsigned gx = 768u / ftiles;                       // three workgroups per CU are resident
                if (gx < 1) gx = 1;
                if (gx > dbk::divup(n, 256)) gx = dbk::divup(n, 256);
                auto kq = mt == 16 ? corr1ord_wide_kernel<16> : corr1ord_wide_kernel<24>;
                DBK_HIP(hipFuncSetAttribute((const void*)kq, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_q));
                hipLaunchKernelGGL(kq, dim3(gx, ftiles), dim3(256), smem_q, st, (const float*)W, (unsigned)m, (unsigned)F, X, n, (float*)Z);
                DBK_LAUNCH_OK();
            }
        }
        if (mt && mt <= 24) {
            const unsigned ftiles = dbk::divup(F, FT), chunk = 4 * WSUBS_W * PSUB;
            DBK_CHECK(ftiles <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
            const size_t smem_p = (chunk + mt - 1 + 7) & ~(size_t)3;
            unsigned gx = (mt == 8 ? 768u : 512u) / ftiles;         // the register planes leave room for two workgroups per CU (three with 8 taps)
            if (gx < 1) gx = 1;
            if (gx > dbk::divup(n, chunk)) gx = dbk::divup(n, chunk);
            auto kp = mt == 8 ? corr1ord_planes_kernel<8> : mt == 16 ? corr1ord_planes_kernel<16> : corr1ord_planes_kernel<24>;
            hipLaunchKernelGGL(kp, dim3(gx, ftiles), dim3(256), smem_p, st, (const float*)W, (unsigned)m, (unsigned)F, X, n, (float*)Z);
            DBK_LAUNCH_OK();
        }
    }
    if (mt) {
        const unsigned ftiles = dbk::divup(F, FT), chunk = 4 * WSUBS * PSUB;
        DBK_CHECK(ftiles <= 65535u, "ValueError: too many filters (%zu) for one launch", F);
        const size_t smem_w = (size_t)mt * NL * FT * sizeof(T) + ((chunk + mt - 1 + 7) & ~(size_t)3);
        if (smem_w <= lds_limit()) {
            unsigned gx = 1024u / ftiles;                      // a few resident workgroups per CU, each building its table once
            if (gx < 1) gx = 1;
            if (gx > dbk::divup(n, chunk)) gx = dbk::divup(n, chunk);
            auto kw = mt == 8 ? corr1ord_window_kernel<T, 8> : mt == 16 ? corr1ord_window_kernel<T, 16>
                    : mt == 24 ? corr1ord_window_kernel<T, 24> : corr1ord_window_kernel<T, 32>;
            DBK_HIP(hipFuncSetAttribute((const void*)kw, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_w));
            hipLaunchKernelGGL(kw, dim3(gx, ftiles), dim3(256), smem_w, st, W, (unsigned)m, (unsigned)F, X, n, Z);
            DBK_LAUNCH_OK();
        }
    }
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

// The same sum for many slabs: a workgroup takes 64 elements, each of its four waves a quarter of the slabs (pairwise
// in eights, as above), and the four quarter sums are added as (q0 + q1) + (q2 + q3): four times as many loads in
// flight per element, a shape that depends on nslab only.
__global__ __launch_bounds__(256) void reduce_partials_quarters_kernel(float* __restrict__ dW, const float* __restrict__ partial, size_t nelem, unsigned nslab)
{
    __shared__ float part[4][64];
    const unsigned el = threadIdx.x & 63, q = threadIdx.x >> 6;
    const size_t e = (size_t)blockIdx.x * 64 + el;
    const unsigned per = (nslab + 3) / 4, first = q * per, last = first + per < nslab ? first + per : nslab;
    float total = 0.0f;
    if (e < nelem) {
        for (unsigned base = first; base < last; base += 8) {
            float buf[8];
#pragma unroll
            for (unsigned s = 0; s < 8; ++s) buf[s] = base + s < last ? partial[(size_t)(base + s) * nelem + e] : 0.0f;
            total += ((buf[0] + buf[1]) + (buf[2] + buf[3])) + ((buf[4] + buf[5]) + (buf[6] + buf[7]));
        }
    }
    part[q][el] = total;
    __syncthreads();
    if (q == 0 && e < nelem) dW[e] += (part[0][el] + part[1][el]) + (part[2][el] + part[3][el]);
}

// ---------------------------------------------------------------------------------------------
// forward on the matrix cores (float32, filters of up to 32 taps, bulk sizes)
// ---------------------------------------------------------------------------------------------
// Z (n x F) = H (n x 4m) . W (4m x F), H the one-hot windows (see the filter gradient below: the same exact
// bf16 operands, here with W in three pieces). A wave owns 32 filters (its pieces of W stay in registers) and a
// share of the rows, which it takes in chunks of 192: the chunk's letters become a table in LDS of one entry per
// position (the one-hot rows of this letter and the next, 8 bf16), a lane's operand for a k-step is one 16-byte
// read, and each block of 32 rows leaves the accumulator as 16 row segments of 128 bytes. The sums are those of the
// lookup kernels above in another order: equal to round-off, not bit for bit (which is why only bulk sizes come here).
constexpr unsigned GF_CHUNK = 192, GF_TABLE = 256;                 // rows per chunk; positions in its table (rows + window)

template <int KS>
__global__ __launch_bounds__(256) void corr1ord_mfma_kernel(const float* __restrict__ W, unsigned m, unsigned F,
                                                            const uint8_t* __restrict__ X, size_t n, float* __restrict__ Z,
                                                            unsigned chunks_per_wg)
{
    using namespace dbk_mfma;
    extern __shared__ __align__(16) unsigned char smem[];
    uint2* onehot = reinterpret_cast<uint2*>(smem);               // [256]: the four bf16 of a letter code's rows
    const unsigned lane = threadIdx.x & 63, wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned col = lane & 31, g = lane >> 5;
    uint4* hotw = reinterpret_cast<uint4*>(smem + 256 * 8) + (size_t)wave * (2 * GF_TABLE);   // this wave's tables: the chunk in work, the next one
    {
        const unsigned c = threadIdx.x, one = 0x3f80u, quarter = 0x3e803e80u;
        uint2 e;
        if (c < 4u) { e.x = c == 0u ? one : (c == 1u ? one << 16 : 0u); e.y = c == 2u ? one : (c == 3u ? one << 16 : 0u); }
        else if (c == 254u) { e.x = 0u; e.y = 0u; }
        else { e.x = quarter; e.y = quarter; }
        onehot[c] = e;
    }
    const size_t nbytes = n + m - 1;
    size_t c = (size_t)blockIdx.y * chunks_per_wg * GF_CHUNK;     // first row of the chunk in work
    const size_t end = c + (size_t)chunks_per_wg * GF_CHUNK < n ? c + (size_t)chunks_per_wg * GF_CHUNK : n;
    unsigned letters = c < end ? load_letters4(X, nbytes, c + 4u * lane) : 0xfefefefeu;
    // ---- this lane's column of W, rows 16s + 8g .. + 7 of every k-step, in three bf16 pieces
    const unsigned f = (blockIdx.x * 4 + wave) * 32 + col;
    uint4 B[KS][3];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        unsigned pc[3][8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const unsigned row = 16u * s + 8u * g + i;
            const float w = (row < 4u * m && f < F) ? W[(size_t)row * F + f] : 0.0f;
            split3(w, pc[0][i], pc[1][i], pc[2][i]);
        }
#pragma unroll
        for (int q = 0; q < 3; ++q)
            B[s][q] = make_uint4(pack_upper_halves(pc[q][0], pc[q][1]), pack_upper_halves(pc[q][2], pc[q][3]),
                                 pack_upper_halves(pc[q][4], pc[q][5]), pack_upper_halves(pc[q][6], pc[q][7]));
    }
    __syncthreads();
    unsigned buf = 0u;
    for (; c < end; c += GF_CHUNK, buf ^= 1u) {
        // ---- the chunk's table; the next chunk's letters start their way
        uint4* hc = hotw + buf * GF_TABLE;
        const unsigned after = (unsigned)__shfl_down((int)letters, 1, 64);   // the next lane's four letters
        uint2 t[5];
#pragma unroll
        for (int k2 = 0; k2 < 4; ++k2) t[k2] = onehot[(letters >> (8 * k2)) & 0xffu];
        t[4] = onehot[after & 0xffu];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k2 = 0; k2 < 4; ++k2) hc[4u * lane + k2] = make_uint4(t[k2].x, t[k2].y, t[k2 + 1].x, t[k2 + 1].y);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (c + GF_CHUNK < end) letters = load_letters4(X, nbytes, c + GF_CHUNK + 4u * lane);
        const size_t cend = c + GF_CHUNK < end ? c + GF_CHUNK : end;
        for (size_t c0 = c; c0 < cend; c0 += 32) {
            const uint4* hot = hc + (c0 - c) + col + 2u * g;
            f32x16_t acc;
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const uint4 A = hot[4 * s];
#pragma unroll
                for (int q = 0; q < 3; ++q) acc = mfma_bf16(A, B[s][q], acc);
            }
            if (f < F) {
                float* out = Z + (c0 + 4u * g) * F + f;
                if (c0 + 32 <= cend) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) out[(size_t)((i & 3) + 8 * (i >> 2)) * F] = acc[i];
                } else {
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        if (c0 + 4u * g + (i & 3) + 8 * (i >> 2) < cend) out[(size_t)((i & 3) + 8 * (i >> 2)) * F] = acc[i];
                }
            }
        }
    }
}

// Bulk sizes only (the results differ from the lookup kernels' in the last bits).
inline bool fprop_mfma_takes(size_t m, size_t F, size_t n) { return m <= 32 && F >= 32 && n * F >= ((size_t)1 << 25); }

inline int launch_fprop_mfma(hipStream_t st, const float* W, size_t m, size_t F, const uint8_t* X, size_t n, float* Z)
{
    const unsigned fgroups = dbk::divup(F, 128);
    const size_t nchunk = dbk::divup(n, GF_CHUNK);
    size_t gy = 768 / fgroups;                                     // three workgroups per CU's worth
    if (gy < 1) gy = 1;
    if (gy > nchunk) gy = nchunk;
    const unsigned per = (unsigned)dbk::divup(nchunk, gy);
    gy = dbk::divup(nchunk, per);
    const size_t smem = 256 * 8 + 4 * 2 * GF_TABLE * 16;
    const unsigned ks = (unsigned)((4 * m + 15) / 16);
    auto kern = ks <= 2 ? corr1ord_mfma_kernel<2> : ks <= 4 ? corr1ord_mfma_kernel<4> : ks <= 6 ? corr1ord_mfma_kernel<6> : corr1ord_mfma_kernel<8>;
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(fgroups, (unsigned)gy), dim3(256), smem, st, W, (unsigned)m, (unsigned)F, X, n, Z, per);
    DBK_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------
// filter gradient on the matrix cores (float32, filters of up to 32 taps, bulk sizes)
// ---------------------------------------------------------------------------------------------
// dW (4m x F) = H^T (4m x n) . dZ (n x F), H the one-hot windows: row 4j + k of H^T has a 1 at output row i where
// X[i + j] is letter k (1/4 in all four rows for code 255 and other non-letters, nothing for 254). 0, 1 and 1/4 are
// exact in bf16 and every dZ value enters as three bf16 pieces that add up to it exactly, so the products are exact
// and v_mfma_f32_32x32x16_bf16 accumulates them in float32: the sums of the kernels above in another order.
// A wave owns 32 filters and all 4m rows of dW (up to four 32 x 32 accumulators) over its workgroup's share of the
// rows; the four waves of a workgroup take four neighbouring blocks of 32 filters. Per round of 64 rows the wave
// turns the letters into one bit per (letter, position) with ballots; a lane (row 4j + k of a 32-row block, half
// g) shifts its letter's bits by (j mod 8) + 8g once, after which the eight bits of a k-step are a whole byte of
// the shifted word, and a 256-entry table in LDS turns the byte into the eight bf16 of the operand.
// Deterministic: a fixed order per wave, one partial result per workgroup, the fixed-shape reduction above.
constexpr unsigned GW_ROUND = 64;                                  // rows per round: four k-steps of 16

template <int MB>
__global__ __launch_bounds__(256) void corr1ord_bprop_W_mfma_kernel(float* __restrict__ partial, unsigned m, unsigned F,
                                                                    const uint8_t* __restrict__ X, size_t n,
                                                                    const float* __restrict__ dZ, unsigned rounds_per_wg)
{
    using namespace dbk_mfma;
    __shared__ uint4 ones[256];                                    // byte -> eight bf16: 1.0 where the bit is set
    const unsigned lane = threadIdx.x & 63, wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned col = lane & 31, g = lane >> 5;
    {
        const unsigned v = threadIdx.x;
        unsigned d[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) d[q] = ((v >> (2 * q)) & 1u ? 0x3f80u : 0u) | ((v >> (2 * q + 1)) & 1u ? 0x3f800000u : 0u);
        ones[v] = make_uint4(d[0], d[1], d[2], d[3]);
    }
    const unsigned f = (blockIdx.x * 4 + wave) * 32 + col;
    const bool fok = f < F;
    const size_t nbytes = n + m - 1, nround = (n + GW_ROUND - 1) / GW_ROUND, nfull = n / GW_ROUND;
    size_t rd = (size_t)blockIdx.y * rounds_per_wg;               // round in work
    const size_t rd_end = rd + rounds_per_wg < nround ? rd + rounds_per_wg : nround;
    const unsigned k = col & 3u, sh = (col >> 2) + 8u * g;         // this lane's letter; its bit offset within a byte step
    f32x16_t acc[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[b][i] = 0.0f;
    // a round's operands as loaded: dZ rows 16 ks + 8g + t of this lane's filter (a column past F reads the last one,
    // and is not written), and two letters per lane (positions lane and 64 + lane of the round; past the end: "nothing")
    const float* src = dZ + (rd * GW_ROUND + 8u * g) * F + (fok ? f : F - 1);
    const size_t hop = (size_t)GW_ROUND * F;
    struct round_in { float d[4][8]; unsigned x0, x1; };
#define DBK_LOAD_ROUND(IN, RD)                                                                            \
    {                                                                                                     \
        const size_t g0 = (RD) * GW_ROUND + lane, g1 = g0 + 64;                                           \
        IN.x0 = X[g0 < nbytes ? g0 : nbytes - 1];                                                         \
        IN.x1 = X[g1 < nbytes ? g1 : nbytes - 1];                                                         \
        IN.x0 = g0 < nbytes ? IN.x0 : 254u;                                                               \
        IN.x1 = g1 < nbytes ? IN.x1 : 254u;                                                               \
        _Pragma("unroll") for (int ks = 0; ks < 4; ++ks)                                                  \
            _Pragma("unroll") for (int t = 0; t < 8; ++t) IN.d[ks][t] = src[(size_t)(16 * ks + t) * F];   \
        src += hop;                                                                                       \
    }
    // The products of a round. One bit per position: this lane's letter, and "any letter" (weight 1/4, the products add).
#define DBK_ROUND(IN)                                                                                     \
    {                                                                                                     \
        const unsigned v0 = letter_of(IN.x0), v1 = letter_of(IN.x1);                                      \
        unsigned long long L0[4], L1[4];                                                                  \
        _Pragma("unroll") for (int l = 0; l < 4; ++l) { L0[l] = __ballot(v0 == (unsigned)l); L1[l] = __ballot(v1 == (unsigned)l); } \
        const unsigned long long N0 = __ballot(v0 == 4u), N1 = __ballot(v1 == 4u);                        \
        const unsigned long long m0 = k == 0u ? L0[0] : k == 1u ? L0[1] : k == 2u ? L0[2] : L0[3];        \
        const unsigned long long m1 = k == 0u ? L1[0] : k == 1u ? L1[1] : k == 2u ? L1[2] : L1[3];        \
        const unsigned w0 = (unsigned)m0, w1 = (unsigned)(m0 >> 32), w2 = (unsigned)m1, w3 = (unsigned)(m1 >> 32); \
        const unsigned V[3] = { __builtin_amdgcn_alignbit(w1, w0, sh), __builtin_amdgcn_alignbit(w2, w1, sh), __builtin_amdgcn_alignbit(w3, w2, sh) }; \
        const bool any_n = (N0 | N1) != 0ull;                                                             \
        const unsigned q0 = (unsigned)N0, q1 = (unsigned)(N0 >> 32), q2 = (unsigned)N1, q3 = (unsigned)(N1 >> 32); \
        const unsigned VN[3] = { __builtin_amdgcn_alignbit(q1, q0, sh), __builtin_amdgcn_alignbit(q2, q1, sh), __builtin_amdgcn_alignbit(q3, q2, sh) }; \
        _Pragma("unroll") for (int ks = 0; ks < 4; ++ks) {                                                \
            unsigned pc[3][8];                                                                            \
            _Pragma("unroll") for (int t = 0; t < 8; ++t) split3(IN.d[ks][t], pc[0][t], pc[1][t], pc[2][t]); \
            uint4 B[3];                                                                                   \
            _Pragma("unroll") for (int q = 0; q < 3; ++q)                                                 \
                B[q] = make_uint4(pack_upper_halves(pc[q][0], pc[q][1]), pack_upper_halves(pc[q][2], pc[q][3]), \
                                  pack_upper_halves(pc[q][4], pc[q][5]), pack_upper_halves(pc[q][6], pc[q][7])); \
            /* taps 8b .. 8b + 7: byte 2 ks + b of the shifted bits holds rows 16 ks + 8g .. + 7 at this lane's tap */ \
            _Pragma("unroll") for (int b = 0; b < MB; ++b) {                                              \
                const uint4 A = ones[(V[(2 * ks + b) >> 2] >> (8 * ((2 * ks + b) & 3))) & 0xffu];         \
                _Pragma("unroll") for (int q = 0; q < 3; ++q) acc[b] = mfma_bf16(A, B[q], acc[b]);        \
            }                                                                                             \
            if (any_n) {                                                                                  \
                _Pragma("unroll") for (int b = 0; b < MB; ++b) {                                          \
                    const unsigned bits = (VN[(2 * ks + b) >> 2] >> (8 * ((2 * ks + b) & 3))) & 0xffu;    \
                    if (__ballot(bits != 0u) != 0ull) {           /* some lane of the wave has one in these rows and taps */ \
                        uint4 A = ones[bits];                                                             \
                        A.x &= 0x3e803e80u; A.y &= 0x3e803e80u; A.z &= 0x3e803e80u; A.w &= 0x3e803e80u;   \
                        _Pragma("unroll") for (int q = 0; q < 3; ++q) acc[b] = mfma_bf16(A, B[q], acc[b]); \
                    }                                                                                     \
                }                                                                                         \
            }                                                                                             \
        }                                                                                                 \
    }
    // whole rounds, two per turn: the one being multiplied and the one on its way change places without copies
    const bool owns_last = rd_end == nround && nfull < nround && rd <= nfull;   // the partial round at the end is this workgroup's
    const size_t full_end = rd_end < nfull ? rd_end : nfull;
    round_in ra, rb;
    if (rd < full_end) DBK_LOAD_ROUND(ra, rd)
    __syncthreads();
    while (rd < full_end) {
        if (rd + 1 < full_end) DBK_LOAD_ROUND(rb, rd + 1)
        DBK_ROUND(ra)
        if (++rd >= full_end) break;
        if (rd + 1 < full_end) DBK_LOAD_ROUND(ra, rd + 1)
        DBK_ROUND(rb)
        ++rd;
    }
    if (owns_last) {
        // the last, partial round: a row past the end reads the last row and counts as zero
        const size_t base = nfull * GW_ROUND, left = n - base;
        const size_t g0 = base + lane, g1 = g0 + 64;
        ra.x0 = X[g0 < nbytes ? g0 : nbytes - 1];
        ra.x1 = X[g1 < nbytes ? g1 : nbytes - 1];
        ra.x0 = g0 < nbytes ? ra.x0 : 254u;
        ra.x1 = g1 < nbytes ? ra.x1 : 254u;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const size_t rel = 16u * ks + 8u * g + t;
                const float v = dZ[(base + (rel < left ? rel : left - 1)) * F + (fok ? f : F - 1)];
                ra.d[ks][t] = rel < left ? v : 0.0f;
            }
        DBK_ROUND(ra)
    }
#undef DBK_LOAD_ROUND
#undef DBK_ROUND
    // ---- the workgroup's partial result: rows 32b + (i & 3) + 8 (i >> 2) + 4g of this lane's filter
    float* out = partial + (size_t)blockIdx.y * 4 * m * F;
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const unsigned row = 32u * b + (i & 3) + 8 * (i >> 2) + 4u * g;
            if (row < 4u * m && fok) out[(size_t)row * F + f] = acc[b][i];
        }
}

template <int MB>
void launch_bprop_W_mfma_mb(hipStream_t st, float* partial, unsigned gy, unsigned rounds, size_t m, size_t F, const uint8_t* X, size_t n, const float* dZ)
{
    hipLaunchKernelGGL(corr1ord_bprop_W_mfma_kernel<MB>, dim3(dbk::divup(F, 128), gy), dim3(256), 0, st, partial, (unsigned)m, (unsigned)F, X, n, dZ, rounds);
}

// Bulk sizes only: below, the partial results (one 4m x F block per workgroup) cost more than the rows.
inline bool bprop_W_mfma_takes(size_t m, size_t F, size_t n) { return m <= 32 && F >= 32 && n * F >= ((size_t)1 << 22) && n >= 4096; }

inline int launch_bprop_W_mfma(hipStream_t st, float* dW, size_t m, size_t F, const uint8_t* X, size_t n, const float* dZ)
{
    const unsigned fgroups = dbk::divup(F, 128);
    const size_t nround = dbk::divup(n, GW_ROUND);
    size_t gy = 512 / fgroups;                                     // two workgroups per CU's worth (more only adds partial results)
    if (gy < 1) gy = 1;
    if (gy > nround / 4) gy = nround / 4 ? nround / 4 : 1;         // at least four rounds per workgroup
    const unsigned rounds = (unsigned)dbk::divup(nround, gy);
    gy = dbk::divup(nround, rounds);
    const size_t nelem = 4 * m * F;
    float* partial = (float*)dbk::workspace(nelem * gy * sizeof(float), st);
    DBK_CHECK(partial != nullptr, "MemoryError: could not allocate %zu bytes of scratch (%s)", nelem * gy * sizeof(float), dbk::workspace_error());
    switch ((4 * m + 31) / 32) {
    case 1:  launch_bprop_W_mfma_mb<1>(st, partial, (unsigned)gy, rounds, m, F, X, n, dZ); break;
    case 2:  launch_bprop_W_mfma_mb<2>(st, partial, (unsigned)gy, rounds, m, F, X, n, dZ); break;
    case 3:  launch_bprop_W_mfma_mb<3>(st, partial, (unsigned)gy, rounds, m, F, X, n, dZ); break;
    default: launch_bprop_W_mfma_mb<4>(st, partial, (unsigned)gy, rounds, m, F, X, n, dZ); break;
    }
    hipLaunchKernelGGL(reduce_partials_quarters_kernel, dim3((unsigned)dbk::divup(nelem, 64)), dim3(256), 0, st, dW, (const float*)partial, nelem, (unsigned)gy);
    DBK_LAUNCH_OK();
}

// float32 filters of at most 24 taps: register-resident gradient columns
inline int launch_bprop_W_window(hipStream_t st, float* dW, size_t m, size_t F, const uint8_t* X, size_t n, const float* dZ)
{
    const unsigned mt = m <= 8 ? 8 : (m <= 16 ? 16 : 24);
    const unsigned ftiles = dbk::divup(F, FT), chunk = 4 * WSUBS_W * PSUB;
    const unsigned nchunk = dbk::divup(n, chunk);
    unsigned gy = (mt == 8 ? 768u : 512u) / ftiles;           // three workgroups fit a CU with 8 taps' register planes, else two
    if (gy < 1) gy = 1;
    if (gy > nchunk) gy = nchunk;
    const size_t nelem = 4 * m * F;
    float* partial = (float*)dbk::workspace(nelem * gy * sizeof(float), st);
    DBK_CHECK(partial != nullptr, "MemoryError: could not allocate %zu bytes of scratch (%s)", nelem * gy * sizeof(float), dbk::workspace_error());
    const size_t smem = (size_t)mt * 4 * FT * sizeof(float) + ((chunk + mt - 1 + 7) & ~(size_t)3);
    auto kern = mt == 8 ? corr1ord_bprop_W_window_kernel<8> : mt == 16 ? corr1ord_bprop_W_window_kernel<16> : corr1ord_bprop_W_window_kernel<24>;
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(ftiles, gy), dim3(256), smem, st, partial, (unsigned)m, (unsigned)F, X, n, dZ);
    hipLaunchKernelGGL(reduce_partials_kernel<float>, dim3(dbk::ew_grid(nelem)), dim3(256), 0, st, dW, (const float*)partial, nelem, gy);
    DBK_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------------
// input gradient on the matrix cores (float32, filters of up to 32 taps, bulk sizes)
// ---------------------------------------------------------------------------------------------
// Y (rows x 4m) = dZ (rows x F) . W^T (F x 4m), then dX[i, c] += sum_k Y[i - k, 4k + c]. Both operands are float32
// data, so both enter as three bf16 pieces and six of the nine piece products are formed (hi.hi, hi.mid, mid.hi,
// mid.mid, hi.lo, lo.hi; the three left out are below 2^-24 of the result), accumulated in float32.
// A workgroup takes 512 to 1024 output rows and 128 filters (the launcher issues one launch per 128 filters: dX accumulates),
// wave b of it the taps 8b .. 8b + 7 (32 columns of Y; W's pieces for them stay in registers, 96 registers). A
// block of 32 rows of dZ is read by the whole workgroup as whole 512-byte row segments and staged in LDS (a lane
// reading its own row from memory touches 32 cache lines per instruction, and the tag rate of the CU's cache then sets
// the pace). The rows are requested a whole block ahead - right after the registers that carry them have been emptied
// into LDS, between the two barriers of the block before - and nothing else goes to or comes from global memory inside
// the loop (the workgroup's rows of the result collect in LDS and join dX in one pass at the end), so the wait for them
// waits for nothing else. Every wave reads the same staged pieces (every value is split once, by the thread that loaded
// it: the planes hold bf16), the 32 x 4m tile of Y goes to LDS, and 128 threads add up the taps of their (row, letter)
// in ascending order, reaching into the previous block's tile for rows before the block (the first block of a
// workgroup recomputes its predecessor's last rows instead of sharing them). Deterministic: one writer per element,
// fixed orders.
constexpr unsigned GX_ROWS = 512;                                  // output rows per workgroup, at least (a multiple of 32)
constexpr unsigned GX_WGROWS = 1024;                               // ... and at most: they are held in LDS until the workgroup ends
constexpr unsigned GX_FILTERS = 128;                               // filters per launch: eight k-steps of 16
constexpr unsigned GX_ZS = GX_FILTERS + 8;                         // row stride of a staged plane in bf16: 68 words = 4 mod 32, so that the 32 rows' 16-byte reads spread over the banks

template <int MB, bool WHOLE>
__global__ __launch_bounds__(64 * MB) void corr1ord_bprop_X_mfma_kernel(float* __restrict__ dX, size_t n, const float* __restrict__ W,
                                                                        unsigned m, unsigned F, unsigned f0, const float* __restrict__ dZ, unsigned rows_per_wg)
{
    using namespace dbk_mfma;
    constexpr int YS = 32 * MB + 4;                                // row stride of a tile of Y: 4 mod 32, so that the adders' reads spread over the banks
    constexpr int NT = 64 * MB, PER = (32 * (GX_FILTERS / 4) + NT - 1) / NT;   // threads; 16-byte pieces of a dZ tile per thread
    __shared__ float Y[2][32][YS];
    __shared__ __align__(16) unsigned short Zt[3][32][GX_ZS];     // the block's rows of dZ (this launch's filters) as three planes of bf16 pieces (lo, mid, hi)
    __shared__ float out[GX_WGROWS * 4];                          // the workgroup's rows of the result
    const unsigned lane = threadIdx.x & 63, nb = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned col = lane & 31, g = lane >> 5;
    // ---- W's rows 32 nb + col (tap 8 nb + col / 4, letter col % 4), filters f0 + 16 ks + 8g .. + 7, in three pieces
    uint4 B[8][3];
    {
        const unsigned wrow = 32u * nb + col;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            unsigned pc[3][8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const unsigned f = f0 + 16u * ks + 8u * g + t;
                const float w = (wrow < 4u * m && f < F) ? W[(size_t)wrow * F + f] : 0.0f;
                split3(w, pc[0][t], pc[1][t], pc[2][t]);
            }
#pragma unroll
            for (int q = 0; q < 3; ++q)
                B[ks][q] = make_uint4(pack_upper_halves(pc[q][0], pc[q][1]), pack_upper_halves(pc[q][2], pc[q][3]),
                                      pack_upper_halves(pc[q][4], pc[q][5]), pack_upper_halves(pc[q][6], pc[q][7]));
        }
    }
    const size_t o0 = (size_t)blockIdx.x * rows_per_wg, o1 = o0 + rows_per_wg < n ? o0 + rows_per_wg : n;
    // A block's rows of dZ, requested by the whole workgroup as 16-byte pieces in row order (a wave reads whole
    // 512-byte row segments). Every thread loads every time (a row past the end reads the last row, a piece past the
    // block the block's last piece; what must count as zero is zeroed when it is used): nothing but these loads is
    // on its way to or from global memory inside the loop, the same number on every path, so that waiting for the
    // older of two blocks' rows does not wait for the newer.
    auto request = [&](size_t i0_, float4 (&piece)[PER]) {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            unsigned e = threadIdx.x + j * NT;
            if (e >= 32u * (GX_FILTERS / 4)) e = 32u * (GX_FILTERS / 4) - 1u;
            const unsigned r = e / (GX_FILTERS / 4), c4 = e % (GX_FILTERS / 4);
            size_t row = i0_ + r;
            if (row >= n) row = n - 1;
            const float* src = dZ + row * F + f0 + 4u * c4;
            float4 p;
            if (WHOLE) {
                p = *reinterpret_cast<const float4*>(src);
            } else {
                const unsigned f = f0 + 4u * c4;
                p.x = src[f < F ? 0 : -(int)(f - (F - 1))]; p.y = src[f + 1 < F ? 1 : -(int)(f - (F - 1))];
                p.z = src[f + 2 < F ? 2 : -(int)(f - (F - 1))]; p.w = src[f + 3 < F ? 3 : -(int)(f - (F - 1))];
            }
            piece[j] = p;
        }
    };
    // every value is split once, by the thread that loaded it: four values' pieces are 8 bytes per plane
    auto deposit = [&](size_t i0_, const float4 (&piece)[PER]) {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const unsigned e = threadIdx.x + j * NT, r = e / (GX_FILTERS / 4), c4 = e % (GX_FILTERS / 4);
            if (e < 32 * (GX_FILTERS / 4)) {
                const bool row_in = i0_ + r < n;
                float v[4] = { piece[j].x, piece[j].y, piece[j].z, piece[j].w };
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (!row_in || (!WHOLE && f0 + 4u * c4 + t >= F)) v[t] = 0.0f;
                unsigned pc[3][4];
#pragma unroll
                for (int t = 0; t < 4; ++t) split3(v[t], pc[0][t], pc[1][t], pc[2][t]);
#pragma unroll
                for (int q = 0; q < 3; ++q)
                    *reinterpret_cast<uint2*>(&Zt[q][r][4 * c4]) = make_uint2(pack_upper_halves(pc[q][0], pc[q][1]), pack_upper_halves(pc[q][2], pc[q][3]));
            }
        }
    };
    // One block: this block's tile of Y from the staged pieces; between the two barriers the next block's rows (on
    // their way since the middle of the block before) go to LDS, the rows of the block after it are requested into the
    // same registers, and this block's taps are added up into the workgroup's rows of the result in LDS.
    unsigned slot = 0u;
    float4 piece[PER];
    auto block = [&](size_t i0) {
        f32x16_t acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
        // this lane supplies row i0 + col: its eight values of a k-step are 16 bytes of each plane
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            uint4 A[3];
#pragma unroll
            for (int q = 0; q < 3; ++q) A[q] = *reinterpret_cast<const uint4*>(&Zt[q][col][16 * ks + 8 * g]);
            // pieces: 0 = lo, 1 = mid, 2 = hi; the small products first
            acc = mfma_bf16(A[0], B[ks][2], acc);
            acc = mfma_bf16(A[2], B[ks][0], acc);
            acc = mfma_bf16(A[1], B[ks][1], acc);
            acc = mfma_bf16(A[1], B[ks][2], acc);
            acc = mfma_bf16(A[2], B[ks][1], acc);
            acc = mfma_bf16(A[2], B[ks][2], acc);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) Y[slot][(i & 3) + 8 * (i >> 2) + 4 * g][32 * nb + col] = acc[i];
        __syncthreads();                                           // the tile is complete; nobody reads the staged pieces any more
        if (i0 + 32 < o1) deposit(i0 + 32, piece);
        request(i0 + 64, piece);
        if (i0 >= o0) {
            // ---- rows i0 .. i0 + 31 of the result: taps in ascending order, rows before the block from the previous tile
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const unsigned t = threadIdx.x + h * NT;
                if (!(t < 128 && (h == 0 || NT < 128))) continue;
                const unsigned r = t >> 2, c = t & 3u;
                const size_t i = i0 + r;
                if (i < o1) {
                    float y[8 * MB];
#pragma unroll
                    for (int k = 0; k < 8 * MB; ++k) {
                        const unsigned kk = (unsigned)k < m ? (unsigned)k : 0u;
                        const float* tile = kk <= r ? &Y[slot][r - kk][0] : &Y[slot ^ 1u][32 + r - kk][0];
                        y[k] = tile[4 * kk + c];
                    }
                    float sum = 0.0f;
#pragma unroll
                    for (int k = 0; k < 8 * MB; ++k) sum += ((unsigned)k < m && i >= (size_t)k) ? y[k] : 0.0f;
                    out[(i - o0) * 4 + c] = sum;
                }
            }
        }
        __syncthreads();                                           // the next block's pieces are staged; this tile's readers are done
        slot ^= 1u;
    };
    size_t i0 = o0 >= 32 ? o0 - 32 : 0;
    request(i0, piece);
    deposit(i0, piece);
    request(i0 + 32, piece);
    __syncthreads();
    for (; i0 < o1; i0 += 32) block(i0);
    // ---- the workgroup's rows of the result join what is there (the launches of other filters): one coalesced pass
    const size_t nout = (o1 - o0) * 4;
    for (size_t e = threadIdx.x; e < nout; e += NT) dX[o0 * 4 + e] += out[e];
}

inline bool bprop_X_mfma_takes(size_t m, size_t F, size_t n) { return m <= 32 && F >= 64 && n * F >= ((size_t)1 << 22) && n >= 4096; }

inline int launch_bprop_X_mfma(hipStream_t st, float* dX, size_t n, const float* W, size_t m, size_t F, const float* dZ)
{
    // two workgroups fit a CU: about 512 of them in all, so that the weights' pieces are formed once per many rows
    // (512 rows per workgroup: 0.61 ms at 1.0 M rows x 256 filters; 1/512 of the rows: 0.54 ms; at most 1024, the result
    // rows in LDS and the rows of dZ requested a block ahead: 0.51 ms)
    unsigned rows = (unsigned)(((n + 511) / 512 + 31) / 32 * 32);
    if (rows < GX_ROWS) rows = GX_ROWS;
    if (rows > GX_WGROWS) rows = GX_WGROWS;
    const unsigned gx = (unsigned)dbk::divup(n, rows), mb = (unsigned)((4 * m + 31) / 32);
    for (size_t f0 = 0; f0 < F; f0 += GX_FILTERS) {
        const bool whole = F % 4 == 0 && f0 + GX_FILTERS <= F;
#define DBK_GO(MB_)                                                                                                   \
        if (whole) hipLaunchKernelGGL((corr1ord_bprop_X_mfma_kernel<MB_, true>), dim3(gx), dim3(64 * MB_), 0, st, dX, n, W, (unsigned)m, (unsigned)F, (unsigned)f0, dZ, rows); \
        else hipLaunchKernelGGL((corr1ord_bprop_X_mfma_kernel<MB_, false>), dim3(gx), dim3(64 * MB_), 0, st, dX, n, W, (unsigned)m, (unsigned)F, (unsigned)f0, dZ, rows);
        switch (mb) {
        case 1:  DBK_GO(1) break;
        case 2:  DBK_GO(2) break;
        case 3:  DBK_GO(3) break;
        default: DBK_GO(4) break;
        }
#undef DBK_GO
    }
    DBK_LAUNCH_OK();
}

inline int launch_bprop_X_ring(hipStream_t st, float* dX, size_t n, const float* W, size_t m, size_t F, const float* dZ)
{
    if (m <= 8) {
        hipLaunchKernelGGL((corr1ord_bprop_X_ring_kernel<8, 96>), dim3(dbk::divup(n, 4 * 96)), dim3(256), 0, st, dX, n, W, (unsigned)m, (unsigned)F, dZ);
    } else if (m <= 16) {
        hipLaunchKernelGGL((corr1ord_bprop_X_ring_kernel<16, 96>), dim3(dbk::divup(n, 4 * 96)), dim3(256), 0, st, dX, n, W, (unsigned)m, (unsigned)F, dZ);
    } else {
        hipLaunchKernelGGL((corr1ord_bprop_X_ring_kernel<24, 96>), dim3(dbk::divup(n, 4 * 96)), dim3(256), 0, st, dX, n, W, (unsigned)m, (unsigned)F, dZ);
    }
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
    DBK_CHECK(partial != nullptr, "MemoryError: could not allocate %zu bytes of scratch (%s)", nelem * gy * sizeof(T), dbk::workspace_error());
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
    if (dtype == DBK_F32 && !dbk::exact_scan() && fprop_mfma_takes(m, nfilter, n)) return launch_fprop_mfma(dbk::as_stream(stream), (const float*)W, m, nfilter, X, n, (float*)Z);
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
    if (dtype == DBK_F32 && !dbk::exact_scan() && bprop_W_mfma_takes(m, nfilter, n)) return launch_bprop_W_mfma(dbk::as_stream(stream), (float*)dW, m, nfilter, X, n, (const float*)dZ);
    if (dtype == DBK_F32 && m <= 24) return launch_bprop_W_window(dbk::as_stream(stream), (float*)dW, m, nfilter, X, n, (const float*)dZ);
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
    if (dtype == DBK_F32 && !dbk::exact_scan() && bprop_X_mfma_takes(m, nfilter, n)) return launch_bprop_X_mfma(dbk::as_stream(stream), (float*)dX, n, (const float*)W, m, nfilter, (const float*)dZ);
    if (dtype == DBK_F32 && m <= 24) return launch_bprop_X_ring(dbk::as_stream(stream), (float*)dX, n, (const float*)W, m, nfilter, (const float*)dZ);
    if (dtype == DBK_F32) return launch_bprop_X<float>(dbk::as_stream(stream), (float*)dX, n, (const float*)W, m, nfilter, (const float*)dZ);
    return launch_bprop_X<double>(dbk::as_stream(stream), (double*)dX, n, (const double*)W, m, nfilter, (const double*)dZ);
}

}  // extern "C"

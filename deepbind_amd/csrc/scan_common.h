// Pieces shared by the scan kernels: the 6-letter alphabet and the [tap][letter][filter] LDS table.
#pragma once
#include "dbk_common.h"
#include <utility>

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
// QUAD: a row holds filter fl at element (fl % 16) * 4 + fl / 16, i.e. 16 lanes x 4 filters (16 apart) per lane.
template <typename T, bool QUAD = false>
__device__ void build_letter_table(T* lut, const T* __restrict__ W, unsigned m, unsigned F, unsigned f0, unsigned mpad = 0)
{
    if (mpad < m) mpad = m;
    // two taps per thread and round, so that eight loads are in flight together (a plain strided loop waits
    // for each round's loads before it issues the next)
    for (unsigned e0 = threadIdx.x; e0 < mpad * FT; e0 += 2 * blockDim.x) {
        T w[2][4];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const unsigned e = e0 + u * blockDim.x, j = e / FT, f = f0 + e % FT;
            const bool in = e < mpad * FT && f < F && j < m;
#pragma unroll
            for (int c = 0; c < 4; ++c) w[u][c] = in ? W[(4 * j + c) * (size_t)F + f] : (T)0;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const unsigned e = e0 + u * blockDim.x, j = e / FT, fl = e % FT;
            if (e >= mpad * FT) break;
            T z = w[u][0];
            z += w[u][1];
            z += w[u][2];
            z += w[u][3];
            T* row = lut + (size_t)j * NL * FT + (QUAD ? (fl & 15u) * 4u + (fl >> 4) : fl);
            row[0 * FT] = w[u][0];
            row[1 * FT] = w[u][1];
            row[2 * FT] = w[u][2];
            row[3 * FT] = w[u][3];
            row[4 * FT] = z * (T)0.25;
            row[5 * FT] = (T)0;
        }
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

// ---- four filters per lane ---------------------------------------------------------------------------
// A lane owns four filters and a table row holds [16 lanes][4 filters], so the 16 lanes of a quarter wave read one
// aligned 256-byte line per ds_read_b128 (about twice the bytes per clock of 4-byte reads); the four quarters of a
// wave work on four consecutive windows of PSUB positions. The letters of a quarter's window sit in vector
// registers (they differ between the quarters).
template <int MT> struct wide_shape {
    static constexpr unsigned words = (PSUB + MT - 1 + 3) / 4;               // window words per quarter
    static constexpr unsigned xbytes = (3 * PSUB + 4 * words + 15) & ~15u;   // letters a wave stages per round of 4 x PSUB positions
    static_assert(xbytes <= 128, "a lane stages at most two letters per round");
};

// Letters of positions c0 .. c0 + xbytes - 1 into the wave's own LDS bytes (two per lane; past the end of X:
// "nothing"), then this quarter's window words. A wave's LDS accesses execute in program order, so only the
// compiler has to be kept from reordering them.
template <int MT>
__device__ __forceinline__ void wide_stage(uint8_t* xw, const uint8_t* __restrict__ X, size_t N, size_t c0, unsigned lane,
                                           unsigned (&wq)[wide_shape<MT>::words])
{
    constexpr unsigned XB = wide_shape<MT>::xbytes;
    const size_t g0 = c0 + lane, g1 = g0 + 64;
    const unsigned v0 = g0 < N ? letter_of(X[g0]) : 5u;
    const unsigned v1 = (lane + 64 < XB && g1 < N) ? letter_of(X[g1]) : 5u;
    __builtin_amdgcn_wave_barrier();                               // the previous round's window reads come first
    xw[lane] = (uint8_t)v0;
    if (lane + 64 < XB) xw[lane + 64] = (uint8_t)v1;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const unsigned* src = reinterpret_cast<const unsigned*>(xw + PSUB * (lane >> 4));
#pragma unroll
    for (unsigned t = 0; t < wide_shape<MT>::words; ++t) wq[t] = src[t];
}

// acc[p] = sum over taps j < MT of the table row (j, letter at window position p + j), four filters at a time,
// taps in ascending order per position. lut4: the table as float4, already offset by this lane's place in a row.
// One bit-field extract and one address add per letter serve up to PSUB reads with immediate offsets.
template <int MT>
__device__ __forceinline__ void scan16_wide(const float4* __restrict__ lut4, const unsigned (&wq)[wide_shape<MT>::words], float4 (&acc)[PSUB])
{
#pragma unroll
    for (int p = 0; p < PSUB; ++p) acc[p] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
    for (int q = 0; q < PSUB + MT - 1; ++q) {
        const unsigned letter = (wq[q >> 2] >> ((q & 3) * 8)) & 0xffu;
        const float4* col = lut4 + letter * 16u;
#pragma unroll
        for (int p = 0; p < PSUB; ++p) {
            const int j = q - p;
            if (j >= 0 && j < MT) {
                const float4 v = col[j * NL * 16];
                acc[p].x += v.x; acc[p].y += v.y; acc[p].z += v.z; acc[p].w += v.w;
            }
        }
        if ((q & 3) == 3) {
            // pin the running sums (see scan16_window)
#pragma unroll
            for (int p = 0; p < PSUB; ++p) asm volatile("" : "+v"(acc[p].x), "+v"(acc[p].y), "+v"(acc[p].z), "+v"(acc[p].w));
        }
    }
}

// ---- filter-gradient accumulation through the VGPR index mode -------------------------------------
// dW[tap j][letter c][filter] += g[position p] for every (p, j) of a window whose letter at p + j is c.
// The letter is the same for all lanes (a scalar), the filter is the lane. Spelled with ordinary
// arithmetic this takes four multiply-adds per (p, j) (letter weights 1 / 0 / 1/4 per channel); with
// the accumulators laid out as six planes of MT consecutive registers - plane = letter: A, C, G, T,
// "mean of the four", "nothing" - and the hardware's register index mode (s_set_gpr_idx_on: M0[7:0]
// is added to the register number of src0 and dst), it is ONE v_add_f32 per (p, j) plus one scalar
// instruction per letter. The planes live in fixed registers v96.. so that the instruction text can
// name them; the compiler keeps everything else below. Plane 4 is spread over the four channels
// (x 1/4) and plane 5 is dropped when the planes are read out.
typedef float v32f __attribute__((ext_vector_type(32)));
typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int GRAD_PLANES = 6;

template <int MT> struct grad_planes {
    static_assert(MT == 8 || MT == 16 || MT == 24, "plane sets exist for 8, 16 and 24 taps");
    v32f t0, t1, t2, t3;            // v[96:127], v[128:159], v[160:191], v[192:223]   (as many as 6*MT needs)
    v16f u0;                        // MT = 8: v[128:143], MT = 24: v[224:239]
    __device__ __forceinline__ void clear()
    {
#pragma unroll
        for (int i = 0; i < 32; ++i) t0[i] = t1[i] = t2[i] = t3[i] = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) u0[i] = 0.0f;
    }
    // register e of the plane set (plane * MT + tap)
    template <int E> __device__ __forceinline__ float reg() const
    {
        static_assert(E >= 0 && E < GRAD_PLANES * MT, "register outside the plane set");
        if constexpr (MT == 8) return E < 32 ? t0[E % 32] : u0[(E - 32) % 16];
        else if constexpr (E < 32) return t0[E % 32];
        else if constexpr (E < 64) return t1[E % 32];
        else if constexpr (E < 96) return t2[E % 32];
        else if constexpr (E < 128) return t3[E % 32];
        else return u0[(E - 128) % 16];
    }
    template <int E> __device__ __forceinline__ void set(float v)
    {
        static_assert(E >= 0 && E < GRAD_PLANES * MT, "register outside the plane set");
        if constexpr (MT == 8) { if constexpr (E < 32) t0[E % 32] = v; else u0[(E - 32) % 16] = v; }
        else if constexpr (E < 32) t0[E % 32] = v;
        else if constexpr (E < 64) t1[E % 32] = v;
        else if constexpr (E < 96) t2[E % 32] = v;
        else if constexpr (E < 128) t3[E % 32] = v;
        else u0[(E - 128) % 16] = v;
    }
    // gradient of tap J, channel C: the letter's own plane plus a quarter of the "mean" plane
    template <int J, int C> __device__ __forceinline__ float grad() const { return reg<C * MT + J>() + 0.25f * reg<4 * MT + J>(); }
};

#define DBK_GP_LIST(...) __VA_ARGS__
#define DBK_GP_SLOT(P) ".if ((%c[q] - " #P ") >= 0) && ((%c[q] - " #P ") < %c[mt])\n\t" \
                       "v_add_f32 v[96 + %c[q] - " #P "], v[96 + %c[q] - " #P "], %[g" #P "]\n\t.endif\n\t"
#define DBK_GP_ASM(PLANES)                                                                                          \
    asm volatile("s_set_gpr_idx_on %[idx], 0x9\n\t"                                                                  \
                 DBK_GP_SLOT(0) DBK_GP_SLOT(1) DBK_GP_SLOT(2) DBK_GP_SLOT(3) DBK_GP_SLOT(4) DBK_GP_SLOT(5) DBK_GP_SLOT(6)   \
                 DBK_GP_SLOT(7) DBK_GP_SLOT(8) DBK_GP_SLOT(9) DBK_GP_SLOT(10) DBK_GP_SLOT(11) DBK_GP_SLOT(12)            \
                 DBK_GP_SLOT(13) DBK_GP_SLOT(14) DBK_GP_SLOT(15)                                                     \
                 "s_set_gpr_idx_off"                                                                                \
                 : PLANES                                                                                           \
                 : [idx] "s"(idx), [q] "n"(Q), [mt] "n"(MT), [g0] "v"(g[0]), [g1] "v"(g[1]), [g2] "v"(g[2]),        \
                   [g3] "v"(g[3]), [g4] "v"(g[4]), [g5] "v"(g[5]), [g6] "v"(g[6]), [g7] "v"(g[7]), [g8] "v"(g[8]),  \
                   [g9] "v"(g[9]), [g10] "v"(g[10]), [g11] "v"(g[11]), [g12] "v"(g[12]), [g13] "v"(g[13]),          \
                   [g14] "v"(g[14]), [g15] "v"(g[15])                                                               \
                 : "m0")

// All (p, j) pairs of the window that meet letter position Q: tap j = Q - p of position p.
template <int Q, int MT>
__device__ __forceinline__ void grad_planes_add(grad_planes<MT>& A, unsigned letter, const float (&g)[PSUB])
{
    static_assert(PSUB == 16, "the instruction text lists 16 positions");
    // M0 (which the index lives in while the mode is on) is left changed and declared as clobbered, so the
    // compiler re-establishes any value of its own in M0 after the block; saving and restoring it here would
    // cost more than the sixteen additions (measured: +48 %). The planes are pinned to v96..v239 because the
    // instruction text under the index mode names its registers relative to v96.
    const unsigned idx = letter * (unsigned)MT;          // first register of the letter's plane, relative to v96
    if constexpr (MT == 8) DBK_GP_ASM(DBK_GP_LIST("+{v[96:127]}"(A.t0), "+{v[128:143]}"(A.u0)));
    else if constexpr (MT == 16) DBK_GP_ASM(DBK_GP_LIST("+{v[96:127]}"(A.t0), "+{v[128:159]}"(A.t1), "+{v[160:191]}"(A.t2)));
    else DBK_GP_ASM(DBK_GP_LIST("+{v[96:127]}"(A.t0), "+{v[128:159]}"(A.t1), "+{v[160:191]}"(A.t2), "+{v[192:223]}"(A.t3), "+{v[224:239]}"(A.u0)));
}

template <int MT, int... Q>
__device__ __forceinline__ void grad_planes_window(grad_planes<MT>& A, const unsigned (&wq)[window<MT>::words], const float (&g)[PSUB],
                                                   std::integer_sequence<int, Q...>)
{
    (grad_planes_add<Q, MT>(A, window_letter(wq, Q), g), ...);
}
// Adds one sub-chunk (PSUB positions with gradients g, window letters wq) into the planes.
template <int MT>
__device__ __forceinline__ void grad_planes_window(grad_planes<MT>& A, const unsigned (&wq)[window<MT>::words], const float (&g)[PSUB])
{
    grad_planes_window<MT>(A, wq, g, std::make_integer_sequence<int, PSUB + MT - 1>{});
}

template <int MT, int... E>
__device__ __forceinline__ void grad_planes_read(const grad_planes<MT>& A, float (&aw)[MT][4], std::integer_sequence<int, E...>)
{
    ((aw[E / 4][E % 4] = A.template grad<E / 4, E % 4>()), ...);
}
// The finished [tap][channel] gradient column of this lane's filter.
template <int MT>
__device__ __forceinline__ void grad_planes_read(const grad_planes<MT>& A, float (&aw)[MT][4])
{
    grad_planes_read<MT>(A, aw, std::make_integer_sequence<int, 4 * MT>{});
}

// ---- the forward scan through the same register planes ---------------------------------------------
// With the lane's filter weights in the planes ([letter][tap]: A, C, G, T, mean of the four, zero) the
// scan needs no table in LDS: Z[p] += plane[letter(p + j)][j] is one v_add_f32 whose first source is
// picked by the register index mode. Taps are added in ascending order per position and the mean row is
// formed as in the LDS table, so the sums are bit-identical to the table kernels'.
template <int MT, int J>
__device__ __forceinline__ void weight_planes_tap(grad_planes<MT>& A, const float* __restrict__ W, unsigned m, unsigned F, unsigned f)
{
    float w0 = 0.0f, w1 = 0.0f, w2 = 0.0f, w3 = 0.0f;
    if (f < F && (unsigned)J < m) {
        w0 = W[(4 * J + 0) * (size_t)F + f];
        w1 = W[(4 * J + 1) * (size_t)F + f];
        w2 = W[(4 * J + 2) * (size_t)F + f];
        w3 = W[(4 * J + 3) * (size_t)F + f];
    }
    float z = w0;
    z += w1;
    z += w2;
    z += w3;
    A.template set<0 * MT + J>(w0);
    A.template set<1 * MT + J>(w1);
    A.template set<2 * MT + J>(w2);
    A.template set<3 * MT + J>(w3);
    A.template set<4 * MT + J>(z * 0.25f);
    A.template set<5 * MT + J>(0.0f);
}
template <int MT, int... J>
__device__ __forceinline__ void weight_planes_load(grad_planes<MT>& A, const float* __restrict__ W, unsigned m, unsigned F, unsigned f,
                                                   std::integer_sequence<int, J...>)
{
    (weight_planes_tap<MT, J>(A, W, m, F, f), ...);
}
// Fills the planes with filter f's weights from W (4m, F); taps >= m and filters >= F read as zero.
template <int MT>
__device__ __forceinline__ void weight_planes_load(grad_planes<MT>& A, const float* __restrict__ W, unsigned m, unsigned F, unsigned f)
{
    A.clear();
    weight_planes_load<MT>(A, W, m, F, f, std::make_integer_sequence<int, MT>{});
}

#define DBK_WP_SLOT(P) ".if ((%c[q] - " #P ") >= 0) && ((%c[q] - " #P ") < %c[mt])\n\t" \
                       "v_add_f32 %[a" #P "], v[96 + %c[q] - " #P "], %[a" #P "]\n\t.endif\n\t"
#define DBK_WP_ASM(PLANES)                                                                                          \
    asm volatile("s_set_gpr_idx_on %[idx], 0x1\n\t"                                                                  \
                 DBK_WP_SLOT(0) DBK_WP_SLOT(1) DBK_WP_SLOT(2) DBK_WP_SLOT(3) DBK_WP_SLOT(4) DBK_WP_SLOT(5) DBK_WP_SLOT(6)   \
                 DBK_WP_SLOT(7) DBK_WP_SLOT(8) DBK_WP_SLOT(9) DBK_WP_SLOT(10) DBK_WP_SLOT(11) DBK_WP_SLOT(12)            \
                 DBK_WP_SLOT(13) DBK_WP_SLOT(14) DBK_WP_SLOT(15)                                                     \
                 "s_set_gpr_idx_off"                                                                                \
                 : [a0] "+v"(acc[0]), [a1] "+v"(acc[1]), [a2] "+v"(acc[2]), [a3] "+v"(acc[3]), [a4] "+v"(acc[4]),   \
                   [a5] "+v"(acc[5]), [a6] "+v"(acc[6]), [a7] "+v"(acc[7]), [a8] "+v"(acc[8]), [a9] "+v"(acc[9]),   \
                   [a10] "+v"(acc[10]), [a11] "+v"(acc[11]), [a12] "+v"(acc[12]), [a13] "+v"(acc[13]),              \
                   [a14] "+v"(acc[14]), [a15] "+v"(acc[15])                                                         \
                 : PLANES, [idx] "s"(idx), [q] "n"(Q), [mt] "n"(MT)                                                 \
                 : "m0")

template <int Q, int MT>
__device__ __forceinline__ void weight_planes_add(const grad_planes<MT>& A, unsigned letter, float (&acc)[PSUB])
{
    static_assert(PSUB == 16, "the instruction text lists 16 positions");
    const unsigned idx = letter * (unsigned)MT;          // (M0 is clobbered: see grad_planes_add)
    if constexpr (MT == 8) DBK_WP_ASM(DBK_GP_LIST("{v[96:127]}"(A.t0), "{v[128:143]}"(A.u0)));
    else if constexpr (MT == 16) DBK_WP_ASM(DBK_GP_LIST("{v[96:127]}"(A.t0), "{v[128:159]}"(A.t1), "{v[160:191]}"(A.t2)));
    else DBK_WP_ASM(DBK_GP_LIST("{v[96:127]}"(A.t0), "{v[128:159]}"(A.t1), "{v[160:191]}"(A.t2), "{v[192:223]}"(A.t3), "{v[224:239]}"(A.u0)));
}
template <int MT, int... Q>
__device__ __forceinline__ void scan16_planes(const grad_planes<MT>& A, const unsigned (&wq)[window<MT>::words], float (&acc)[PSUB],
                                              std::integer_sequence<int, Q...>)
{
    (weight_planes_add<Q, MT>(A, window_letter(wq, Q), acc), ...);
}
// acc[p] = sum over taps of the window's weights for positions p = 0..15 (the counterpart of scan16_window).
template <int MT>
__device__ __forceinline__ void scan16_planes(const grad_planes<MT>& A, const unsigned (&wq)[window<MT>::words], float (&acc)[PSUB])
{
#pragma unroll
    for (int p = 0; p < PSUB; ++p) acc[p] = 0.0f;
    scan16_planes<MT>(A, wq, acc, std::make_integer_sequence<int, PSUB + MT - 1>{});
}

// Stages letters for absolute positions [c0, c0+cnt) into xl; past the end of X -> "nothing".
__device__ __forceinline__ void stage(uint8_t* xl, const uint8_t* __restrict__ X, size_t N, size_t c0, unsigned cnt)
{
    for (unsigned t = threadIdx.x; t < cnt; t += blockDim.x) {
        size_t g = c0 + t;
        xl[t] = g < N ? (uint8_t)letter_of(X[g]) : (uint8_t)5;
    }
}


// Element e summed over nslab slabs of nelem entries: 32 slabs in flight per round, added as four 8-wide trees in
// ascending order, whatever the round size (the one summation order every reduction of slabs uses).
__device__ __forceinline__ float slab_sum(const float* __restrict__ slabs, size_t nelem, size_t e, unsigned nslab)
{
    float total = 0.0f;
    for (unsigned base = 0; base < nslab; base += 32) {
        float buf[32];
#pragma unroll
        for (unsigned s = 0; s < 32; ++s) buf[s] = base + s < nslab ? slabs[(size_t)(base + s) * nelem + e] : 0.0f;
#pragma unroll
        for (unsigned q = 0; q < 32; q += 8)
            if (base + q < nslab)
                total += ((buf[q] + buf[q + 1]) + (buf[q + 2] + buf[q + 3])) + ((buf[q + 4] + buf[q + 5]) + (buf[q + 6] + buf[q + 7]));
    }
    return total;
}

inline size_t lds_limit()
{
    // LDS bytes a workgroup may use on the current device (asked once per device)
    static size_t cached[64] = {0};
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 65536;
    if (!cached[dev]) {
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && v > 0)
            cached[dev] = (size_t)v;
        else
            cached[dev] = 65536;
    }
    return cached[dev];
}

inline unsigned cu_count()
{
    // compute units of the current device (asked once per device); 1 when the question fails
    static unsigned cached[64] = {0};
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 1u;
    if (!cached[dev]) {
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            cached[dev] = (unsigned)v;
        else
            cached[dev] = 1u;
    }
    return cached[dev];
}

}  // namespace dbk_scan

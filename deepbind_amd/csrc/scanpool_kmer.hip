// Fast path of the fused scan + bias + ReLU + region pooling forward: a 3-mer lookup table in LDS.
//
// The scan is a gather-add: Z[p,f] = sum_j w(j, X[p+j], f). Grouping taps three at a time turns
// it into G = ceil(m/3) adds per (position, filter): Z[p,f] = sum_g L_g[kmer(p+3g)][f], where
// kmer(t) indexes the 5-letter triple (X[t], X[t+1], X[t+2]) (A,C,G,T and "mean of the four" for
// N / padding: 125 triples) and L_g holds the three taps' weights pre-summed (bias folded into
// L_0). That cuts executed VALU adds and LDS bytes per algorithmic add by 3.
//
// Mapping to the hardware:
//  * A workgroup owns 32 filters. Its table fills the CU's LDS (126 KB for m = 24), one workgroup
//    per CU: lut[triple][line i][lane l][4 floats] with line i holding tap groups 2i and 2i+1 and the
//    lane's 16 bytes holding (group 2i, filters 2l and 2l+1 | group 2i+1, filters 2l and 2l+1).
//  * ds_read_b128 only reaches the LDS's full rate (~210 B/clk/CU measured, against ~155 otherwise)
//    when each group of 16 lanes reads one 256-byte-ALIGNED line. So a "stream" is 16 lanes walking
//    one region, 2 filters per lane, and a step's G/2 reads are the G/2 lines of the step's triple:
//    always aligned, never conflicting. A wave carries 4 streams (4 regions at once).
//  * Each lane keeps a ring of 3 x G float2 accumulators in VGPRs: at text position t the read of
//    line i adds group 2i into position t-6i and group 2i+1 into position t-6i-3; group 0 starts a
//    position (plain assignment), group G-1 completes it, it is folded into the running max and
//    its slot is reused. The step loop is unrolled over 3G positions so every ring index is a
//    compile-time register; per (position, 2 filters) that is 2(G-1) adds and ~1.3 max
//    instructions for 2*3G algorithmic adds.
//  * The sequence is pre-translated once into one byte per position (the triple index). A stream's
//    16 lanes fetch a block's 3G indices cooperatively (one or two bytes per lane, one block ahead)
//    and each step takes its index from the owning lane with a DPP row_share folded into the add
//    that forms the LDS address: one VALU instruction of addressing per step.
//  * A workgroup owns a contiguous range of regions; its streams claim them one at a time from a counter in LDS (the
//    SIMD favours its oldest wave: equal static shares would finish 5 % apart). A step's table lines are asked for
//    one step before they are added (scheduling barriers keep that order in the unrolled block): four to eight
//    ds_read_b128 in flight per wave, one wait per step, the LDS pipe busy 99 % of the time.
//  * Plain max pooling goes on from one region into the next where they follow each other in the text: with filters of up
//    to 18 taps through whole runs of regions (table_scan_runs), with 19-24 taps through pairs (table_scan_pairs).
//  * Positions outside a region never need a test. At a region's start every ring slot is reset to
//    a large negative "poison" (-1e30), so the partial sums in flight from before the region finish
//    far below any real value; and the steps a region's last block runs past its final useful
//    position read a 126th table entry that is all poison, which sinks exactly the positions that
//    lie beyond the region. The running max ignores both, and ReLU follows the max.
//
// Pooling variants share the loop: the running max (plain, or with the index of the winning triple of
// positions, whose exact position is settled at the region's end by re-adding those three positions'
// entries in the same order), and / or the running sum of rectified values for average pooling
// (positions outside the region carry a poison term, so their rectified value is exactly zero).
//
// Shapes this path declines (filter length > 24, code 254 present, regions reaching past the last row
// the scan defines) go through the general kernel in scanpool.hip.
//
// Reference chain being fused: kangaroo/_ext/corr1ord.py:97-117 -> deepity/std/elemwise.py:162-180,71-82
// -> kangaroo/_ext/poolrgn.py:56-76 (kernels corr1ord.cuh:139-157, poolrgn.cuh:44-79).
#include "dbk_common.h"
#include "scan_common.h"
#include <cmath>
#include <mutex>

namespace dbk_scanpool_general {
int fprop(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
          const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax, const unsigned* run_if_flag,
          unsigned long long* act);
}

namespace dbk_scanpool_kmer {

constexpr int FTILE = 32;            // filters per workgroup
constexpr int ROWB = FTILE * 4;      // bytes per table row
constexpr int NKMER = 125;          // real triples; entry 125 is the poison entry
constexpr float POISON = -1.0e30f;
constexpr int KPAD = 128;            // index bytes readable past the end of the sequence

__device__ __forceinline__ unsigned letter5(unsigned code) { return code < 4u ? code : 4u; }

__global__ void clear_flag_kernel(unsigned* flag) { flag[0] = 0; }

// K[t] = 25*l(X[t]) + 5*l(X[t+1]) + l(X[t+2]) for t < N + KPAD, reading past the end as N (letter 4).
// Sets flag[0] (cleared beforehand) when the table kernel must stand down: a code 254 ("contributes
// nothing") is present, for which the table has no letter, or a region is reversed or reaches past
// row ndef, the last row the scan defines. A thread makes four indices from two aligned 32-bit loads.
__global__ __launch_bounds__(256) void kmer_index_kernel(const uint8_t* __restrict__ X, size_t N, uint8_t* __restrict__ K, unsigned* flag,
                                                         const uint32_t* __restrict__ R, size_t P, size_t ndef)
{
    const size_t total = N + KPAD;                       // a multiple of 4 is not required: the tail is done bytewise
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nthread = (size_t)gridDim.x * blockDim.x;
    unsigned bad = 0;
    for (size_t r = tid; r < P; r += nthread) {
        const uint2 ab = reinterpret_cast<const uint2*>(R)[r];
        bad |= (ab.y < ab.x || ab.y > ndef);
    }
    const bool aligned = (reinterpret_cast<uintptr_t>(X) & 3) == 0 && (reinterpret_cast<uintptr_t>(K) & 3) == 0;
    const size_t nquad = aligned ? total / 4 : 0;
    const size_t nword = (N + 3) / 4;                    // 32-bit words of X that may be read
    for (size_t q = tid; q < nquad; q += nthread) {
        unsigned w0 = q < nword ? reinterpret_cast<const unsigned*>(X)[q] : 0xffffffffu;
        unsigned w1 = q + 1 < nword ? reinterpret_cast<const unsigned*>(X)[q + 1] : 0xffffffffu;
        unsigned l[6];
#pragma unroll
        for (int j = 0; j < 6; ++j) {
            const size_t t = 4 * q + j;
            unsigned c = ((j < 4 ? w0 : w1) >> (8 * (j & 3))) & 0xffu;
            if (t >= N) c = 255u;                        // bytes of the last word past the end of the stream
            bad |= (j < 4 && c == 254u);
            l[j] = letter5(c);
        }
        unsigned out = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) out |= (25u * l[j] + 5u * l[j + 1] + l[j + 2]) << (8 * j);
        reinterpret_cast<unsigned*>(K)[q] = out;
    }
    for (size_t t = 4 * nquad + tid; t < total; t += nthread) {
        unsigned c0 = t < N ? X[t] : 255u, c1 = t + 1 < N ? X[t + 1] : 255u, c2 = t + 2 < N ? X[t + 2] : 255u;
        bad |= (c0 == 254u);
        K[t] = (uint8_t)(25u * letter5(c0) + 5u * letter5(c1) + letter5(c2));
    }
    if (bad) atomicOr(flag, 1u);
}

// Value of `v` held by lane `src` of the caller's row of 16 lanes (DPP row_share, folded by the
// compiler into the consuming VALU instruction).
template <int SRC>
__device__ __forceinline__ unsigned row_share(unsigned v)
{
    return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x150 + SRC, 0xf, 0xf, false);
}

// MODE bits: what a finished position is folded into
constexpr int M_MAX = 1, M_ARG = 2, M_SUM = 4;

// The table byte offset of block position T, taken from the lane of the stream that fetched it.
template <int T>
__device__ __forceinline__ unsigned block_offset(unsigned k0, unsigned k1)
{
    if constexpr (T < 16) return row_share<T>(k0);
    else return row_share<T - 16>(k1);
}

// A step's G/2 table lines for this lane: 16 bytes of each.
template <int G, int T>
__device__ __forceinline__ void read_step(const char* __restrict__ lds, unsigned k0, unsigned k1, unsigned lanebase, float4 (&v)[G / 2])
{
    const unsigned addr = block_offset<T>(k0, k1) + lanebase;
#pragma unroll
    for (int i = 0; i < G / 2; ++i) v[i] = *reinterpret_cast<const float4*>(lds + addr + i * 256);
}

// How a block's finished positions are kept apart when regions follow each other without a fresh start (plain max pooling):
// NP parts of PP positions each, every part with a maximum of its own.
template <int G> struct run_parts {
    static constexpr int NP = (G % 4 == 0) ? 4 : 2, PP = 3 * G / NP;
};

template <int G, int MODE, int T, bool PARTS = false>
__device__ __forceinline__ void scan_steps(const char* __restrict__ lds, unsigned k0, unsigned k1, unsigned n0, unsigned n1,
                                           float2 (&acc)[3][G], float2& mx, uint2& best, float2& sum, unsigned lanebase, unsigned triple0,
                                           float4 (&cur)[G / 2], float2 (&part)[run_parts<G>::NP])
{
    constexpr int H = G / 2, q = T / 3, c = T % 3;
    // the next step's lines (the next block's first step after the last one) are asked for before this step's are added:
    // a wave keeps G/2 to G reads in flight and waits once per step
    float4 nxt[H];
    if constexpr (T + 1 < 3 * G) read_step<G, T + 1>(lds, k0, k1, lanebase, nxt);
    else read_step<G, 0>(lds, n0, n1, lanebase, nxt);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < H; ++i) {
        const float4 v = cur[i];
        const int s0 = (((q - 2 * i) % G) + G) % G;          // position t - 6i   takes group 2i
        const int s1 = (((q - 2 * i - 1) % G) + G) % G;      // position t - 6i-3 takes group 2i+1
        if (i == 0) { acc[c][s0].x = v.x; acc[c][s0].y = v.y; }     // group 0 starts a position
        else { acc[c][s0].x += v.x; acc[c][s0].y += v.y; }
        acc[c][s1].x += v.z; acc[c][s1].y += v.w;
    }
    if constexpr (c == 2) {
        // group G-1 just landed in slot (q+1) mod G of each class: three finished positions, in text order
        constexpr int cs = (q + 1) % G;
        if (MODE & M_ARG) {
            // remember which triple of positions holds the running maximum (strictly greater: the earliest
            // triple wins ties); the position inside the triple is settled when the region ends
            const float m3x = fmaxf(fmaxf(acc[0][cs].x, acc[1][cs].x), acc[2][cs].x);
            const float m3y = fmaxf(fmaxf(acc[0][cs].y, acc[1][cs].y), acc[2][cs].y);
            const bool ux = m3x > mx.x, uy = m3y > mx.y;
            mx.x = ux ? m3x : mx.x;
            mx.y = uy ? m3y : mx.y;
            best.x = ux ? triple0 + q : best.x;
            best.y = uy ? triple0 + q : best.y;
        } else if (PARTS) {
            constexpr int h = 3 * q / run_parts<G>::PP;
            part[h].x = fmaxf(fmaxf(part[h].x, acc[0][cs].x), acc[1][cs].x); part[h].y = fmaxf(fmaxf(part[h].y, acc[0][cs].y), acc[1][cs].y);
            part[h].x = fmaxf(part[h].x, acc[2][cs].x); part[h].y = fmaxf(part[h].y, acc[2][cs].y);
        } else if (MODE & M_MAX) {
            mx.x = fmaxf(fmaxf(mx.x, acc[0][cs].x), acc[1][cs].x); mx.y = fmaxf(fmaxf(mx.y, acc[0][cs].y), acc[1][cs].y);
            mx.x = fmaxf(mx.x, acc[2][cs].x); mx.y = fmaxf(mx.y, acc[2][cs].y);
        }
        if (MODE & M_SUM) {
            // positions outside the region carry a poison term: their rectified value is exactly 0
#pragma unroll
            for (int cc = 0; cc < 3; ++cc) {
                sum.x += fmaxf(acc[cc][cs].x, 0.f);
                sum.y += fmaxf(acc[cc][cs].y, 0.f);
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < H; ++i) cur[i] = nxt[i];
    if constexpr (T + 1 < 3 * G) scan_steps<G, MODE, T + 1, PARTS>(lds, k0, k1, n0, n1, acc, mx, best, sum, lanebase, triple0, cur, part);
}

// One unrolled block of 3G text positions for one lane.
//   k0, k1    table byte offsets (triple index * bytes per triple) of this block's positions, spread
//             over the stream's 16 lanes: lane i holds position i in k0 and position 16+i in k1
//   n0, n1    the same for the block after it
//   acc       ring of partial sums (2 filters per lane), mx the running max
//   cur       the lines of this block's first step (read by the block before); on return, those of the next block's
template <int G, int MODE>
__device__ __forceinline__ void scan_block(const char* __restrict__ lds, unsigned k0, unsigned k1, unsigned n0, unsigned n1,
                                           float2 (&acc)[3][G], float2& mx, uint2& best, float2& sum, unsigned lanebase, unsigned triple0,
                                           float4 (&cur)[G / 2])
{
    float2 none[run_parts<G>::NP];
    scan_steps<G, MODE, 0>(lds, k0, k1, n0, n1, acc, mx, best, sum, lanebase, triple0, cur, none);
}

// The sum of one position's G table entries for this lane's two filters, groups in ascending order:
// the same additions, in the same order, as the ring performs.
template <int G>
__device__ __forceinline__ float2 rescan_position(const char* __restrict__ lds, const uint8_t* __restrict__ K, size_t t0, unsigned lanebase)
{
    constexpr unsigned KSTRIDE = G * ROWB;
    float2 z = make_float2(0.f, 0.f);
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const unsigned km = K[t0 + 3 * g];
        const float4 v = *reinterpret_cast<const float4*>(lds + km * KSTRIDE + lanebase + (g >> 1) * 256);
        const float vx = (g & 1) ? v.z : v.x, vy = (g & 1) ? v.w : v.y;
        if (g == 0) { z.x = vx; z.y = vy; }
        else { z.x += vx; z.y += vy; }
    }
    return z;
}

// The workgroup's table for the 32 filters from f0 on: per-tap, per-letter weights first (taps >= m are zero), then
// the 3-mer sums, taps in ascending order, bias first for group 0; entry 125 is all poison. All threads take part;
// ends with a barrier.
template <int G>
__device__ __forceinline__ void build_table(float* __restrict__ lut, float* __restrict__ w5, const float* __restrict__ W,
                                            const float* __restrict__ bias, unsigned m, unsigned F, unsigned f0)
{
    constexpr int STEPS = 3 * G;
    for (unsigned e = threadIdx.x; e < (unsigned)STEPS * FTILE; e += blockDim.x) {
        const unsigned j = e / FTILE, fl = e % FTILE, f = f0 + fl;
        float w0 = 0.f, w1 = 0.f, w2 = 0.f, w3 = 0.f;
        if (j < m && f < F) {
            w0 = W[(size_t)(4 * j + 0) * F + f];
            w1 = W[(size_t)(4 * j + 1) * F + f];
            w2 = W[(size_t)(4 * j + 2) * F + f];
            w3 = W[(size_t)(4 * j + 3) * F + f];
        }
        float z = w0; z += w1; z += w2; z += w3;
        float* row = w5 + (size_t)j * 5 * FTILE + fl;
        row[0 * FTILE] = w0; row[1 * FTILE] = w1; row[2 * FTILE] = w2; row[3 * FTILE] = w3; row[4 * FTILE] = z * 0.25f;
    }
    __syncthreads();
    // a lane's 16 bytes of a line at a time: unit u -> (triple, line i, lane l) holds group 2i for filters 2l, 2l + 1, then
    // group 2i + 1 for the same two (one decode of u, six 8-byte reads of the letter weights and one 16-byte write per unit)
    const unsigned fmax = F > f0 ? F - f0 : 0u;                  // filters of this tile that exist
    for (unsigned u = threadIdx.x; u < (unsigned)(NKMER + 1) * (G / 2) * 16u; u += blockDim.x) {
        const unsigned l = u & 15u, i = (u >> 4) % (unsigned)(G / 2), km = u / (unsigned)(8 * G), fl = 2 * l;
        const unsigned l0 = km / 25u, l1 = (km / 5u) % 5u, l2 = km % 5u;
        float4 v = make_float4(POISON, POISON, POISON, POISON);
        if (km < (unsigned)NKMER) {
            float2 sg[2];
#pragma unroll
            for (unsigned j = 0; j < 2; ++j) {
                const unsigned g = 2 * i + j;
                float2 t = make_float2(0.0f, 0.0f);
                if (g == 0) { t.x = fl < fmax ? bias[f0 + fl] : 0.0f; t.y = fl + 1 < fmax ? bias[f0 + fl + 1] : 0.0f; }
                const float2 a0 = *reinterpret_cast<const float2*>(w5 + ((size_t)(3 * g + 0) * 5 + l0) * FTILE + fl);
                const float2 a1 = *reinterpret_cast<const float2*>(w5 + ((size_t)(3 * g + 1) * 5 + l1) * FTILE + fl);
                const float2 a2 = *reinterpret_cast<const float2*>(w5 + ((size_t)(3 * g + 2) * 5 + l2) * FTILE + fl);
                t.x += a0.x; t.y += a0.y;
                t.x += a1.x; t.y += a1.y;
                t.x += a2.x; t.y += a2.y;
                sg[j] = t;
            }
            v = make_float4(sg[0].x, sg[0].y, sg[1].x, sg[1].y);
        }
        reinterpret_cast<float4*>(lut)[u] = v;
    }
    __syncthreads();
}

// A wave of the table scan. Its four streams take the workgroup's regions as they come: a stream that finishes a region
// claims the next unclaimed one from `counter` (LDS; set to the first region before the table's barriers), up to `rend`.
// The SIMD favours its oldest wave, so waves that were given equal shares would finish 5-20 % apart; which stream scans a
// region does not change a bit of its result.
template <int G, int MODE>
__device__ __forceinline__ void table_scan(const char* __restrict__ lds, unsigned F, unsigned f0, const uint8_t* __restrict__ K,
                                           const uint32_t* __restrict__ R, unsigned* counter, unsigned rend,
                                           float* __restrict__ pooled, uint32_t* __restrict__ argmax)
{
    constexpr int STEPS = 3 * G;
    constexpr unsigned KSTRIDE = G * ROWB;                     // bytes per triple: G/2 lines of 256 B
    const unsigned P = rend;
    const unsigned lane = threadIdx.x & 63;
    const unsigned lanebase = (lane & 15u) * 16u;
    constexpr unsigned TAIL = 3 * (G - 1);                       // steps between a position's start and its completion
    auto claim = [&]() -> unsigned {
        unsigned v = 0u;
        if ((lane & 15u) == 0u) v = atomicAdd(counter, 1u);
        return row_share<0>(v);
    };

    unsigned r = claim(), rn = claim();                          // the region in work, the one after it
    unsigned a = 0, rows = 0, a_next = 0, rows_next = 0;
    if (r < P) { a = R[2 * (size_t)r]; rows = R[2 * (size_t)r + 1] - a; }
    if (rn < P) { a_next = R[2 * (size_t)rn]; rows_next = R[2 * (size_t)rn + 1] - a_next; }
    unsigned nblk = (rows + TAIL + STEPS - 1) / STEPS;
    if (nblk < 1) nblk = 1;

    // lane i of a stream fetches the triple index of block positions i and 16+i; positions at or
    // past rows+TAIL (nothing valid completes there any more) read the poison entry instead
    const unsigned q16 = lane & 15;
    const unsigned q16b = 16u + (STEPS > 16 ? (q16 < (unsigned)(STEPS - 16) ? q16 : (unsigned)(STEPS - 17)) : 0u);
    auto fetch = [&](unsigned base, unsigned limit, unsigned pos0, unsigned& o0, unsigned& o1) {
        // base: absolute text position of the block's first step, pos0: its region-relative position,
        // limit: rows + TAIL of the block's region
        unsigned v0 = K[(size_t)base + q16];
        unsigned v1 = STEPS > 16 ? (unsigned)K[(size_t)base + q16b] : 0u;
        o0 = (pos0 + q16 < limit ? v0 : (unsigned)NKMER) * KSTRIDE;
        o1 = (pos0 + q16b < limit ? v1 : (unsigned)NKMER) * KSTRIDE;
    };
    unsigned k0, k1;
    fetch(a, r < P ? rows + TAIL : 0u, 0u, k0, k1);

    float2 acc[3][G];
#pragma unroll
    for (int c = 0; c < 3; ++c)
#pragma unroll
        for (int s = 0; s < G; ++s) acc[c][s] = make_float2(POISON, POISON);
    float2 mx = make_float2(POISON, POISON);
    uint2 best = make_uint2(0u, 0u);
    float2 sum = make_float2(0.f, 0.f);
    unsigned blk = 0;
    float4 cur[G / 2];                                           // the lines of the coming block's first step
    read_step<G, 0>(lds, k0, k1, lanebase, cur);

    while (true) {
        const bool active = r < P;
        if (!__any(active)) break;
        const bool last = blk + 1 >= nblk;
        // the next block's indices travel while this block computes
        unsigned n0, n1;
        if (last) fetch(a_next, rn < P ? rows_next + TAIL : 0u, 0u, n0, n1);
        else fetch(a + (blk + 1) * STEPS, rows + TAIL, (blk + 1) * STEPS, n0, n1);
        scan_block<G, MODE>(lds, k0, k1, n0, n1, acc, mx, best, sum, lanebase, blk * (unsigned)G, cur);
        k0 = n0;
        k1 = n1;
        if (last) {
            // ReLU and store this lane's two of the region's 32 pooled features
            if (active) {
                const unsigned f = f0 + (lane & 15u) * 2;
                const float inv = 1.0f / (float)rows;
                if (MODE == M_SUM) {
                    float* out = pooled + (size_t)r * F + f;
                    if (f + 0 < F) out[0] = sum.x * inv;
                    if (f + 1 < F) out[1] = sum.y * inv;
                } else if (MODE & M_SUM) {
                    float* out = pooled + ((size_t)r * F + f) * 2;           // (max, avg) interleaved per filter
                    if (f + 0 < F) { out[0] = fmaxf(mx.x, 0.f); out[1] = sum.x * inv; }
                    if (f + 1 < F) { out[2] = fmaxf(mx.y, 0.f); out[3] = sum.y * inv; }
                } else {
                    float* out = pooled + (size_t)r * F + f;
                    if (f + 0 < F) out[0] = fmaxf(mx.x, 0.f);
                    if (f + 1 < F) out[1] = fmaxf(mx.y, 0.f);
                }
                if (MODE & M_ARG) {
                    // first row of the region whose rectified value equals the maximum: the region's first row when
                    // nothing is positive, else the first position of the winning triple that reproduces the maximum
                    unsigned px = 0, py = 0;
                    if (mx.x > 0.f) {
#pragma unroll
                        for (int c = 2; c >= 0; --c) {
                            const int p = (int)(3u * best.x) + c - (int)TAIL;
                            if (p >= 0 && (unsigned)p < rows && rescan_position<G>(lds, K, (size_t)a + p, lanebase).x == mx.x) px = (unsigned)p;
                        }
                    }
                    if (mx.y > 0.f) {
#pragma unroll
                        for (int c = 2; c >= 0; --c) {
                            const int p = (int)(3u * best.y) + c - (int)TAIL;
                            if (p >= 0 && (unsigned)p < rows && rescan_position<G>(lds, K, (size_t)a + p, lanebase).y == mx.y) py = (unsigned)p;
                        }
                    }
                    uint32_t* am = argmax + (size_t)r * F + f;
                    if (f + 0 < F) am[0] = (uint32_t)(((size_t)a + px) * F + f);
                    if (f + 1 < F) am[1] = (uint32_t)(((size_t)a + py) * F + f + 1);
                }
            }
            // new region: everything still in the ring belongs to the old one
            mx = make_float2(POISON, POISON);
            best = make_uint2(0u, 0u);
            sum = make_float2(0.f, 0.f);
#pragma unroll
            for (int c = 0; c < 3; ++c)
#pragma unroll
                for (int s = 0; s < G; ++s) acc[c][s] = make_float2(POISON, POISON);
            r = rn;
            rn = claim();
            a = a_next; rows = rows_next; blk = 0;
            nblk = (rows + TAIL + STEPS - 1) / STEPS;
            if (nblk < 1) nblk = 1;
            a_next = 0; rows_next = 0;
            if (rn < P) { a_next = R[2 * (size_t)rn]; rows_next = R[2 * (size_t)rn + 1] - a_next; }
        } else {
            ++blk;
        }
    }
}

// table_scan for plain max pooling with filters of 19-24 taps: two regions that follow each other in the text are scanned
// as one stretch, so the fill of the ring (TAIL steps) and the rounding to whole blocks are paid once per pair. The block
// grid starts `lead` steps before the first region, chosen so that the first region's last position completes exactly at a
// block's end: there its maximum is written out and the running maximum starts again, and nothing else changes - the ring
// goes on, since what is in flight belongs to the second region. Steps before the first region read the poison entry
// like those past the end, which sinks every position that does not belong to the pair. A stream claims two regions at
// a time (`nclaim` = 2; with 1 - calls too small to give every stream a few pairs - regions are taken singly, as in
// table_scan); two that do not follow each other are scanned one after the other.
template <int G, int MODE>
__device__ __forceinline__ void table_scan_pairs(const char* __restrict__ lds, unsigned F, unsigned f0, const uint8_t* __restrict__ K,
                                                 const uint32_t* __restrict__ R, unsigned* counter, unsigned nclaim, unsigned rend, float* __restrict__ pooled)
{
    constexpr unsigned STEPS = 3 * G, KSTRIDE = G * ROWB, TAIL = 3 * (G - 1), NONE = 0xffffffffu;
    const unsigned P = rend;
    const unsigned lane = threadIdx.x & 63;
    const unsigned lanebase = (lane & 15u) * 16u;
    const unsigned q16 = lane & 15;
    const unsigned q16b = 16u + (STEPS > 16 ? (q16 < (unsigned)(STEPS - 16) ? q16 : (unsigned)(STEPS - 17)) : 0u);
    unsigned carry = NONE;                                       // the second region of a claim whose two do not follow each other
    // The next item: its first region (P: none left), the text position of its block grid, the steps that are real
    // ([lead, lead + span)), and the number of blocks after which the first region of a pair is complete (0: a single).
    auto take = [&](unsigned& rr, unsigned& grid, unsigned& lead, unsigned& span, unsigned& bnd) {
        bool fresh = carry == NONE;
        if (fresh) {
            unsigned v = 0u;
            if (q16 == 0u) v = atomicAdd(counter, nclaim);
            rr = row_share<0>(v);
        } else {
            rr = carry;
            carry = NONE;
        }
        grid = 0u; lead = 0u; span = 0u; bnd = 0u;
        if (rr >= P) { rr = P; return; }
        const unsigned a_ = R[2 * (size_t)rr], rows_ = R[2 * (size_t)rr + 1] - a_;
        grid = a_; span = rows_ + TAIL;
        if (fresh && nclaim == 2u && rr + 1u < P) {
            const unsigned a2 = R[2 * (size_t)rr + 2], rows2 = R[2 * (size_t)rr + 3] - a2;
            const unsigned ld = (STEPS - (rows_ + TAIL) % STEPS) % STEPS;
            if (a2 == a_ + rows_ && a_ >= ld) {
                grid = a_ - ld; lead = ld; span = rows_ + rows2 + TAIL; bnd = (ld + rows_ + TAIL) / STEPS;
            } else {
                carry = rr + 1u;
            }
        }
    };
    auto fetch = [&](unsigned text, unsigned pos0, unsigned lead, unsigned span, unsigned& o0, unsigned& o1) {
        // text: position of the block's first step, pos0: the same counted from the grid's start
        unsigned v0 = K[(size_t)text + q16];
        unsigned v1 = STEPS > 16 ? (unsigned)K[(size_t)text + q16b] : 0u;
        o0 = (pos0 + q16 - lead < span ? v0 : (unsigned)NKMER) * KSTRIDE;
        o1 = (pos0 + q16b - lead < span ? v1 : (unsigned)NKMER) * KSTRIDE;
    };
    unsigned r, grid, lead, span, bnd, rn, grid_n, lead_n, span_n, bnd_n;
    take(r, grid, lead, span, bnd);
    take(rn, grid_n, lead_n, span_n, bnd_n);
    unsigned nblk = (lead + span + STEPS - 1) / STEPS;
    if (nblk < 1) nblk = 1;
    unsigned k0, k1;
    fetch(grid, 0u, lead, r < P ? span : 0u, k0, k1);

    float2 acc[3][G];
#pragma unroll
    for (int c = 0; c < 3; ++c)
#pragma unroll
        for (int s = 0; s < G; ++s) acc[c][s] = make_float2(POISON, POISON);
    float2 mx = make_float2(POISON, POISON);
    uint2 best = make_uint2(0u, 0u);
    float2 sum = make_float2(0.f, 0.f);
    float2 mx1 = make_float2(POISON, POISON), sum1 = make_float2(0.f, 0.f);   // the first region's maximum and sum while the second is scanned
    unsigned blk = 0;
    float4 cur[G / 2];                                           // the lines of the coming block's first step
    read_step<G, 0>(lds, k0, k1, lanebase, cur);
    const unsigned f = f0 + q16 * 2;

    while (true) {
        const bool active = r < P;
        if (!__any(active)) break;
        const bool last = blk + 1 >= nblk;
        // the next block's indices travel while this block computes
        unsigned n0, n1;
        if (last) fetch(grid_n, 0u, lead_n, rn < P ? span_n : 0u, n0, n1);
        else fetch(grid + (blk + 1) * STEPS, (blk + 1) * STEPS, lead, span, n0, n1);
        scan_block<G, MODE>(lds, k0, k1, n0, n1, acc, mx, best, sum, lanebase, 0u, cur);
        k0 = n0;
        k1 = n1;
        // where the first region of a pair is complete (and nothing of the second is) its maximum is put aside and the
        // running maximum starts again; the ring goes on. (Selects, not a branch: any control flow between the unrolled
        // block and the loop's end that leaves the ring alive costs the compiler its register allocation.)
        const bool first_done = blk + 1 == bnd;
        if (MODE & M_MAX) {
            mx1.x = first_done ? mx.x : mx1.x; mx1.y = first_done ? mx.y : mx1.y;
            mx.x = first_done ? POISON : mx.x; mx.y = first_done ? POISON : mx.y;
        }
        if (MODE & M_SUM) {
            sum1.x = first_done ? sum.x : sum1.x; sum1.y = first_done ? sum.y : sum1.y;
            sum.x = first_done ? 0.f : sum.x; sum.y = first_done ? 0.f : sum.y;
        }
        if (last) {
            // ReLU and store this lane's two of each region's 32 pooled features
            if (active) {
                // (the first region's rows from where its last position completed; the second's are the rest)
                const unsigned rows1 = bnd * STEPS - lead - TAIL, rows2 = span - TAIL - (bnd != 0u ? rows1 : 0u);
                auto put = [&](unsigned rr, float2 vmax, float2 vsum, unsigned nrow) {
                    const float inv = 1.0f / (float)nrow;
                    if (MODE == M_SUM) {
                        float* out = pooled + (size_t)rr * F + f;
                        if (f + 0 < F) out[0] = vsum.x * inv;
                        if (f + 1 < F) out[1] = vsum.y * inv;
                    } else if (MODE & M_SUM) {
                        float* out = pooled + ((size_t)rr * F + f) * 2;          // (max, avg) interleaved per filter
                        if (f + 0 < F) { out[0] = fmaxf(vmax.x, 0.f); out[1] = vsum.x * inv; }
                        if (f + 1 < F) { out[2] = fmaxf(vmax.y, 0.f); out[3] = vsum.y * inv; }
                    } else {
                        float* out = pooled + (size_t)rr * F + f;
                        if (f + 0 < F) out[0] = fmaxf(vmax.x, 0.f);
                        if (f + 1 < F) out[1] = fmaxf(vmax.y, 0.f);
                    }
                };
                if (bnd != 0u) put(r, mx1, sum1, rows1);
                put(r + (bnd != 0u ? 1u : 0u), mx, sum, rows2);
            }
            // a new item: everything still in the ring belongs to the old one
            mx = make_float2(POISON, POISON);
            sum = make_float2(0.f, 0.f);
#pragma unroll
            for (int c = 0; c < 3; ++c)
#pragma unroll
                for (int s = 0; s < G; ++s) acc[c][s] = make_float2(POISON, POISON);
            r = rn; grid = grid_n; lead = lead_n; span = span_n; bnd = bnd_n; blk = 0;
            nblk = (lead + span + STEPS - 1) / STEPS;
            if (nblk < 1) nblk = 1;
            take(rn, grid_n, lead_n, span_n, bnd_n);
        } else {
            ++blk;
        }
    }
}

// One position's sum for this lane's two filters from index bytes that lie spread over the stream's lanes (lane i holds
// the table offsets of bytes i and 16 + i of a stretch of text in e0 / e1): position C of the stretch takes its group g
// from byte C + 3g. The same additions, in the same order, as the ring performs.
template <int G, int C, int GG>
__device__ __forceinline__ void readd_group(const char* __restrict__ lds, unsigned e0, unsigned e1, unsigned lanebase, float2& z)
{
    const float2 v = *reinterpret_cast<const float2*>(lds + block_offset<C + 3 * GG>(e0, e1) + lanebase + (GG >> 1) * 256 + (GG & 1) * 8);
    if constexpr (GG == 0) { z.x = v.x; z.y = v.y; }
    else { z.x += v.x; z.y += v.y; }
    if constexpr (GG + 1 < G) readd_group<G, C, GG + 1>(lds, e0, e1, lanebase, z);
}
// The PP positions of the part of a block that held the end of a region: the first `nold` go to the maximum of the region
// that ended (o), the others to that of the region that followed it (n).
template <int G, int C>
__device__ __forceinline__ void readd_part(const char* __restrict__ lds, unsigned e0, unsigned e1, unsigned lanebase, unsigned nold,
                                           float2& o, float2& n)
{
    float2 z;
    readd_group<G, C, 0>(lds, e0, e1, lanebase, z);
    const bool old = (unsigned)C < nold;
    o.x = fmaxf(o.x, old ? z.x : POISON); o.y = fmaxf(o.y, old ? z.y : POISON);
    n.x = fmaxf(n.x, old ? POISON : z.x); n.y = fmaxf(n.y, old ? POISON : z.y);
    __builtin_amdgcn_sched_barrier(0);                           // (a position at a time: this path has no registers to spare)
    if constexpr (C + 1 < run_parts<G>::PP) readd_part<G, C + 1>(lds, e0, e1, lanebase, nold, o, n);
}

// The table scan for plain max pooling. As table_scan, but a stream claims `run` consecutive regions at a time and, where
// a region starts at the text position at which the one before it ended (sequences packed back to back) and is at
// least three blocks long, walks on without a fresh start: the last positions of a region complete while the first of
// the next are under way, which saves the TAIL steps of drain and the rounding to whole blocks that every region
// otherwise costs (29 of 552 steps at 523 rows, 35 % at 101). A block keeps the maxima of its finished positions in NP
// parts; where a region ends inside a block the parts before the boundary go to it, those after it to its follower, and
// the part that holds the boundary is left out: its PP positions are added up again from the table one region later
// (index bytes asked for at the boundary), just before the region that ended is written out. A region that does not
// follow on ends the run: poison from its last step on, as in table_scan, and a fresh start.
// Every position's sum is formed by the same additions in the same order either way.
template <int G>
__device__ __forceinline__ void table_scan_runs(const char* __restrict__ lds, unsigned F, unsigned f0, const uint8_t* __restrict__ K,
                                                const uint32_t* __restrict__ R, unsigned* counter, unsigned run, unsigned rend, float* __restrict__ pooled)
{
    constexpr unsigned STEPS = 3 * G, NP = run_parts<G>::NP, PP = run_parts<G>::PP, FOLLOW_ROWS = 3 * STEPS, NOLIMIT = 0xffffffffu;
    constexpr unsigned KSTRIDE = G * ROWB;                     // bytes per triple: G/2 lines of 256 B
    constexpr unsigned TAIL = 3 * (G - 1);                       // steps between a position's start and its completion
    const unsigned P = rend;
    const unsigned lane = threadIdx.x & 63;
    const unsigned lanebase = (lane & 15u) * 16u;
    // the stream's share of the workgroup's regions: `run` consecutive ones per claim
    unsigned mine = 0u, mine_end = 0u;
    bool dry = false;                                            // a claim came back past the last region
    auto take = [&]() -> unsigned {
        if (mine >= mine_end && !dry) {
            unsigned v = 0u;
            if ((lane & 15u) == 0u) v = atomicAdd(counter, run);
            mine = row_share<0>(v);
            mine_end = mine + run < P ? mine + run : P;
            dry = mine >= P;
        }
        return dry ? P : mine++;
    };
    auto bounds = [&](unsigned rr, unsigned& a_, unsigned& rows_) {
        a_ = 0u; rows_ = 0u;
        if (rr < P) { a_ = R[2 * (size_t)rr]; rows_ = R[2 * (size_t)rr + 1] - a_; }
    };
    unsigned r = take(), r1 = take();                            // the region in work, the one after it
    unsigned a, rows, a1, rows1;
    bounds(r, a, rows); bounds(r1, a1, rows1);
    unsigned base = a, end = rows, s0 = 0u;                      // the run's first text position; the region's end and the block's first step, relative to it
    // the next region continues the run (a region that ends in the run's first block would need positions from before it)
    bool follows = r1 == r + 1u && r1 < P && a1 == a + rows && rows1 >= FOLLOW_ROWS && rows >= STEPS;

    const unsigned q16 = lane & 15;
    const unsigned q16b = 16u + (STEPS > 16 ? (q16 < (unsigned)(STEPS - 16) ? q16 : (unsigned)(STEPS - 17)) : 0u);
    auto fetch = [&](unsigned text, unsigned limit, unsigned pos0, unsigned& o0, unsigned& o1) {
        // text: position of the block's first step, pos0: the same relative to the run's start; steps at or past `limit`
        // read the poison entry
        unsigned v0 = K[(size_t)text + q16];
        unsigned v1 = STEPS > 16 ? (unsigned)K[(size_t)text + q16b] : 0u;
        o0 = (pos0 + q16 < limit ? v0 : (unsigned)NKMER) * KSTRIDE;
        o1 = (pos0 + q16b < limit ? v1 : (unsigned)NKMER) * KSTRIDE;
    };
    unsigned k0, k1;
    fetch(base, r < P ? (follows ? NOLIMIT : end + TAIL) : 0u, 0u, k0, k1);

    float2 acc[3][G];
#pragma unroll
    for (int c = 0; c < 3; ++c)
#pragma unroll
        for (int s = 0; s < G; ++s) acc[c][s] = make_float2(POISON, POISON);
    float2 mx = make_float2(POISON, POISON);
    uint2 best = make_uint2(0u, 0u);
    float2 sum = make_float2(0.f, 0.f);
    float4 cur[G / 2];                                           // the lines of the coming block's first step
    read_step<G, 0>(lds, k0, k1, lanebase, cur);
    // the region before the one in work, while the part that held its end waits to be added up again
    bool pending = false;
    float2 prev = make_float2(POISON, POISON);                   // its maximum without that part
    unsigned e0 = 0u, e1 = 0u, pold = 0u;                        // the part's index bytes; how many of its positions are the region's

    while (true) {
        const bool active = r < P;
        if (!__any(active)) break;
        const unsigned fin = end + TAIL;                         // the first step at which nothing of the region completes any more
        const bool closes = fin <= s0 + STEPS;                   // the region's last position completes in this block
        const bool splits = closes && follows, stops = closes && !follows;
        // the next block's indices travel while this block computes
        unsigned n0, n1;
        if (stops) fetch(a1, r1 < P ? rows1 + TAIL : 0u, 0u, n0, n1);
        else fetch(base + s0 + STEPS, follows ? NOLIMIT : fin, s0 + STEPS, n0, n1);
        float2 part[NP];
#pragma unroll
        for (unsigned h = 0; h < NP; ++h) part[h] = make_float2(POISON, POISON);
        scan_steps<G, M_MAX, 0, true>(lds, k0, k1, n0, n1, acc, mx, best, sum, lanebase, 0u, cur, part);
        k0 = n0;
        k1 = n1;
        float2 mx2 = make_float2(POISON, POISON);                // what completed of the region that follows
        unsigned hb = NP, rem = 0u;                              // the part that holds the region's end; how many of its positions are the region's
        // (the flag passes through an empty asm statement: knowing it ahead of the block, the compiler would make a second
        // copy of the whole unrolled block for the rare case and run out of registers where the two meet)
        unsigned split_at = splits ? fin - s0 : 0u;
        asm volatile("" : "+v"(split_at));
        if (__any(split_at != 0u)) {
            if (split_at != 0u) { hb = split_at / PP; rem = split_at - hb * PP; }
#pragma unroll
            for (unsigned h = 0; h < NP; ++h) {
                const bool before = h < hb, after = h > hb || (h == hb && rem == 0u);
                mx.x = fmaxf(mx.x, before ? part[h].x : POISON); mx.y = fmaxf(mx.y, before ? part[h].y : POISON);
                mx2.x = fmaxf(mx2.x, after ? part[h].x : POISON); mx2.y = fmaxf(mx2.y, after ? part[h].y : POISON);
            }
        } else {
#pragma unroll
            for (unsigned h = 0; h < NP; h += 2) { mx.x = fmaxf(fmaxf(mx.x, part[h].x), part[h + 1].x); mx.y = fmaxf(fmaxf(mx.y, part[h].y), part[h + 1].y); }
        }
        if (closes) {
            const unsigned f = f0 + (lane & 15u) * 2;
            if (pending) {
                // the region before: the part that held its end, position by position, between it and this one; then out
                if (pold != 0u) readd_part<G, 0>(lds, e0, e1, lanebase, pold, prev, mx);
                float* out = pooled + (size_t)(r - 1u) * F + f;
                if (f + 0 < F) out[0] = fmaxf(prev.x, 0.f);
                if (f + 1 < F) out[1] = fmaxf(prev.y, 0.f);
                pending = false;
            }
            if (splits) {
                // the run goes on: this region waits for the part that holds its end; what completed of the next is its start
                pending = true;
                prev = mx;
                pold = rem;
                if (rem != 0u) {
                    const size_t text = (size_t)base + s0 + hb * PP - TAIL;
                    e0 = K[text + q16] * KSTRIDE;
                    e1 = K[text + 16u + q16] * KSTRIDE;
                }
                mx = mx2;
                end += rows1;
                s0 += STEPS;
            } else {
                // ReLU and store this lane's two of the region's 32 pooled features; a fresh start
                if (active) {
                    float* out = pooled + (size_t)r * F + f;
                    if (f + 0 < F) out[0] = fmaxf(mx.x, 0.f);
                    if (f + 1 < F) out[1] = fmaxf(mx.y, 0.f);
                }
                mx = make_float2(POISON, POISON);
#pragma unroll
                for (int c = 0; c < 3; ++c)
#pragma unroll
                    for (int s = 0; s < G; ++s) acc[c][s] = make_float2(POISON, POISON);
                base = a1; end = rows1; s0 = 0u;
            }
            r = r1; rows = rows1;
            r1 = take();
            bounds(r1, a1, rows1);
            follows = r1 == r + 1u && r1 < P && a1 == base + end && rows1 >= FOLLOW_ROWS && rows >= STEPS;
        } else {
            s0 += STEPS;
        }
    }
}

template <int G, int MAXT, int MODE>
__global__ __launch_bounds__(MAXT) __attribute__((amdgpu_waves_per_eu(3, 3))) void scanpool_kmer_kernel(const float* __restrict__ W, const float* __restrict__ bias,
                                                            unsigned m, unsigned F, const uint8_t* __restrict__ K, size_t N,
                                                            const uint32_t* __restrict__ R, unsigned P, unsigned nsplit,
                                                            const unsigned* __restrict__ flag, float* __restrict__ pooled,
                                                            uint32_t* __restrict__ argmax)
{
    extern __shared__ __align__(16) unsigned char smem[];
    if (flag[0] != 0) return;                                   // the general kernel takes this call
    float* lut = reinterpret_cast<float*>(smem);
    float* w5 = lut + (size_t)(NKMER + 1) * G * FTILE;         // [3G taps][5 letters][32 filters]
    unsigned* counter = reinterpret_cast<unsigned*>(w5 + (size_t)3 * G * 5 * FTILE);
    const unsigned split = blockIdx.x % nsplit, tile = blockIdx.x / nsplit;
    const unsigned f0 = tile * FTILE;
    // this workgroup's regions
    const unsigned lo = (unsigned)((unsigned long long)P * split / nsplit), hi = (unsigned)((unsigned long long)P * (split + 1) / nsplit);
    if (threadIdx.x == 0) counter[0] = lo;
    build_table<G>(lut, w5, W, bias, m, F, f0);
    // Plain max pooling with filters of up to 18 taps walks through regions that follow each other (16 % faster at 101 nt
    // x 16 taps, 7 % at 500 nt). At 19-24 taps the ring's 48 registers and the 32 of the read-ahead leave no room for the
    // run's bookkeeping at three waves per SIMD (the compiler spills ~140 registers, the table lines it has just read
    // among them), and the read-ahead is worth more there than the drain it would save; there two regions that follow each
    // other are scanned as one stretch, which needs no branch beside the block (1.3 % at 500 nt, 5 % at 101 nt).
    // (eight regions per claim where every stream gets at least four claims; fewer on small calls, so that no stream idles;
    // pairs where every stream gets at least two)
    const unsigned per_stream = (hi - lo) / (blockDim.x >> 4), run = per_stream >= 32u ? 8u : (per_stream >= 4u ? per_stream / 4u : 1u);
    if constexpr (MODE == M_MAX && G <= 6) table_scan_runs<G>(reinterpret_cast<const char*>(smem), F, f0, K, R, counter, run, hi, pooled);
    else if constexpr (!(MODE & M_ARG)) table_scan_pairs<G, MODE>(reinterpret_cast<const char*>(smem), F, f0, K, R, counter, per_stream >= 4u ? 2u : 1u, hi, pooled);
    else table_scan<G, MODE>(reinterpret_cast<const char*>(smem), F, f0, K, R, counter, hi, pooled, argmax);
}

template <int G, int MODE>
int launch_mode(hipStream_t st, unsigned nwave, unsigned grid, size_t smem, const float* W, const float* bias, size_t m, size_t F,
                const uint8_t* K, size_t N, const uint32_t* R, size_t P, unsigned nsplit, const unsigned* flag, float* pooled,
                uint32_t* argmax)
{
    auto kern = scanpool_kmer_kernel<G, 768, MODE>;
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(nwave * 64), smem, st, W, bias, (unsigned)m, (unsigned)F, K, N, R,
                       (unsigned)P, nsplit, flag, pooled, argmax);
    return 0;
}

template <int G>
int launch(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* K, size_t N,
           const uint32_t* R, size_t P, const unsigned* flag, int ptype, float* pooled, uint32_t* argmax)
{
    size_t smem = ((size_t)(NKMER + 1) * G * FTILE + (size_t)3 * G * 5 * FTILE) * sizeof(float) + 16;   // table, letter weights, region counter
    if (smem > dbk_scan::lds_limit()) return -1;
    const unsigned ntile = dbk::divup(F, FTILE);
    unsigned nsplit = 256u / ntile;
    if (nsplit < 1) nsplit = 1;
    // 12 waves (3 per SIMD) measured fastest on MI355X: 8 leave LDS latency exposed, 16 add nothing.
    const unsigned nwave = 12;
    while (nsplit > 1 && (size_t)(nsplit - 1) * nwave * 4 >= P) --nsplit;       // no more streams than regions
    const unsigned grid = ntile * nsplit;
#define DBK_GO(MODE) return launch_mode<G, MODE>(st, nwave, grid, smem, W, bias, m, F, K, N, R, P, nsplit, flag, pooled, argmax)
    if (ptype == DBK_PT_MAX) { if (argmax) DBK_GO(M_MAX | M_ARG); DBK_GO(M_MAX); }
    if (ptype == DBK_PT_ALL) { if (argmax) DBK_GO(M_MAX | M_SUM | M_ARG); DBK_GO(M_MAX | M_SUM); }
    DBK_GO(M_SUM);
#undef DBK_GO
}

// Whether a call of this size goes to the table kernel when the choice is left to the library: building the tables and
// the index pre-pass make the smallest call ~36 us, which only bulk work repays. From 9 taps on the general path scans on
// the matrix cores and stays ahead for longer. Measured break-even on 101 nt sequences x 8 tiles, in rows x tiles:
// 9 and 12 taps ~2 M (0.028 ms either way), 16, 20 and 24 taps ~4 M (0.053-0.066 ms either way); at 8 M the table
// kernel is 10-40 % ahead, and about twice as fast per row once its tables are built.
bool takes(size_t m, size_t F, size_t N, size_t P)
{
    if (m > 24 || N == 0 || N > 0x7fffff00u || P > 0x7fff0000u) return false;
    return (double)N * dbk::divup(F, FTILE) >= (m > 12 ? 4.0e6 : 2.0e6);
}

// Bytes of device scratch a call over N sequence bytes needs: the flag word's 256-byte line, then the index bytes.
inline size_t scratch_bytes(size_t N) { return 256 + ((N + KPAD + 255) & ~(size_t)255); }

// force: take the fast path whenever the shape allows, regardless of problem size.
// ws: device scratch of scratch_bytes(N) bytes the caller provides, or null to take the stream's grow-on-demand buffer.
int fprop_impl(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
               const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax, bool force, unsigned char* ws = nullptr)
{
    if (ptype != DBK_PT_MAX && ptype != DBK_PT_AVG && ptype != DBK_PT_ALL) return -1;
    if (ptype == DBK_PT_AVG && argmax != nullptr) return -1;
    if (m > 24 || N == 0 || N > 0x7fffff00u || P > 0x7fff0000u) return -1;
    if (!force && !takes(m, F, N, P)) return -1;
    if (!ws) {
        ws = (unsigned char*)dbk::workspace(scratch_bytes(N), st);
        if (!ws) { dbk::set_error("MemoryError: could not allocate %zu bytes of scratch (%s)", scratch_bytes(N), dbk::workspace_error()); return 1; }
    }
    unsigned* flag = (unsigned*)ws;
    uint8_t* K = ws + 256;
    const size_t ndef = N + 1 >= m + 1 ? N - m + 1 : 0;          // rows the scan defines
    hipLaunchKernelGGL(clear_flag_kernel, dim3(1), dim3(1), 0, st, flag);
    hipLaunchKernelGGL(kmer_index_kernel, dim3(dbk::ew_grid((N + KPAD) / 4 + 1)), dim3(256), 0, st, X, N, K, flag, R, P, ndef);
    int G = (int)((m + 2) / 3);
    G += G & 1;
    int rc;
    switch (G) {
    case 2: rc = launch<2>(st, W, bias, m, F, K, N, R, P, flag, ptype, pooled, argmax); break;
    case 4: rc = launch<4>(st, W, bias, m, F, K, N, R, P, flag, ptype, pooled, argmax); break;
    case 6: rc = launch<6>(st, W, bias, m, F, K, N, R, P, flag, ptype, pooled, argmax); break;
    default: rc = launch<8>(st, W, bias, m, F, K, N, R, P, flag, ptype, pooled, argmax); break;
    }
    if (rc != 0) return rc;
    // inputs the table cannot express (code 254, regions outside the sequence): the general kernel
    // runs instead, gated on the same device flag so that no host synchronisation is needed
    rc = dbk_scanpool_general::fprop(st, W, bias, m, F, X, N, R, P, ptype, pooled, argmax, flag, nullptr);
    return rc;
}

int fprop(hipStream_t st, const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
          const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax)
{
    return fprop_impl(st, W, bias, m, F, X, N, R, P, ptype, pooled, argmax, false);
}

// ---- scratch that is part of the loaded code object, for callers that must not allocate ------------------
// Every device the library runs on holds its own copy of this array, at its own address, from the moment the code
// object is loaded there until the process ends. The array's name is a host-side handle, not a device address:
// host code asks the runtime for the address once per device and passes that pointer to the kernels.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t(64) << 20) + 512;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
static unsigned char* g_static_scratch[64] = {nullptr};
static std::mutex g_static_scratch_mutex;

// Address of the current device's copy of `scratch` (looked up on the first call per device); null on failure.
static unsigned char* static_scratch()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { dbk::set_error("RuntimeError: no current device below 64"); return nullptr; }
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (!g_static_scratch[dev]) {
        unsigned char* p = nullptr;
        hipError_t e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            dbk::set_error("RuntimeError: hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_static_scratch[dev] = p;
    }
    return g_static_scratch[dev];
}

}  // namespace dbk_scanpool_kmer

extern "C" int dbk_scanpool_fprop_kmer_static(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                                              const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                                              float* pooled, uint32_t* argmax)
{
    using namespace dbk_scanpool_kmer;
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    if (nfilter == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && regions && pooled, "ValueError: null pointer argument");
    DBK_CHECK(!(argmax && ptype == DBK_PT_AVG), "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    DBK_CHECK(!argmax || (double)N * (double)nfilter <= 4294967296.0,
              "ValueError: %zu rows x %zu filters overflow the 32-bit argmax index; score in smaller batches or without argmax", N, nfilter);
    DBK_CHECK(scratch_bytes(N) <= STATIC_SCRATCH_BYTES,
              "ValueError: %zu sequence bytes need %zu bytes of scratch, the built-in buffer holds %zu (at most %zu sequence bytes per call); "
              "score in smaller batches or call dbk_scanpool_fprop_kmer", N, scratch_bytes(N), STATIC_SCRATCH_BYTES,
              STATIC_SCRATCH_BYTES - 256 - KPAD - 255);
    unsigned char* ws = static_scratch();
    if (!ws) return 2;
    // The flag word and the index bytes are rewritten from the inputs by the call's first two launches, so
    // nothing of an earlier call's contents is read.
    int rc = fprop_impl(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax, true, ws);
    DBK_CHECK(rc >= 0, "NotImplementedError: the k-mer table path takes max / avg / all pooling and filter length <= 24");
    return rc;
}

extern "C" int dbk_scanpool_fprop_kmer(dbk_stream_t stream, const float* W, const float* bias, size_t m, size_t nfilter,
                                       const uint8_t* X, size_t N, const uint32_t* regions, size_t nregion, int ptype,
                                       float* pooled, uint32_t* argmax)
{
    DBK_CHECK(m >= 1, "ValueError: filter length must be >= 1");
    if (nfilter == 0 || nregion == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(W && bias && X && regions && pooled, "ValueError: null pointer argument");
    DBK_CHECK(!(argmax && ptype == DBK_PT_AVG), "ValueError: pooledmaps_argmax can only be used for max/all pooling.");
    DBK_CHECK(!argmax || (double)N * (double)nfilter <= 4294967296.0,
              "ValueError: %zu rows x %zu filters overflow the 32-bit argmax index; score in smaller batches or without argmax", N, nfilter);
    int rc = dbk_scanpool_kmer::fprop_impl(dbk::as_stream(stream), W, bias, m, nfilter, X, N, regions, nregion, ptype, pooled, argmax, true);
    DBK_CHECK(rc >= 0, "NotImplementedError: the k-mer table path takes max / avg / all pooling and filter length <= 24");
    return rc;
}

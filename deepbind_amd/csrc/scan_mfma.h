// The fused forward pass (scan + bias + rectifier + pooling) on the matrix cores, for batches of many regions.
//
// The scan is a product: Z (positions x filters) = H (positions x 4m) . W (4m x filters), H holding for every
// position the one-hot letters of its window (row 4*tap + letter of W is the weight of that letter at that tap;
// code 255 and any other non-letter put 1/4 in all four rows of the tap, code 254 nothing). 0, 1 and 1/4 are exact
// in bf16 and a float32 weight is exactly the sum of three bf16 numbers (8 + 8 + 8 significant bits), so
// Z = H.W_lo + H.W_mid + H.W_hi with exact products, accumulated in float32 by v_mfma_f32_32x32x16_bf16: the
// same sum the lookup kernels form, in another order (agreement to round-off, not bit for bit).
//
// A wave owns 32 filters of its workgroup's 64-filter tile (the three bf16 pieces of their weights stay in
// registers, 12 per 16 rows of W) and walks regions in blocks of 32 positions: the block's letters go through LDS,
// each lane turns its two letters per k-step into the four one-hot registers with a 256-entry table, 3 * ceil(4m/16)
// matrix instructions give 32 x 32 sums, and the bias / rectifier / pooling / activity masks read them from the
// accumulator layout (lane = filter, 16 registers = rows (i & 3) + 8 * (i >> 2) + 4 * (lane >> 5)).
// reference chain: kangaroo/_ext/corr1ord.py:97-117, deepity/std/elemwise.py:71-82,162-180, kangaroo/_ext/poolrgn.py:56-76
#pragma once
#include "mfma_common.h"

namespace dbk_scanpool_general {

using namespace dbk_mfma;

constexpr unsigned MFMA_ROWS = 32;                                // positions per block
constexpr unsigned MFMA_CHUNK = 192;                              // rows whose letters a wave stages at a time: six blocks
constexpr unsigned MFMA_XBYTES = 256;                             // a chunk's positions: 192 rows + a window of up to 32 taps (last read: 160 + 31 + 2 + 28), four per lane
constexpr size_t MFMA_SMEM = 256 * 8 + 32 * 16 + 4 * 2 * MFMA_XBYTES * 16;   // letter table + 32 empty entries + four waves' one-hot tables, two chunks each
inline unsigned mfma_ksteps(size_t m) { return (unsigned)((4 * m + 15) / 16); }
inline bool mfma_takes(size_t m) { return m >= 1 && m <= 32; }

// The words of eight ballots into the lanes that carry their rows' numbers. Register I of the accumulator holds row
// (I & 3) + 8 * (I >> 2) in lanes 0-31 and that row + 4 in lanes 32-63, so ballot I's low word belongs in lane
// (I & 3) + 8 * (I >> 2) and its high word four lanes on. One v_writelane_b32 per word (the compiler's own form
// compares the lane number every time, or keeps 32 masks alive in scalar registers). The wait states come first:
// the scalar registers were written by vector compares, which the assembler does not see from inside the block.
template <int I0>
__device__ __forceinline__ unsigned ballots_to_lanes(unsigned v, const unsigned long long (&open)[8])
{
#define DBK_LO(k) "s"((unsigned)open[k])
#define DBK_HI(k) "s"((unsigned)(open[k] >> 32))
    asm("s_nop 4\n\t"
        "v_writelane_b32 %0, %1, %17\n\tv_writelane_b32 %0, %2, %18\n\t"
        "v_writelane_b32 %0, %3, %19\n\tv_writelane_b32 %0, %4, %20\n\t"
        "v_writelane_b32 %0, %5, %21\n\tv_writelane_b32 %0, %6, %22\n\t"
        "v_writelane_b32 %0, %7, %23\n\tv_writelane_b32 %0, %8, %24\n\t"
        "v_writelane_b32 %0, %9, %25\n\tv_writelane_b32 %0, %10, %26\n\t"
        "v_writelane_b32 %0, %11, %27\n\tv_writelane_b32 %0, %12, %28\n\t"
        "v_writelane_b32 %0, %13, %29\n\tv_writelane_b32 %0, %14, %30\n\t"
        "v_writelane_b32 %0, %15, %31\n\tv_writelane_b32 %0, %16, %32"
        : "+v"(v)
        : DBK_LO(0), DBK_HI(0), DBK_LO(1), DBK_HI(1), DBK_LO(2), DBK_HI(2), DBK_LO(3), DBK_HI(3),
          DBK_LO(4), DBK_HI(4), DBK_LO(5), DBK_HI(5), DBK_LO(6), DBK_HI(6), DBK_LO(7), DBK_HI(7),
          "n"(2 * I0 + 0), "n"(2 * I0 + 4), "n"(2 * I0 + 1), "n"(2 * I0 + 5), "n"(2 * I0 + 2), "n"(2 * I0 + 6), "n"(2 * I0 + 3), "n"(2 * I0 + 7),
          "n"(2 * I0 + 8), "n"(2 * I0 + 12), "n"(2 * I0 + 9), "n"(2 * I0 + 13), "n"(2 * I0 + 10), "n"(2 * I0 + 14), "n"(2 * I0 + 11), "n"(2 * I0 + 15));
#undef DBK_LO
#undef DBK_HI
    return v;
}

// max(a, b) as one instruction (the compiler's fmaxf first quiets a possible signalling NaN with an instruction of its own)
__device__ __forceinline__ float plain_max(float a, float b)
{
    float r;
    asm("v_max_f32_e32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// One block of 32 rows as the wave walks its regions: where its one-hot letters lie, and what the pooling needs to know.
struct mfma_block {
    const uint4* hot;         // the block's first position in the chunk's one-hot table
    size_t r;                 // region
    unsigned a, b, c0;        // the region's bounds, the block's first row
    bool valid;
};

template <int PT, bool WANT_ARGMAX, bool ACT, int KS>
__device__ __forceinline__ void scanpool_fprop_mfma_body(const wg_t wg, const float* __restrict__ W, const float* __restrict__ bias,
                                                         unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                         const uint32_t* __restrict__ R, size_t P,
                                                         float* __restrict__ pooled, uint32_t* __restrict__ argmax,
                                                         unsigned long long* __restrict__ act)
{
    extern __shared__ __align__(16) unsigned char smem[];
    uint2* onehot = reinterpret_cast<uint2*>(smem);               // [256]: the four bf16 of a letter code's rows
    const unsigned lane = threadIdx.x & 63, wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned col = lane & 31, g = lane >> 5;
    const unsigned fb = wave & 1u, stream = wave >> 1;            // which half of the tile; which of the workgroup's two region streams
    uint4* nothing = reinterpret_cast<uint4*>(smem + 256 * 8);    // 32 all-zero entries: the window of a row the scan does not define
    uint4* hotw = nothing + 32 + (size_t)wave * (2 * MFMA_XBYTES);   // this wave's one-hot tables: the chunk in work, the next one
    {
        const unsigned c = threadIdx.x, one = 0x3f80u, quarter = 0x3e803e80u;
        uint2 e;
        if (c < 4u) { e.x = c == 0u ? one : (c == 1u ? one << 16 : 0u); e.y = c == 2u ? one : (c == 3u ? one << 16 : 0u); }
        else if (c == 254u) { e.x = 0u; e.y = 0u; }
        else { e.x = quarter; e.y = quarter; }
        if (c < 256u) onehot[c] = e;
        if (c < 32u) nothing[c] = make_uint4(0u, 0u, 0u, 0u);
    }
    // ---- the first regions' bounds and letters are on their way while the weights are prepared
    const size_t stride = (size_t)wg.gx * 2;
    size_t r = (size_t)wg.x * 2 + stream, rn = r + stride;
    unsigned a = 0u, b = 0u, an = 0u, bn = 0u;
    if (r < P) { a = R[2 * r]; b = R[2 * r + 1]; }
    if (rn < P) { an = R[2 * rn]; bn = R[2 * rn + 1]; }
    a = (unsigned)__builtin_amdgcn_readfirstlane((int)a); b = (unsigned)__builtin_amdgcn_readfirstlane((int)b);
    unsigned letters = load_letters4(X, N, (size_t)a + 4u * lane);
    // ---- this lane's column of W, rows 16s + 8g .. + 7 of every k-step, in three bf16 pieces
    const unsigned f = wg.y * FT + fb * 32u + col;
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
    // The sums leave the matrix cores without the bias b: "z + b > 0" is "z > -b", the maximum of z + b is the
    // maximum of z, plus b, and relu(z + b) = max(z, -b) + b.
    const float bf = f < F ? bias[f] : 0.0f, nb = -bf;
    const size_t n = N >= (size_t)m ? N - m + 1 : 0;              // rows the scan defines; later rows are relu(bias)
    unsigned* act32 = reinterpret_cast<unsigned*>(act);           // a tile's 64-bit word as two halves, this wave's is `fb`
    const unsigned rg = 4u * g;                                   // this half-wave's rows are 4 further down
    __syncthreads();

    // ---- the walk over the wave's blocks: region after region, a region in chunks of MFMA_CHUNK rows. A chunk's
    // letters become a table in LDS of one entry per position q: the one-hot rows of letters q and q + 1 (8 bf16), so
    // that a lane's operand for a k-step is one 16-byte read; the next chunk's letters are on their way meanwhile.
    unsigned c = a, c0 = a, buf = 0u;                             // start of the chunk in work, of the next block
    bool fresh = true;                                            // the chunk's letters are still in `letters`
    auto next_block = [&]() -> mfma_block {
        mfma_block k;
        k.valid = r < P;
        k.r = r; k.a = a; k.b = b; k.c0 = c0;
        uint4* hc = hotw + buf * MFMA_XBYTES;
        k.hot = hc + (c0 - c);
        if (!k.valid) return k;
        const bool last_chunk = b <= c || b - c <= MFMA_CHUNK;    // the region ends in this chunk
        if (fresh) {
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
            fresh = false;
            const unsigned ans = (unsigned)__builtin_amdgcn_readfirstlane((int)an);
            const unsigned cnext = last_chunk ? ans : c + MFMA_CHUNK;
            if (!last_chunk || rn < P) letters = load_letters4(X, N, (size_t)cnext + 4u * lane);
        }
        // advance
        if (b <= c0 || b - c0 <= MFMA_ROWS) {
            r = rn; rn += stride;
            a = (unsigned)__builtin_amdgcn_readfirstlane((int)an); b = (unsigned)__builtin_amdgcn_readfirstlane((int)bn);
            if (rn < P) { an = R[2 * rn]; bn = R[2 * rn + 1]; }
            c = a; c0 = a; buf ^= 1u; fresh = true;
        } else {
            c0 += MFMA_ROWS;
            if (c0 - c >= MFMA_CHUNK) { c = c0; buf ^= 1u; fresh = true; }
        }
        return k;
    };
    // a block's sums: position `col`, taps 4s + 2g and 4s + 2g + 1 of every k-step
    auto scan_block = [&](const mfma_block& k) -> f32x16_t {
        const uint4* hot = (size_t)k.c0 + col < n ? k.hot + col + 2u * g : nothing;
        f32x16_t acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const uint4 A = hot[4 * s];
#pragma unroll
            for (int q = 0; q < 3; ++q)
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, A), __builtin_bit_cast(bf16x8_t, B[s][q]), acc, 0, 0, 0);
        }
        return acc;
    };

    float mz = 0.0f, sum = 0.0f;                                  // running maximum of the rectified values, their sum
    unsigned xi = 0u;                                             // row of the maximum, relative to a
    // rectifier, pooling over this lane's 16 rows (ascending), activity masks
    auto pool_block = [&](const mfma_block& k, const f32x16_t& acc) {
        const unsigned rows = k.b > k.c0 ? k.b - k.c0 : 0u;        // rows of the region from c0 on
        float z[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) z[i] = acc[i];
        if (rows < MFMA_ROWS) {
            // the region's last block: a row past the region is given -b, where it is closed, cannot win and adds nothing
#pragma unroll
            for (int i = 0; i < 16; ++i) z[i] = rg + ((i & 3) + 8 * (i >> 2)) < rows ? z[i] : nb;
        }
        if (ACT) {
            unsigned mine = 0u;
            unsigned long long open[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) open[i] = __ballot(z[i] > nb);
            mine = ballots_to_lanes<0>(mine, open);               // registers 0-7: rows 0-15
#pragma unroll
            for (int i = 0; i < 8; ++i) open[i] = __ballot(z[8 + i] > nb);
            mine = ballots_to_lanes<8>(mine, open);               // registers 8-15: rows 16-31
            if (lane < rows && lane < MFMA_ROWS) act32[((size_t)(k.c0 + lane) * wg.gy + wg.y) * 2 + fb] = mine;
        }
        if (PT != DBK_PT_AVG) {
            float bm = z[0];
            unsigned bi = 0u;
#pragma unroll
            for (int i = 1; i < 16; ++i) {
                const bool gt = z[i] > bm;
                bm = gt ? z[i] : bm;
                bi = gt ? (unsigned)i : bi;
            }
            bm += bf;
            if (bm > mz) { mz = bm; xi = (k.c0 - k.a) + rg + (bi & 3u) + 8u * (bi >> 2); }
        }
        if (PT != DBK_PT_MAX) {
            float part = 16.0f * bf;
#pragma unroll
            for (int i = 0; i < 16; ++i) part += plain_max(z[i], nb);
            sum += part;
        }
        if (rows <= MFMA_ROWS) {
            // ---- the region's last block. Fold the two half-waves: larger value wins, equal values keep the earlier row
            const float vm = __shfl_xor(mz, 32, 64);
            const unsigned vi = (unsigned)__shfl_xor((int)xi, 32, 64);
            const float vs = __shfl_xor(sum, 32, 64);
            if (vm > mz || (vm == mz && vi < xi)) { mz = vm; xi = vi; }
            sum += vs;
            if (g == 0 && f < F) {
                const size_t j = k.r * F + f;
                if (PT == DBK_PT_MAX) pooled[j] = mz;
                else if (PT == DBK_PT_AVG) pooled[j] = sum / (float)(k.b - k.a);
                else { pooled[2 * j] = mz; pooled[2 * j + 1] = sum / (float)(k.b - k.a); }
                if (WANT_ARGMAX && PT != DBK_PT_AVG) argmax[j] = (uint32_t)(((size_t)k.a + xi) * F + f);
            }
            mz = 0.0f; sum = 0.0f; xi = 0u;
        }
    };

    // (Matrix and vector instructions do not overlap on a SIMD: issuing the next block's products before this block's
    // pooling gains nothing, so the blocks are simply taken one after the other; other waves fill the LDS latency.)
    for (mfma_block cur = next_block(); cur.valid; cur = next_block()) {
        const f32x16_t acc = scan_block(cur);
        pool_block(cur, acc);
    }
}

template <int PT, bool WANT_ARGMAX, bool ACT, int KS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void scanpool_fprop_mfma_kernel(const float* __restrict__ W, const float* __restrict__ bias,
                                                                  unsigned m, unsigned F, const uint8_t* __restrict__ X, size_t N,
                                                                  const uint32_t* __restrict__ R, size_t P,
                                                                  float* __restrict__ pooled, uint32_t* __restrict__ argmax,
                                                                  unsigned long long* __restrict__ act)
{
    scanpool_fprop_mfma_body<PT, WANT_ARGMAX, ACT, KS>(this_wg(), W, bias, m, F, X, N, R, P, pooled, argmax, act);
}

}  // namespace dbk_scanpool_general

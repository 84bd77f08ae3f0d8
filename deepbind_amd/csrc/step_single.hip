// One whole optimiser step of a SMALL model group in ONE launch.
//
// A training step on a minibatch of a hundred short sequences and one to four models is a few million
// additions: issued as forward / head / backward / update launches it costs what four dependent launches
// cost (30-40 us), and a 64-filter tile leaves most lanes of a wave idle when the group has 16 filters.
// Here a workgroup takes a few regions (sequences) of the batch through the WHOLE step without leaving the
// CU - scan + bias + ReLU + pooling, the dense head forward and backward, the filter gradients - writes its
// share of every parameter's gradient to a partial-sum buffer, and after ONE grid-wide barrier all
// workgroups together add up the shares in a fixed order and apply the Nesterov update. Nothing but the
// partial sums and the predictions goes through HBM.
//
//   lanes        a wave's 64 lanes are (64 / Fp) position groups x Fp filters (Fp = 16, 32 or 64 = the
//                group's filters rounded up), so a single 16-filter model keeps all lanes busy: every
//                position group scans its own contiguous block of a region's positions, four positions at a
//                time, the block's letters sliding through registers (one LDS word per four positions)
//   forward      z[p][f] = sum over taps of table[tap][letter(p + tap)][f], taps ascending (the order of the
//                reference kernel, kangaroo_smat/corr1ord.cuh:139-157), + bias, ReLU, running max / first
//                argmax / sum per lane, folded over position groups and waves (poolrgn.cuh:44-160)
//   head         dropout (the library generator, same element numbering as dbk_dropout_fp_tr) -> dense
//                (+ shared feature columns) -> bias [-> ReLU -> dense -> bias] -> logistic | identity ->
//                dA = (Z - Y) / n with Ymask and the reverse-complement pair rule -> gradients
//                (deepity/std/full.py:78-178, loss.py:98-119, dropout.cu:41-109)
//   backward     a thread owns (tap, filter) pairs and keeps their five letter accumulators (A, C, G, T,
//                "mean of the four") in registers over the workgroup's regions. The average-pooling part
//                needs no pass over the positions: the gradient is the same number c = dpooled / rows at every
//                position whose rectifier is open, so dW[tap][letter][f] += c * popcount(open(f) & letters
//                (letter) >> tap) with one bit per position (the rectifier bits are left by the forward pass,
//                the letter bits by the staging). The max-pooling part adds the pooled gradient at the argmax
//                row's letters (corr1ord_bprop.cuh:91-137, poolrgn_bprop.cuh:45-127)
//   update       g = sum of the workgroups' shares: a workgroup takes 64 consecutive parameters, each of its waves
//                adds a run of workgroups in ascending order (one contiguous load per wave and workgroup), a fixed
//                tree adds the waves' sums; + L1 term, frozen filters zeroed,
//                Nesterov step from the look-ahead P + mrate * mP (gradstep.cu:41-72, full.py:111-119,
//                corr1ord.py:120-138)
//
// The barrier is a set of flags in the caller's workspace; every workgroup of the grid must be resident, so
// the grid never exceeds 256 workgroups of at most 512 threads, nor the device's number of CUs (a CU holds at least
// one), and the wait is bounded. Whether a launch steps or is abandoned (a workgroup waited too long, a region has too
// many rows) is settled once for the whole grid by a compare-and-swap on one word (see grid_barrier): an abandoned
// launch changes no parameter, sets the workspace's status word, and every later launch on that workspace does
// nothing until the host has zeroed the workspace's header again.
// Results are deterministic (no float atomics; LDS atomics only OR bits), within the tolerances of the
// multi-launch step but not its bits (other summation orders).
#include <type_traits>
#include "dbk_common.h"
#include "rng.h"
#include "scan_common.h"

namespace {

using dbk_scan::NL;
using dbk_scan::letter_of;
using dbk::small_div;

constexpr int NTMIN = 256, NTMAX = 512, NWMAX = NTMAX / 64;    // threads of a workgroup: 256, or 512 when it has a single region
constexpr unsigned MAXROWS = 256;                 // rows of one region
constexpr unsigned AW = MAXROWS / 32;             // words of rectifier bits per (region, filter)
constexpr unsigned LW = AW + 2;                   // words of letter bits per (region, letter): rows + taps - 1 positions
constexpr unsigned TXTB = 384;                    // staged letters per region (a dword-aligned copy, padded with "nothing")
constexpr unsigned MAXG = 256;                    // workgroups of a launch (all resident at once: a CU holds at least one)
constexpr size_t WORK_HEADER = 32768;              // bytes of the workspace before the shares: launch number, status, "go", flags, pair words
constexpr unsigned GO_AT = 32, FLAGS_AT = 64;     // words of the workspace: the "go" word; the first workgroup flag
constexpr unsigned PAIR_AT = 2048;                // ... the predictions that the two workgroups of a (forward, reverse) pair show each other: [workgroup][model] 8 bytes
constexpr unsigned FLAG_STRIDE = 4;               // words from one workgroup's flag to the next (measured: 4 beats 1 and 16 by ~0.1 us per step)
constexpr unsigned SPIN_LIMIT = 400000;           // polls of the barrier before a workgroup gives up (~0.2 s)

// LDS carve-up (all offsets in 4-byte words), computed on the host for the launch size and handed to the kernel.
struct lds_map {
    unsigned wt, look, Y, Ym, misc, text, lmask, amask, PL, arg, gmax, cavg, rows, red, H0, H1, D1, dA, ls, zs, kept, total;
};
struct single_args {
    unsigned nmodel, nfilter, F, Fp, lgFp, m, hidden, h1, k, kt, kf, ptype, loss_kind, revcomp;
    unsigned RC, G;                               // regions per workgroup, workgroups
    unsigned nparam, pstride;                     // parameters; floats of one workgroup's share (nparam + nmodel, padded)
    float *P, *dP, *mP;
    const float *drate, *mrate, *decay;
    unsigned off_Wc, off_bc, off_W1, off_b1, off_W2, off_b2;
    const uint8_t* X; unsigned N;                 // (fewer than 2^32 - 256 rows: checked on the host)
    const uint32_t* R; unsigned nregion;
    const float* Y; const uint8_t* Ymask; const float* feats;
    const float* rate; unsigned long long seed; unsigned long long* counter; unsigned long long draws;
    int freeze_scan;
    float *Z, *loss;
    unsigned* sync;                               // [0] number of the last launch, [1] status (non-zero: see grid_barrier), [64..] flags
    float* partial;                               // [G][pstride]
    lds_map L;
};

inline lds_map make_map(unsigned MT, unsigned Fp, unsigned nm, unsigned kt, unsigned k, unsigned h1, unsigned nparam,
                                            unsigned RC, bool dense)
{
    lds_map o;
    unsigned at = 0;
    auto take = [&](unsigned n) { const unsigned r = at; at += (n + 3u) & ~3u; return r; };
    o.wt = take(MT * NL * Fp);
    o.look = take(nparam);                        // the whole look-ahead vector: the dense layers are read from it in place
    o.Y = take(RC * nm);
    o.Ym = take(RC * nm);
    o.misc = take(8 + nm);                        // generator position (2 words), barrier target, dropout rates
    o.text = take(RC * TXTB / 4);
    o.lmask = take(RC * 5 * LW);
    o.amask = take(dense ? RC * Fp * AW : 0);
    o.PL = take(RC * nm * k);
    o.arg = take(RC * Fp);
    o.gmax = take(RC * Fp);
    o.cavg = take(RC * Fp);
    o.rows = take(RC * 2);
    o.red = take(NWMAX * 3 * Fp);
    o.H0 = take(RC * nm * kt);
    o.H1 = take(RC * nm * h1);
    o.D1 = take(RC * nm * h1);
    o.dA = take(RC * nm);
    o.ls = take(RC * nm);
    o.zs = take(RC * nm);
    o.kept = take((RC * nm * k + 3) / 4);
    o.total = at;
    return o;
}

// Scans this lane's block of positions [start, start + Bq) of a region whose letters are staged at tw (dword view,
// dword 0 = the region's first row), four positions per round. rows: positions of the region; row0: the region's
// first row in X; nscan: rows of X the scan defines (later rows read as bias only).
template <int MT>
__device__ __forceinline__ void scan_block(const float* __restrict__ wt, const unsigned* __restrict__ tw, unsigned start, unsigned Bq,
                                           unsigned rows, unsigned row0, unsigned nscan, unsigned f, unsigned lgFp, float bf, bool want_bits,
                                           unsigned* __restrict__ abits, float& mx, unsigned& xi, float& sum)
{
    constexpr int WN = (MT + 6) / 4;                              // dwords covering the letters of four positions
    const unsigned Fp4 = 4u << lgFp;                              // bytes of one table row
    const char* lane_row = reinterpret_cast<const char*>(wt) + 4u * f;
    unsigned w[WN];
    const unsigned* src = tw + (start >> 2);
#pragma unroll
    for (int i = 0; i < WN; ++i) w[i] = src[i];
    for (unsigned j = 0; j < Bq; j += 4) {
        float z[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int t = 0; t < MT; ++t) {
#pragma unroll
            for (int ph = 0; ph < 4; ++ph) {
                const int q = ph + t;
                const unsigned letter = (w[q >> 2] >> ((q & 3) * 8)) & 0xffu;
                z[ph] += *reinterpret_cast<const float*>(lane_row + letter * Fp4 + (unsigned)t * NL * Fp4);
            }
        }
#pragma unroll
        for (int ph = 0; ph < 4; ++ph) {
            const unsigned p = start + j + ph;
            if (p < rows) {
                float v = (row0 + p < nscan ? z[ph] : 0.0f) + bf;
                const bool open = v > 0.0f;
                v = open ? v : 0.0f;
                if (v > mx) { mx = v; xi = p; }
                sum += v;
                if (want_bits && open) atomicOr(&abits[p >> 5], 1u << (p & 31));
            }
        }
#pragma unroll
        for (int i = 0; i + 1 < WN; ++i) w[i] = w[i + 1];
        w[WN - 1] = src[(j >> 2) + WN];
    }
}

// All workgroups of the grid meet here once. Accesses of many workgroups to ONE address at device scope are served
// one after the other (measured: ~50 ns per read-modify-write, 6.5 us for a counter that 128 workgroups increment;
// 2-4 us per poll when every workgroup reads every other's flag, in lines of their own or side by side), so no word is
// shared more than it must be: each workgroup raises a flag of its own; workgroup 0 alone reads all the flags (up to
// four per lane of its first wave) and, when they are all up, publishes its decision in the "go" word, which every
// other workgroup polls with one lane.
//
// Words carry the number of the launch (one more than the number the workspace held when the kernel started, 31 bits)
// so that what an earlier launch left is never taken for this one's: flag = 2 * number + (1: this workgroup must not
// update - a region too long, a partner that never answered); go = 2 * number + (1: the step is abandoned).
// Whether the grid steps or abandons is decided ONCE, by whoever first moves the "go" word from a value of an earlier
// launch to a value of this one with a compare-and-swap: workgroup 0 when it has seen all flags (go, or abandon if a
// flag says so) or has waited SPIN_LIMIT polls for them (abandon); any other workgroup that has polled the word twice
// as long (abandon: workgroup 0 is not running). Whoever loses the exchange takes the winner's value. So either every
// workgroup of the launch applies its part of the update or none does.
// Returns 0 when the step goes on, 1 when it is abandoned (the workspace's status word is then non-zero).
__device__ __forceinline__ unsigned decide(unsigned* go, unsigned seen, unsigned want, unsigned number)
{
    for (;;) {
        const unsigned old = atomicCAS(go, seen, want);
        if (old == seen) return want;
        if ((old >> 1) == number) return old;                      // decided by another workgroup
        seen = old;
    }
}

__device__ __forceinline__ unsigned grid_barrier(unsigned* sync, unsigned G, unsigned launch, bool bad)
{
    __shared__ unsigned verdict;
    unsigned* flags = sync + FLAGS_AT;
    unsigned* go = sync + GO_AT;
    const unsigned number = launch & 0x7fffffffu;
    __syncthreads();
    if (threadIdx.x < 64) {
        const unsigned lane = threadIdx.x;
        if (lane == 0) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");     // this workgroup's shares are visible device-wide
            __hip_atomic_store(&flags[blockIdx.x * FLAG_STRIDE], 2u * number + (bad ? 1u : 0u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        unsigned tries = 0, word = 0;
        if (blockIdx.x == 0) {
            bool all_up = false, any_bad = false, decided = false;
            for (;;) {
                unsigned v[MAXG / 64];
#pragma unroll
                for (unsigned u = 0; u < MAXG / 64; ++u)
                    v[u] = lane + 64u * u < G ? __hip_atomic_load(&flags[(lane + 64u * u) * FLAG_STRIDE], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 2u * number;
                if (lane == 0) word = __hip_atomic_load(go, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                bool mine = true, mine_bad = false;
#pragma unroll
                for (unsigned u = 0; u < MAXG / 64; ++u) { mine = mine && (v[u] >> 1) == number; mine_bad = mine_bad || (v[u] & 1u); }
                all_up = __all(mine);
                any_bad = __any(mine && mine_bad);
                decided = ((unsigned)__builtin_amdgcn_readfirstlane((int)word) >> 1) == number;      // (a workgroup that gave up was faster)
                if (all_up || decided || ++tries >= SPIN_LIMIT) break;
                __builtin_amdgcn_s_sleep(1);
            }
            if (lane == 0 && !decided) word = decide(go, word, 2u * number + ((all_up && !any_bad) ? 0u : 1u), number);
        } else if (lane == 0) {
            for (;;) {
                word = __hip_atomic_load(go, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((word >> 1) == number) break;
                if (++tries >= 2u * SPIN_LIMIT) { word = decide(go, word, 2u * number + 1u, number); break; }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        if (lane == 0) {
            if (word & 1u) atomicCAS(&sync[1], 0u, 1u);            // (a more specific status set before the barrier stays)
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");     // the other workgroups' shares are read from memory, not from stale lines
            verdict = word & 1u;
        }
    }
    __syncthreads();
    return verdict;
}

// Orders a wave's own LDS traffic: what its lanes stored before is what its lanes read after (the LDS serves a wave's
// instructions in order; the fences keep the compiler from moving them and wait for the counter).
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// Sum over the wave's 64 lanes, the same bits in every lane: within a row of 16 lanes by data-parallel moves (lane ^ 1,
// lane ^ 2, then the mirrored lane of the eight and of the row: it lies in the other half, and all lanes of a half
// hold the same sum by then), across the rows by two exchanges through the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float lane_move(float v) { return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true)); }
__device__ __forceinline__ float wave_sum(float v)
{
    v += lane_move<0xB1>(v);                                       // quad_perm [1, 0, 3, 2]
    v += lane_move<0x4E>(v);                                       // quad_perm [2, 3, 0, 1]
    v += lane_move<0x141>(v);                                      // row_half_mirror
    v += lane_move<0x140>(v);                                      // row_mirror
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

// A share is stored through the cache levels that other workgroups do not see (a relaxed store at device scope), on its
// way while the workgroup computes the rest: the barrier's release fence then finds little left to write back.
__device__ __forceinline__ void put_share(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// SHAPE: what of the launch shape is known when the kernel is compiled. 1: one region per workgroup of 512 threads
// (batches of at most MAXG regions). 2: that, and a single model of at most 16 filters. 3 / 4: one region per workgroup
// and 17-32 / 33-64 filters in all. 0: nothing. Whatever is known
// folds out of the index arithmetic and takes whole branches with it (the instance for shape 2 is a third as long as
// the general one), and with a step this short the instructions a wave issues one after the other are what it costs.
template <int MT, int SHAPE>
__global__ __launch_bounds__(NTMAX) void k_step_single(const single_args a)
{
    extern __shared__ __align__(16) unsigned smem[];
    const bool dense = a.ptype != DBK_PT_MAX, sparse = a.ptype != DBK_PT_AVG;
    constexpr bool ONE = SHAPE == 2;
    const unsigned nm = ONE ? 1u : a.nmodel, RC = SHAPE ? 1u : a.RC;
    const unsigned Fp = ONE ? 16u : SHAPE == 3 ? 32u : SHAPE == 4 ? 64u : a.Fp, lgFp = ONE ? 4u : SHAPE == 3 ? 5u : SHAPE == 4 ? 6u : a.lgFp;
    const lds_map& L = a.L;
    float* wt = reinterpret_cast<float*>(smem + L.wt);
    float* Lk = reinterpret_cast<float*>(smem + L.look);
    const float* W1s = Lk + a.off_W1;
    const float* b1s = Lk + a.off_b1;
    const float* W2s = Lk + a.off_W2;
    const float* b2s = Lk + a.off_b2;
    float* Ys = reinterpret_cast<float*>(smem + L.Y);
    unsigned* Yms = smem + L.Ym;
    unsigned* misc = smem + L.misc;
    float* rates = reinterpret_cast<float*>(smem + L.misc + 8);
    uint8_t* text = reinterpret_cast<uint8_t*>(smem + L.text);
    unsigned* lmask = smem + L.lmask;
    unsigned* amask = smem + L.amask;
    float* PL = reinterpret_cast<float*>(smem + L.PL);
    unsigned* argp = smem + L.arg;
    float* gmax = reinterpret_cast<float*>(smem + L.gmax);
    float* cavg = reinterpret_cast<float*>(smem + L.cavg);
    unsigned* rinfo = smem + L.rows;                               // [RC][2]: rows, first row (low 32 bits are enough: N < 2^32 checked)
    float* red = reinterpret_cast<float*>(smem + L.red);
    float* H0 = reinterpret_cast<float*>(smem + L.H0);
    float* H1 = reinterpret_cast<float*>(smem + L.H1);
    float* D1 = reinterpret_cast<float*>(smem + L.D1);
    float* dAs = reinterpret_cast<float*>(smem + L.dA);
    float* lss = reinterpret_cast<float*>(smem + L.ls);
    float* zs = reinterpret_cast<float*>(smem + L.zs);
    uint8_t* kept = reinterpret_cast<uint8_t*>(smem + L.kept);

    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, NT = SHAPE ? (unsigned)NTMAX : blockDim.x, NW = NT >> 6;
    const unsigned F = a.F, k = a.k, kt = a.kt, h1 = a.h1, hidden = a.hidden, m = a.m;
    const unsigned r0 = blockIdx.x * RC;                           // first region of this workgroup
    const unsigned nreg = r0 < a.nregion ? (a.nregion - r0 < RC ? a.nregion - r0 : RC) : 0u;
    const unsigned kpf = a.ptype == DBK_PT_ALL ? 2u : 1u;          // pooled features per filter
    const small_div by_nm(nm), by_k(k), by_nmk(nm * k), by_h1(h1), by_kt(kt), by_kf(a.kf), by_nmkf(nm * a.kf);

    // ---------------- everything this workgroup reads from global memory before the barrier, requested in one round:
    // its regions' bounds, targets, masks, dropout rates, the generator position and the look-ahead vector
    // P + mrate * mP (gradstep.cu:41-51). (Dependent round trips, not arithmetic, are what a step of this size costs.)
    {
        unsigned ra = 0, rb = 0;
        float y = 0.0f, dr = 0.0f;
        unsigned ym = 1u, c_lo = 0u, c_hi = 0u, tickets = 0u, stale = 0u;
        constexpr unsigned UN = 6;
        float vp[UN], vr[UN], vm[UN];
#pragma unroll
        for (unsigned u = 0; u < UN; ++u) {
            const unsigned e = tid + u * NT;
            const bool in = e < a.nparam;
            vp[u] = in ? a.P[e] : 0.0f;
            vr[u] = in ? a.mrate[e] : 0.0f;
            vm[u] = in ? a.mP[e] : 0.0f;
        }
        if (tid < RC && r0 + tid < a.nregion) { ra = a.R[2 * (r0 + tid)]; rb = a.R[2 * (r0 + tid) + 1]; }
        if (tid < RC * nm && r0 + by_nm.quot(tid) < a.nregion) {
            const unsigned i = (unsigned)r0 * nm + tid;
            y = a.Y[i];
            if (a.Ymask) ym = a.Ymask[i];
        }
        if (tid < nm && a.rate) dr = a.rate[tid];
        if (tid == 0) {
            if (a.counter) { const unsigned long long c = a.counter[0]; c_lo = (unsigned)c; c_hi = (unsigned)(c >> 32); }
            tickets = __hip_atomic_load(&a.sync[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            stale = __hip_atomic_load(&a.sync[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (unsigned u = 0; u < UN; ++u)
            if (tid + u * NT < a.nparam) Lk[tid + u * NT] = vp[u] + vr[u] * vm[u];
        for (unsigned e = tid + (unsigned)UN * NT; e < a.nparam; e += NT) Lk[e] = a.P[e] + a.mrate[e] * a.mP[e];      // a long parameter vector: the rest
        bool too_long = false;
        if (tid < RC) {
            unsigned rows = rb > ra ? rb - ra : 0u;
            if (rows > MAXROWS) {                                  // not a shape this kernel takes: flag it, touch nothing of the region
                atomicExch(&a.sync[1], 2u);
                rows = 0u;
                too_long = true;
            }
            rinfo[2 * tid] = rows;
            rinfo[2 * tid + 1] = ra;
        }
        if (wave == 0) too_long = __any(too_long);                 // (RC <= 16: all in the first wave)
        if (tid < RC * nm) { Ys[tid] = y; Yms[tid] = ym; }
        if (tid < nm) rates[tid] = dr;
        if (tid == 0) {
            misc[0] = c_lo; misc[1] = c_hi;
            misc[2] = tickets + 1u;                                // this launch's number (see grid_barrier)
            misc[3] = stale;                                       // the status the workspace held when this workgroup started
            misc[4] = too_long ? 1u : 0u;                          // non-zero: this workgroup's flag will ask for the step to be abandoned
        }
    }
    for (unsigned e = tid; e < RC * nm * a.kf; e += NT) {          // the shared feature columns follow each model's own inputs
        const unsigned rl = by_nmkf.quot(e), rest = by_nmkf.rem(e, rl), b = by_kf.quot(rest), j = by_kf.rem(rest, b);
        H0[(rl * nm + b) * kt + k + j] = (a.feats && rl < nreg) ? a.feats[((unsigned)r0 + rl) * a.kf + j] : 0.0f;
    }
    for (unsigned e = tid; e < RC * 5 * LW; e += NT) lmask[e] = 0u;
    if (dense)
        for (unsigned e = tid; e < RC * Fp * AW; e += NT) amask[e] = 0u;
    __syncthreads();
    if (misc[3] != 0u) {
        // A workspace that an earlier launch (or a faster workgroup of this one) flagged: nothing is stepped until the host
        // has looked at the status and zeroed the workspace's header. The flag still goes up so that nobody waits for it,
        // and workgroup 0 settles the launch as abandoned.
        if (tid == 0) {
            const unsigned number = misc[2] & 0x7fffffffu;
            __hip_atomic_store(&a.sync[FLAGS_AT + blockIdx.x * FLAG_STRIDE], 2u * number + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (blockIdx.x == 0)
                decide(a.sync + GO_AT, __hip_atomic_load(&a.sync[GO_AT], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), 2u * number + 1u, number);
        }
        return;
    }
    // ---------------- the regions' letters are requested; the letter table [tap][letter][filter] (zero rows past m) is
    // built from the look-ahead meanwhile; then the letters land dword-aligned per region, with one bit per (letter, position)
    constexpr unsigned TXN = (4 * TXTB + NTMIN - 1) / NTMIN;       // letters per thread when the workgroup has up to four regions
    const bool few = RC * TXTB <= TXN * NT;
    unsigned lt[TXN];
    auto letter_at = [&](unsigned e) -> unsigned {
        const unsigned rl = e / TXTB, q = e % TXTB;
        const unsigned rows = rinfo[2 * rl];
        const unsigned g = (unsigned)rinfo[2 * rl + 1] + q;
        return (rows && q < rows + MT - 1 && g < a.N) ? (unsigned)a.X[g] : 254u;
    };
    auto put_letter = [&](unsigned e, unsigned code) {
        const unsigned rl = e / TXTB, q = e % TXTB;
        const unsigned l = letter_of(code);
        text[e] = (uint8_t)l;
        if (l < 5u) atomicOr(&lmask[(rl * 5 + l) * LW + (q >> 5)], 1u << (q & 31));
    };
    if (few) {
#pragma unroll
        for (unsigned i = 0; i < TXN; ++i) lt[i] = tid + i * NT < RC * TXTB ? letter_at(tid + i * NT) : 254u;
    }
    for (unsigned e = tid; e < MT * Fp; e += NT) {
        const unsigned t = e >> lgFp, f = e & (Fp - 1u);
        float w0 = 0.0f, w1 = 0.0f, w2 = 0.0f, w3 = 0.0f;
        if (t < m && f < F) {
            const float* w = Lk + a.off_Wc + (unsigned)(4 * t) * F + f;
            w0 = w[0]; w1 = w[F]; w2 = w[2 * F]; w3 = w[3 * F];
        }
        float z = w0;
        z += w1;
        z += w2;
        z += w3;
        float* row = wt + (unsigned)t * NL * Fp + f;
        row[0 * Fp] = w0; row[1 * Fp] = w1; row[2 * Fp] = w2; row[3 * Fp] = w3;
        row[4 * Fp] = z * 0.25f;
        row[5 * Fp] = 0.0f;
    }
    // which pooled features the dropout keeps (element numbering of the stand-alone kernels): drawn now, while the letters travel
    {
        const unsigned ncol = (unsigned)k * nm;
        const unsigned long long off = (unsigned long long)misc[1] << 32 | misc[0];
        for (unsigned e = NT - 1u - tid; e < RC * nm * k; e += NT) {      // (the last threads first: the first ones build the table)
            const unsigned rl = by_nmk.quot(e), col = by_nmk.rem(e, rl), b = by_k.quot(col);
            const unsigned rr = (unsigned)r0 + rl;
            bool kp = true;
            if (rl < nreg && a.rate) kp = dbk_rng::uniform_at(a.seed, off, (a.revcomp ? (rr >> 1) : rr) * ncol + col) >= rates[b];
            kept[e] = kp;
        }
    }
    if (few) {
#pragma unroll
        for (unsigned i = 0; i < TXN; ++i)
            if (tid + i * NT < RC * TXTB) put_letter(tid + i * NT, lt[i]);
    } else {
        for (unsigned e = tid; e < RC * TXTB; e += NT) put_letter(e, letter_at(e));
    }
    __syncthreads();

    // ---------------- forward: scan + bias + ReLU + pooling, region by region, all four waves on one region
    const unsigned PG = 64u >> lgFp, NG = NW * PG;               // position groups per wave / per workgroup
    const unsigned lgNG4 = (NT == NTMAX ? 3u : 2u) + 6u - lgFp + 2u;                            // log2(4 * NG): NT is 256 or 512
    const unsigned f = lane & (Fp - 1), gidx = wave * PG + (lane >> lgFp);
    const float bf = f < F ? Lk[a.off_bc + f] : 0.0f;
    const unsigned nscan = a.N + 1 >= (unsigned)m + 1 ? a.N - m + 1 : 0;
    for (unsigned rl = 0; rl < nreg; ++rl) {
        const unsigned rows = rinfo[2 * rl];
        const unsigned Bq = 4u * ((rows + 4u * NG - 1u) >> lgNG4);
        const unsigned start = gidx * Bq;
        float mx = -1.0f, sum = 0.0f;
        unsigned xi = 0xffffffffu;
        if (start < rows)
            scan_block<MT>(wt, reinterpret_cast<const unsigned*>(text + rl * TXTB), start, Bq, rows, rinfo[2 * rl + 1], nscan, f, lgFp, bf,
                           dense, amask + (rl * Fp + f) * AW, mx, xi, sum);
        // fold the position groups of the wave (lanes f, f + Fp, ...): larger value wins, equal values keep the earlier row
        for (unsigned d = Fp; d < 64u; d <<= 1) {
            const float om = __shfl_xor(mx, (int)d, 64), os = __shfl_xor(sum, (int)d, 64);
            const unsigned oi = (unsigned)__shfl_xor((int)xi, (int)d, 64);
            if (om > mx || (om == mx && oi < xi)) { mx = om; xi = oi; }
            sum = (lane & d) ? os + sum : sum + os;               // lower group first, on both sides of the exchange
        }
        if (lane < Fp) {
            red[(wave * 3 + 0) * Fp + f] = mx;
            red[(wave * 3 + 1) * Fp + f] = __uint_as_float(xi);
            red[(wave * 3 + 2) * Fp + f] = sum;
        }
        __syncthreads();
        if (tid < Fp) {
            float vm[NWMAX], vs[NWMAX];
            unsigned vi[NWMAX];
#pragma unroll
            for (unsigned w = 0; w < NWMAX; ++w) {                 // all waves' values requested at once; a wave that is not there never wins and adds 0
                const bool in = w < NW;
                vm[w] = in ? red[(w * 3 + 0) * Fp + tid] : -2.0f;
                vi[w] = in ? __float_as_uint(red[(w * 3 + 1) * Fp + tid]) : 0xffffffffu;
                vs[w] = in ? red[(w * 3 + 2) * Fp + tid] : 0.0f;
            }
            float bm = vm[0], bs = vs[0];
            unsigned bi = vi[0];
#pragma unroll
            for (unsigned w = 1; w < NWMAX; ++w) {
                if (vm[w] > bm || (vm[w] == bm && vi[w] < bi)) { bm = vm[w]; bi = vi[w]; }
                bs += vs[w];
            }
            bm = bm > 0.0f ? bm : 0.0f;
            if (bi == 0xffffffffu) bi = 0u;
            argp[rl * Fp + tid] = bi;
            if (tid < F) {
                float* out = PL + (unsigned)rl * nm * k + (unsigned)tid * kpf;
                const float mean = rows ? bs / (float)rows : 0.0f;
                if (a.ptype == DBK_PT_MAX) out[0] = bm;
                else if (a.ptype == DBK_PT_AVG) out[0] = mean;
                else { out[0] = bm; out[1] = mean; }
            }
        }
        if constexpr (!ONE) __syncthreads();                       // (ONE: the wave that wrote the pooled features is the one that goes on with them)
    }

    // ---------------- dense head, forward and backward, for this workgroup's rows
    const float inv_n = 1.0f / (float)a.nregion;
    if (RC == 1u) {
        // A single region: wave b takes model b through the whole head on its own - inputs, hidden layer, prediction,
        // loss gradient, gradients of the hidden units and of the pooled features - and waits for nothing but its own
        // LDS traffic (no workgroup barrier between the steps).
        if (wave < nm) {
            const unsigned b = ONE ? 0u : wave;
            const bool live = nreg != 0u;
            if constexpr (ONE) wave_lds_sync();
            for (unsigned kk = lane; kk < k; kk += 64) H0[b * kt + kk] = (live && kept[b * k + kk]) ? PL[b * k + kk] : 0.0f;
            wave_lds_sync();
            const float* x = H0 + b * kt;
            float hv = 0.0f, w2 = 0.0f, part = 0.0f;               // lane h: hidden unit h and its output weight
            if (hidden) {
                if (lane < hidden) {
                    const float* wcol = W1s + (unsigned)b * kt * hidden + lane;
                    float sacc = 0.0f;
#pragma unroll 8
                    for (unsigned kk = 0; kk < kt; ++kk) sacc += x[kk] * wcol[kk * hidden];
                    sacc += b1s[b * hidden + lane];
                    hv = sacc > 0.0f ? sacc : 0.0f;
                    w2 = W2s[b * hidden + lane];
                    H1[b * hidden + lane] = hv;
                    part += hv * w2;
                }
            } else {
                for (unsigned kk = lane; kk < kt; kk += 64) part += x[kk] * W1s[(unsigned)b * kt + kk];
            }
            part = wave_sum(part);
            const float out = part + (hidden ? b2s[b] : b1s[b]);
            // (the logistic through the hardware's exponential and reciprocal, as the reference's kernels are built: -use_fast_math)
            const float z = a.loss_kind == 0 ? __builtin_amdgcn_rcpf(1.0f + __expf(-out)) : out;
            bool use = live && Yms[b] != 0u;
            if (a.revcomp) {
                // Of a (forward, reverse) pair of rows only the larger prediction trains; ties keep the first row. The
                // partner row is the neighbouring workgroup's: the two show each other their predictions through one
                // 8-byte word each (the number of this launch beside the value, so that a word left by the launch before
                // is not taken for it), one trip through memory. The wait is bounded like the barrier's.
                unsigned long long* words = reinterpret_cast<unsigned long long*>(a.sync + PAIR_AT);
                const unsigned launch = misc[2];
                unsigned long long seen = 0ull;
                if (lane == 0) {
                    __hip_atomic_store(&words[(unsigned)blockIdx.x * 4u + b], ((unsigned long long)launch << 32) | __float_as_uint(z),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const unsigned long long* theirs = &words[(unsigned)(blockIdx.x ^ 1u) * 4u + b];
                    for (unsigned tries = 0; tries < SPIN_LIMIT; ++tries) {
                        seen = __hip_atomic_load(theirs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if ((unsigned)(seen >> 32) == launch) break;
                        __builtin_amdgcn_s_sleep(1);
                    }
                    if ((unsigned)(seen >> 32) != launch) { atomicCAS(&a.sync[1], 0u, 1u); atomicOr(&misc[4], 1u); }      // gave up: this workgroup's flag asks for the step to be abandoned
                }
                const unsigned tag = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(seen >> 32));
                const float zo = __uint_as_float((unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)seen));
                use = use && tag == launch && ((r0 & 1u) ? !(zo >= z) : (z >= zo));
            }
            float dA = 0.0f;
            if (use) dA = dbk::loss_grad((int)a.loss_kind, z, Ys[b]) * inv_n;
            if (lane == 0) { zs[b] = z; dAs[b] = dA; lss[b] = use ? 1.0f : 0.0f; }      // (the loss term is formed later, off this wave's path, where lss says so)
            if (hidden && lane < hidden) D1[b * hidden + lane] = hv > 0.0f ? dA * w2 : 0.0f;
            wave_lds_sync();
            // gradient at the pooled features -> what the scan's backward pass needs
            auto put_pool_grad = [&](unsigned kk, float g) {
                if (!kept[b * k + kk]) g = 0.0f;
                const unsigned fl = b * a.nfilter + (kk >> (kpf - 1u));
                const bool is_avg = a.ptype == DBK_PT_AVG || (a.ptype == DBK_PT_ALL && (kk & 1u));
                if (is_avg) cavg[fl] = (live && rinfo[0]) ? g / (float)rinfo[0] : 0.0f;
                else gmax[fl] = (live && PL[b * k + kk] > 0.0f) ? g : 0.0f;
            };
            // Up to 32 features: the wave's lanes are (64 / 16 or 64 / 32 groups of hidden units) x features, a lane adds
            // its group's products (starting at a unit that depends on the feature: neighbouring lanes then read
            // different LDS banks of the weight rows) and the groups' sums meet in a fixed butterfly.
            const unsigned lgkP = k <= 16 ? 4u : 5u, hs = hidden >> (6u - lgkP);
            if (hidden && k <= 32 && (hs << (6u - lgkP)) == hidden && hs >= 2 && (hs & (hs - 1u)) == 0) {
                const unsigned kk = lane & ((1u << lgkP) - 1u), hq = lane >> lgkP;
                float g = 0.0f;
                if (kk < k) {
                    const float* wrow = W1s + ((unsigned)b * kt + kk) * hidden + hq * hs;
                    const float* drow = D1 + b * hidden + hq * hs;
#pragma unroll 8
                    for (unsigned j = 0; j < hs; ++j) {
                        const unsigned h = (j + kk) & (hs - 1u);
                        g += drow[h] * wrow[h];
                    }
                }
                for (unsigned d = 1u << lgkP; d < 64u; d <<= 1) g += __shfl_xor(g, (int)d, 64);
                if (lane < k) put_pool_grad(lane, g);
            } else {
                for (unsigned kk = lane; kk < k; kk += 64) {
                    float g;
                    if (hidden) {
                        g = 0.0f;
                        const float* wrow = W1s + ((unsigned)b * kt + kk) * hidden;
#pragma unroll 8
                        for (unsigned h = 0; h < hidden; ++h) g += D1[b * hidden + h] * wrow[h];
                    } else {
                        g = dA * W1s[(unsigned)b * kt + kk];
                    }
                    put_pool_grad(kk, g);
                }
            }
        }
    } else {
        for (unsigned e = tid; e < RC * nm * k; e += NT) {             // inputs after dropout
            const unsigned rl = by_nmk.quot(e), col = by_nmk.rem(e, rl), b = by_k.quot(col), kk = by_k.rem(col, b);
            H0[(rl * nm + b) * kt + kk] = (rl < nreg && kept[e]) ? PL[e] : 0.0f;
        }
        __syncthreads();
        if (hidden) {
            for (unsigned e = tid; e < RC * nm * hidden; e += NT) {
                const unsigned rb = by_h1.quot(e), h = by_h1.rem(e, rb), b = by_nm.rem(rb, by_nm.quot(rb));
                const float* x = H0 + rb * kt;
                const float* wcol = W1s + (unsigned)b * kt * hidden + h;
                float s = 0.0f;
#pragma unroll 8
                for (unsigned kk = 0; kk < kt; ++kk) s += x[kk] * wcol[kk * hidden];
                s += b1s[b * hidden + h];
                H1[e] = s > 0.0f ? s : 0.0f;
            }
            __syncthreads();
        }
        // output pre-activation and prediction of (row, model): one wave per output, a lane per input, summed by a fixed butterfly
        for (unsigned e = wave; e < RC * nm; e += NW) {
            const unsigned b = by_nm.rem(e, by_nm.quot(e));
            float part = 0.0f;
            if (hidden) {
                for (unsigned h = lane; h < hidden; h += 64) part += H1[(unsigned)e * hidden + h] * W2s[b * hidden + h];
            } else {
                for (unsigned kk = lane; kk < kt; kk += 64) part += H0[(unsigned)e * kt + kk] * W1s[(unsigned)b * kt + kk];
            }
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) part += __shfl_xor(part, d, 64);
            if (lane == 0) {
                const float out = part + (hidden ? b2s[b] : b1s[b]);
                zs[e] = a.loss_kind == 0 ? 1.0f / (1.0f + expf(-out)) : out;
            }
        }
        __syncthreads();
        // loss gradient of (row, model), formed by every thread that needs it; the hidden units' gradients with it
        for (unsigned e = tid; e < RC * nm * h1; e += NT) {
            const unsigned rb = by_h1.quot(e), h = by_h1.rem(e, rb), rl = by_nm.quot(rb), b = by_nm.rem(rb, rl);
            const unsigned rr = (unsigned)r0 + rl;
            float dA = 0.0f, lterm = 0.0f;
            if (rl < nreg) {
                const float z = zs[rb], y = Ys[rb];
                bool use = Yms[rb] != 0u;
                if (a.revcomp) {                                       // of a (fwd, rev) pair only the larger prediction trains; ties keep the first
                    const float zo = zs[(rl ^ 1u) * nm + b];
                    use = use && ((rr & 1) ? !(zo >= z) : (z >= zo));
                }
                if (use) {
                    dA = dbk::loss_grad((int)a.loss_kind, z, y) * inv_n;
                    if (h == 0) lterm = dbk::loss_term((int)a.loss_kind, z, y);
                }
            }
            if (h == 0) { dAs[rb] = dA; lss[rb] = lterm; }
            if (hidden) D1[e] = H1[e] > 0.0f ? dA * W2s[b * hidden + h] : 0.0f;
        }
        __syncthreads();
        for (unsigned e = tid; e < RC * nm * k; e += NT) {             // gradient at the pooled features -> what the scan's backward pass needs
            const unsigned rl = by_nmk.quot(e), col = by_nmk.rem(e, rl), b = by_k.quot(col), kk = by_k.rem(col, b), rb = rl * nm + b;
            float g;
            if (hidden) {
                g = 0.0f;
                const float* wrow = W1s + ((unsigned)b * kt + kk) * hidden;
#pragma unroll 8
                for (unsigned h = 0; h < hidden; ++h) g += D1[(unsigned)rb * hidden + h] * wrow[h];
            } else {
                g = dAs[rb] * W1s[(unsigned)b * kt + kk];
            }
            if (!kept[e]) g = 0.0f;
            const unsigned fl = b * a.nfilter + (kk >> (kpf - 1u));   // filter of the group
            const bool is_avg = a.ptype == DBK_PT_AVG || (a.ptype == DBK_PT_ALL && (kk & 1u));
            if (is_avg) cavg[rl * Fp + fl] = (rl < nreg && rinfo[2 * rl]) ? g / (float)rinfo[2 * rl] : 0.0f;
            else gmax[rl * Fp + fl] = (rl < nreg && PL[e] > 0.0f) ? g : 0.0f;
        }
    }
    __syncthreads();
    // (from here to the grid barrier nothing waits for a store to global memory: the shares travel while the filter
    // gradients are counted)
    // this workgroup's share of the dense layers' gradients and of the loss, rows ascending
    float* share = a.partial + (unsigned)blockIdx.x * a.pstride;
    for (unsigned e = tid; e < nm * kt * h1; e += NT) {
        const unsigned q1 = by_h1.quot(e), h = by_h1.rem(e, q1), b = by_kt.quot(q1), kk = by_kt.rem(q1, b);
        float s = 0.0f;
        for (unsigned rl = 0; rl < RC; ++rl) {
            const unsigned rb = rl * nm + b;
            s += H0[(unsigned)rb * kt + kk] * (hidden ? D1[(unsigned)rb * hidden + h] : dAs[rb]);
        }
        put_share(&share[a.off_W1 + e], s);
    }
    for (unsigned e = tid; e < nm * h1; e += NT) {
        const unsigned b = by_h1.quot(e), h = by_h1.rem(e, b);
        float gb1 = 0.0f, gW2 = 0.0f;
        for (unsigned rl = 0; rl < RC; ++rl) {
            const unsigned rb = rl * nm + b;
            if (hidden) { gb1 += D1[(unsigned)rb * hidden + h]; gW2 += H1[(unsigned)rb * hidden + h] * dAs[rb]; }
            else gb1 += dAs[rb];
        }
        put_share(&share[a.off_b1 + e], gb1);
        if (hidden) put_share(&share[a.off_W2 + e], gW2);
    }
    for (unsigned b = NT - 1u - tid; b < nm; b += NT) {
        float gb2 = 0.0f, ls = 0.0f;
        if (RC == 1u) {
            gb2 = dAs[b];
            if (lss[b] != 0.0f) {
                const float z = zs[b], y = Ys[b];
                ls = dbk::loss_term((int)a.loss_kind, z, y);
            }
        } else {
            for (unsigned rl = 0; rl < RC; ++rl) { gb2 += dAs[rl * nm + b]; ls += lss[rl * nm + b]; }
        }
        if (hidden) put_share(&share[a.off_b2 + b], gb2);
        put_share(&share[a.nparam + b], ls);
    }
    for (unsigned e = tid; e < nreg * nm; e += NT) put_share(&a.Z[(unsigned)r0 * nm + e], zs[e]);      // the predictions of this workgroup's rows

    // ---------------- scan filters: a thread's (tap, filter) pairs, five letter accumulators each, regions ascending
    constexpr unsigned MAXPAIR = (MT * 64 + NTMIN - 1) / NTMIN;
#pragma unroll
    for (unsigned i = 0; i < MAXPAIR; ++i) {
        const unsigned e = tid + i * NT;
        if (e >= MT * Fp) break;
        const unsigned t = e >> lgFp, fl = e & (Fp - 1);
        float acc[5] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f}, accb = 0.0f;
        for (unsigned rl = 0; rl < nreg; ++rl) {
            const unsigned rows = rinfo[2 * rl];
            if (dense) {
                const float c = cavg[rl * Fp + fl];
                const unsigned* am = amask + (rl * Fp + fl) * AW;
                const unsigned nw = (rows + 31u) >> 5;
                unsigned cnt[5] = {0u, 0u, 0u, 0u, 0u}, open = 0u;
                for (unsigned w = 0; w < nw; ++w) {
                    const unsigned bits = am[w];
                    open += __popc(bits);
#pragma unroll
                    for (int l = 0; l < 5; ++l) {
                        const unsigned* lm = lmask + (rl * 5 + l) * LW + w;
                        const unsigned shifted = (unsigned)(((unsigned long long)lm[1] << 32 | lm[0]) >> t);   // letter bits of positions p + t
                        cnt[l] += __popc(bits & shifted);
                    }
                }
#pragma unroll
                for (int l = 0; l < 5; ++l) acc[l] += c * (float)cnt[l];
                accb += c * (float)open;
            }
            if (sparse) {
                const float g = gmax[rl * Fp + fl];
                const unsigned l = text[rl * TXTB + argp[rl * Fp + fl] + t];
#pragma unroll
                for (int c = 0; c < 5; ++c) acc[c] += l == (unsigned)c ? g : 0.0f;
                accb += g;
            }
        }
        if (t < m && fl < F) {
#pragma unroll
            for (int c = 0; c < 4; ++c) put_share(&share[a.off_Wc + (unsigned)(4 * t + c) * F + fl], acc[c] + 0.25f * acc[4]);
        }
        if (t == 0 && fl < F) put_share(&share[a.off_bc + fl], accb);
    }

    // ---------------- every workgroup's share is written: meet, then add them up and step the parameters.
    // What the update reads of the parameter vectors is requested before the wait (nothing changes it until then).
    // A workgroup steps 64 consecutive parameters: wave w adds the shares of its run of workgroups for them (a lane per
    // parameter: every load of a wave is one contiguous 256 bytes), the waves' sums meet in LDS and wave 0 adds them in a
    // fixed tree and applies the step.
    const unsigned total = a.nparam + nm, estep = (unsigned)a.G * 64;
    const unsigned efirst = (unsigned)blockIdx.x * 64 + lane;
    float q_p = 0.0f, q_rm = 0.0f, q_mp = 0.0f, q_dr = 0.0f, q_dec = 0.0f;
    if (wave == 0 && efirst < a.nparam) {
        q_p = a.P[efirst]; q_rm = a.mrate[efirst]; q_mp = a.mP[efirst]; q_dr = a.drate[efirst];
        if (a.decay) q_dec = a.decay[efirst];
    }
    if (grid_barrier(a.sync, a.G, misc[2], misc[4] != 0u) != 0u) return;
    // (every workgroup read the launch number before it raised its flag, so it can move on now)
    if (blockIdx.x == 0 && tid == 0) __hip_atomic_store(&a.sync[0], misc[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);      // word 0 counts the launches that stepped
    float* sums = wt;                                              // (the letter table is no longer needed)
    const unsigned per = (a.G + NW - 1) / NW;                      // workgroups each wave adds, ascending
    const unsigned g0 = wave * per, g1 = g0 + per < a.G ? g0 + per : a.G;
    for (unsigned base = (unsigned)blockIdx.x * 64; base < total; base += estep) {
        const unsigned e = base + lane;
        float s = 0.0f;
        if (e < total) {
            for (unsigned c0 = g0; c0 < g1; c0 += 16) {           // all of a wave's workgroups requested at once (a full grid: 16)
                float v[16];
#pragma unroll
                for (unsigned u = 0; u < 16; ++u) v[u] = c0 + u < g1 ? a.partial[(unsigned)(c0 + u) * a.pstride + e] : 0.0f;
#pragma unroll
                for (unsigned u = 0; u < 16; ++u)
                    if (c0 + u < g1) s += v[u];
            }
        }
        if (base != (unsigned)blockIdx.x * 64) __syncthreads();      // (a further round: the sums of the last one have been read)
        sums[wave * 64 + lane] = s;
        __syncthreads();
        if (wave != 0 || e >= total) continue;
        float pw[NWMAX];
#pragma unroll
        for (unsigned w = 0; w < NWMAX; ++w) pw[w] = w < NW ? sums[w * 64 + lane] : 0.0f;
        s = ((pw[0] + pw[1]) + (pw[2] + pw[3])) + ((pw[4] + pw[5]) + (pw[6] + pw[7]));
        if (e >= a.nparam) {
            if (a.loss) a.loss[e - a.nparam] = dbk::loss_mean((int)a.loss_kind, s, (float)a.nregion);
            continue;
        }
        if (e != efirst) {
            q_p = a.P[e]; q_rm = a.mrate[e]; q_mp = a.mP[e]; q_dr = a.drate[e];
            if (a.decay) q_dec = a.decay[e];
        }
        float g = s;
        const float lk = q_p + q_rm * q_mp;
        if (a.decay) g += (float)((lk > 0.0f) - (lk < 0.0f)) * q_dec;
        if (a.freeze_scan && e - a.off_Wc < (unsigned)4 * m * F) g = 0.0f;
        a.dP[e] = g;
        const float delta = g * q_dr;
        a.mP[e] = q_mp * q_rm - delta;
        a.P[e] = lk - delta;
    }
    if (a.counter && a.draws && blockIdx.x == 0 && tid == 0) a.counter[0] += a.draws;
}

unsigned ilog2(unsigned v) { unsigned l = 0; while ((1u << l) < v) ++l; return l; }

// Fills the launch shape for a group; false when the single-launch step does not take it.
bool plan(const dbk_train_step_args* a, single_args& s, unsigned& MT, size_t& lds_bytes)
{
    if (!a || a->nmodel < 1 || a->nmodel > 4 || a->nfilter < 1 || a->m < 1 || a->m > 32) return false;
    const size_t F = a->nmodel * a->nfilter;
    if (F > 64 || a->hidden > 64 || !a->nesterov || a->input_rate > 0.0f || a->nregion < 1 || a->N >= 0xffffff00ull) return false;
    if (a->ptype != DBK_PT_MAX && a->ptype != DBK_PT_AVG && a->ptype != DBK_PT_ALL) return false;
    if (a->reverse_complement && (a->nregion & 1)) return false;
    s.nmodel = (unsigned)a->nmodel; s.nfilter = (unsigned)a->nfilter; s.F = (unsigned)F;
    s.Fp = F <= 16 ? 16u : (F <= 32 ? 32u : 64u);
    s.lgFp = ilog2(s.Fp);
    s.m = (unsigned)a->m; s.hidden = (unsigned)a->hidden; s.h1 = s.hidden ? s.hidden : 1u;
    s.k = (unsigned)a->nfilter * (a->ptype == DBK_PT_ALL ? 2u : 1u);
    s.kf = (unsigned)a->nfeat; s.kt = s.k + s.kf;
    if (s.kt > 160) return false;
    s.ptype = (unsigned)a->ptype; s.loss_kind = (unsigned)a->loss_kind; s.revcomp = a->reverse_complement ? 1u : 0u;
    MT = a->m <= 16 ? 16u : (a->m <= 24 ? 24u : 32u);
    // regions per workgroup: as few as keep the grid within MAXG workgroups (one region: eight waves share it),
    // an even number with reverse-complement pairs (a pair's two rows meet in one workgroup)
    // (every workgroup must be resident while the grid waits at the barrier: no more of them than the device has CUs)
    const unsigned cus = dbk_scan::cu_count(), maxg = cus < MAXG ? cus : MAXG;
    unsigned RC = (unsigned)((a->nregion + maxg - 1) / maxg);
    if (a->reverse_complement && RC > 1) RC += RC & 1u;        // (one region per workgroup: the pair's workgroups are neighbours)
    if (RC > 16) return false;
    s.RC = RC;
    s.G = (unsigned)((a->nregion + RC - 1) / RC);
    if (s.G > maxg) return false;
    s.nparam = (unsigned)a->nparam;               // (at most 24576: checked below)
    s.pstride = (unsigned)((a->nparam + a->nmodel + 63) & ~(size_t)63);
    if (a->nparam > 24576) return false;
    s.L = make_map(MT, s.Fp, s.nmodel, s.kt, s.k, s.h1, (unsigned)a->nparam, s.RC, a->ptype != DBK_PT_MAX);
    lds_bytes = (size_t)s.L.total * 4;
    return lds_bytes <= dbk_scan::lds_limit();
}

}  // namespace

extern "C" int dbk_train_step_single_workspace(const dbk_train_step_args* a, size_t* work_bytes)
{
    DBK_CHECK(a && work_bytes, "ValueError: null pointer argument");
    single_args s;
    unsigned MT;
    size_t lds;
    *work_bytes = plan(a, s, MT, lds) ? WORK_HEADER + (size_t)s.G * s.pstride * sizeof(float) : 0;
    dbk::clear_error();
    return 0;
}

extern "C" int dbk_train_step_single(dbk_stream_t stream, const dbk_train_step_args* a, void* work, size_t work_bytes)
{
    single_args s;
    unsigned MT = 0;
    size_t lds = 0;
    DBK_CHECK(plan(a, s, MT, lds), "NotImplementedError: the single-launch step takes 1-4 models with at most 64 filters of at most 32 taps, "
              "Nesterov momentum, no input dropout and at most %u x 16 regions of at most %u rows", MAXG, MAXROWS);
    DBK_CHECK(a->loss_kind >= 0 && a->loss_kind <= 2, "ValueError: loss kind must be 0 (logistic + nll), 1 (linear + mse) or 2 (linear + hinge), got %d", a->loss_kind);
    DBK_CHECK(a->P && a->dP && a->mP && a->drate && a->mrate, "ValueError: null parameter vector");
    DBK_CHECK(a->X && a->regions && a->Y && a->Z, "ValueError: null batch or work buffer");
    DBK_CHECK(!a->rate || a->counter, "ValueError: dropout needs the device generator position");
    DBK_CHECK(work && work_bytes >= WORK_HEADER + (size_t)s.G * s.pstride * sizeof(float) && ((uintptr_t)work & 15) == 0,
              "ValueError: the workspace must hold dbk_train_step_single_workspace() bytes, 16-byte aligned");
    const size_t F = s.F, h1 = s.h1;
    const size_t nWc = 4 * a->m * F, nW1 = (size_t)s.kt * a->nmodel * h1, nb1 = a->nmodel * h1;
    const size_t nW2 = s.hidden ? s.hidden * a->nmodel : 0, nb2 = s.hidden ? a->nmodel : 0;
    DBK_CHECK(nWc + F + nW1 + nb1 + nW2 + nb2 == a->nparam, "ValueError: the parameter blocks do not tile the flat vector (%zu of %zu elements)",
              nWc + F + nW1 + nb1 + nW2 + nb2, a->nparam);
    const size_t need[6] = { a->off_Wc + nWc, a->off_bc + F, a->off_W1 + nW1, a->off_b1 + nb1, a->off_W2 + nW2, a->off_b2 + nb2 };
    for (size_t v : need) DBK_CHECK(v <= a->nparam, "ValueError: a parameter block reaches past the flat vector (%zu > %zu)", v, a->nparam);
    s.P = a->P; s.dP = a->dP; s.mP = a->mP; s.drate = a->drate; s.mrate = a->mrate; s.decay = a->decay;
    s.off_Wc = (unsigned)a->off_Wc; s.off_bc = (unsigned)a->off_bc; s.off_W1 = (unsigned)a->off_W1;       // (all below nparam: checked above)
    s.off_b1 = (unsigned)a->off_b1; s.off_W2 = (unsigned)a->off_W2; s.off_b2 = (unsigned)a->off_b2;
    s.X = a->X; s.N = (unsigned)a->N; s.R = a->regions; s.nregion = (unsigned)a->nregion;
    s.Y = a->Y; s.Ymask = a->Ymask; s.feats = a->feats;
    s.rate = a->rate; s.seed = a->seed; s.counter = (unsigned long long*)a->counter;
    s.draws = a->rate ? (a->nregion * s.k * a->nmodel + 3) / 4 : 0;
    s.freeze_scan = a->freeze_scan; s.Z = a->Z; s.loss = a->loss;
    s.sync = (unsigned*)work;
    s.partial = (float*)((char*)work + WORK_HEADER);
    const int shape = s.RC != 1 ? 0 : (s.Fp == 32 ? 3 : s.Fp == 64 ? 4 : s.nmodel == 1 ? 2 : 1);
    auto pick = [&](auto mt) {
        constexpr int M = decltype(mt)::value;
        return shape == 4 ? k_step_single<M, 4> : shape == 3 ? k_step_single<M, 3> : shape == 2 ? k_step_single<M, 2>
             : shape == 1 ? k_step_single<M, 1> : k_step_single<M, 0>;
    };
    auto kern = MT == 16 ? pick(std::integral_constant<int, 16>{}) : (MT == 24 ? pick(std::integral_constant<int, 24>{}) : pick(std::integral_constant<int, 32>{}));
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kern, dim3(s.G), dim3(s.RC == 1 ? NTMAX : NTMIN), lds, dbk::as_stream(stream), s);
    DBK_LAUNCH_OK();
}

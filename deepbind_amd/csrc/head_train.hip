// Forward + backward of the per-model dense head in two launches.
//
// At training sizes (a few hundred rows, 16-64 inputs, 0-64 hidden units per model) the head is a few
// hundred kFLOP per model: run layer by layer its cost is ~20 kernel launches, not arithmetic. Here
// a workgroup takes one model and a chunk of 32 rows, keeps the model's weights in LDS, and eight
// adjacent lanes share a row: dropout, both layers, the output non-linearity, the loss gradient and
// the gradient back to the pooled features, then the chunk's contribution to every weight gradient
// (rows ascending) goes to a partial-sum buffer. A second small kernel adds the chunks in ascending
// order. No atomics; the summation order depends only on the shapes, so results are bit-reproducible.
//
// Replaces, per step: dropout_fp_train -> blockwise_dot(_combined) -> bias -> relu -> blockwise_dot -> bias
// -> logistic -> loss bprop -> maskout (Ymask, Zmask) -> bias bprop -> blockwise_dot_tn/_nt -> relu bprop -> ... ->
// dropout_bp_tr (reference: deepity/std/elemwise.py:71-180, full.py:78-119, softmax.py:58-77, loss.py:98-119,
// deepity_smat/dropout.cu:41-109, blockwise_dot.cu:77-153, maskout.cu:41-67).
#include "dbk_common.h"
#include "rng.h"
#include "scan_common.h"

namespace {

constexpr int RB = 32;             // rows per workgroup
constexpr int NP = 8;              // adjacent lanes sharing one row
constexpr int NT = RB * NP;        // threads per workgroup

struct head_args {
    size_t n;
    int nblock, k, kf, hidden, loss_kind, revcomp;   // k pooled features per model + kf feature columns shared by all models
    const float *pooled, *feats, *rate, *U;
    unsigned long long seed, offset;
    unsigned long long* counter;
    unsigned long long counter_advance;
    const float *W1, *b1, *W2, *b2, *Y;
    const uint8_t* Ymask;
    float *Z, *dpooled, *dW1, *db1, *dW2, *db2, *loss;
    float* partial;                // [chunk][model][pstride]: dW1 (k*h1), db1 (h1), dW2 (h1), db2, loss sum
    unsigned nchunk, pstride;
};

// Orders a wave's own LDS traffic: what its lanes stored before is what its lanes read after (the LDS serves a wave's
// instructions in order; the fences keep the compiler from moving them and wait for the counter).
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

template <int CTRL>
__device__ __forceinline__ float lane_move(float v) { return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true)); }

// The head of a model with 32 hidden units and 16 or 32 inputs (the shapes of the reference's models: 16 filters, max or
// max + average pooling, cfg/classification/M1.cfg) for a chunk of 32 rows, with the weights in REGISTERS while they
// are used: the workgroup stages the model's W1 in LDS with one 16-byte load per thread, then each of the four waves
// takes eight rows through forward and backward on its own, two rows at a time (a row per half wave), with no
// workgroup barrier until the chunk's gradient sums. A lane holds column j of W1 for the forward pass (lane = hidden
// unit: 32 multiply-adds per row, the row's inputs read from LDS as broadcasts) and row j for the way back (lane =
// input). The eight rows' output non-linearity, loss gradient and loss term are computed ONCE, eight lanes side by side
// (the general body below computes them in every lane of a row, and reads a weight from LDS per multiply-add).
// Every sum is formed in the order of the general body (inputs ascending, hidden units ascending, rows ascending; the
// output sum as eight partial sums of every eighth unit folded by a butterfly), so the two bodies give the same bits.
template <int KT>
__device__ __forceinline__ void head_train_h32(const head_args& a, const unsigned b, const unsigned chunk)
{
    extern __shared__ float hs[];
    constexpr int H = 32, WS = 36;          // hidden units; floats from one row of W1 to the next in LDS (16-byte reads of
                                            // neighbouring rows then start four banks apart)
    float* w1s = hs;                        // [KT][WS]
    float* xs = w1s + KT * WS;              // [RB][KT] inputs after dropout
    float* H1s = xs + RB * KT;              // [RB][H]  hidden activations
    float* D1s = H1s + RB * H;              // [RB][H]  gradient at the hidden pre-activations
    float* dAs = D1s + RB * H;              // [RB]
    float* lss = dAs + RB;                  // [RB]
    unsigned char* kept = reinterpret_cast<unsigned char*>(lss + RB);   // [RB][KT] dropout keep flags
    const unsigned tid = threadIdx.x, lane = tid & 63u, j = lane & 31u, half = lane >> 5;
    const unsigned wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const int k = a.k;
    const size_t r0 = (size_t)chunk * RB, ncol = (size_t)k * a.nblock;

    // ---------------- everything the workgroup reads from global memory, requested in one round
    const float p_drop = a.rate ? a.rate[b] : 0.0f;
    const unsigned long long off = a.counter ? a.counter[0] : a.offset;
    float4 wv = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (tid < (unsigned)(KT * H / 4)) wv = reinterpret_cast<const float4*>(a.W1 + (size_t)b * KT * H)[tid];
    // lane L < 8 of a wave holds the target and mask of the wave's row L
    const size_t r_mine = r0 + 8u * wave + (lane & 7u);
    const bool live_mine = lane < 8u && r_mine < a.n;
    const size_t zi_mine = live_mine ? r_mine * a.nblock + b : 0;
    const float y_mine = live_mine ? a.Y[zi_mine] : 0.0f;
    const bool use_mine = (live_mine && a.Ymask) ? a.Ymask[zi_mine] != 0 : true;
    const float b1v = a.b1[(size_t)b * H + j], w2v = a.W2[(size_t)b * H + j], bias2 = a.b2[b];
    const float inv_n = 1.0f / (float)a.n;
    {   // the chunk's inputs, dropout applied (element numbering of the stand-alone dropout kernels): four consecutive
        // features per thread - one 16-byte load and ONE call of the generator for their four uniforms
        const unsigned kq = (unsigned)k >> 2;
        const dbk::small_div by_kq(kq), by_kf((unsigned)(a.kf > 0 ? a.kf : 1));
        for (unsigned e = tid; e < RB * kq; e += NT) {
            const unsigned row = by_kq.quot(e), kk = 4u * by_kq.rem(e, row);
            const size_t rr = r0 + row, col = (size_t)b * k + kk;
            float4 xv = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            float u[4] = {1.0f, 1.0f, 1.0f, 1.0f};
            const bool in = rr < a.n;
            if (in) {
                xv = *reinterpret_cast<const float4*>(a.pooled + rr * ncol + col);
                if (a.rate) dbk_rng::uniform4_at(a.seed, off, ((a.revcomp ? (rr >> 1) : rr) * ncol + col) >> 2, u);
            }
            const float x4[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const bool kp = !(in && a.rate) || u[c] >= p_drop;
                xs[row * KT + kk + c] = kp ? x4[c] : 0.0f;
                kept[row * KT + kk + c] = kp;
            }
        }
        for (unsigned e = tid; e < RB * (unsigned)a.kf; e += NT) {      // the shared feature columns follow the model's own inputs
            const unsigned row = by_kf.quot(e), jj = by_kf.rem(e, row);
            const size_t rr = r0 + row;
            xs[row * KT + k + jj] = (a.feats && rr < a.n) ? a.feats[rr * a.kf + jj] : 0.0f;
        }
    }
    if (tid < (unsigned)(KT * H / 4)) *reinterpret_cast<float4*>(w1s + (tid >> 3) * WS + 4u * (tid & 7u)) = wv;
    __syncthreads();
    float wc[KT], wr[H];
#pragma unroll
    for (int kk = 0; kk < KT; ++kk) wc[kk] = w1s[kk * WS + j];
#pragma unroll
    for (int q = 0; q < H / 4; ++q) {
        const float4 v = reinterpret_cast<const float4*>(w1s + (j < (unsigned)KT ? j : 0u) * WS)[q];
        wr[4 * q] = v.x; wr[4 * q + 1] = v.y; wr[4 * q + 2] = v.z; wr[4 * q + 3] = v.w;
    }

    // ---------------- forward, two rows per round: lane = hidden unit j of the half wave's row
    // (the four rows' sums advance side by side: each is a chain of dependent additions, inputs ascending)
    float sv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int q = 0; q < KT / 4; ++q) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 x4 = reinterpret_cast<const float4*>(xs + (8u * wave + 2u * i + half) * KT)[q];
            sv[i] += x4.x * wc[4 * q];
            sv[i] += x4.y * wc[4 * q + 1];
            sv[i] += x4.z * wc[4 * q + 2];
            sv[i] += x4.w * wc[4 * q + 3];
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float s = sv[i] + b1v;
        s = s > 0.0f ? s : 0.0f;
        sv[i] = s;
        H1s[(8u * wave + 2u * i + half) * H + j] = s;
    }
    // the rows' output sums: units p, p + 8, p + 16, p + 24 added in that order (p < 8), then a butterfly over the eight;
    // row L of the wave's eight ends up in lane L
    float o_mine = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float v = 0.0f + sv[i] * w2v;
        const float u16 = __shfl_down(v, 16, 64), u24 = __shfl_down(v, 24, 64);
        float t = v + lane_move<0x128>(v);                            // row_ror:8 - unit p + 8 of the same sixteen lanes
        t += u16;
        t += u24;
        t += lane_move<0xB1>(t);                                      // quad_perm [1, 0, 3, 2]
        t += lane_move<0x4E>(t);                                      // quad_perm [2, 3, 0, 1]
        t += lane_move<0x141>(t);                                     // row_half_mirror: the other four of the eight
        const float ta = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t), 0));
        const float tb = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(t), 32));
        if ((lane >> 1) == (unsigned)i) o_mine = (lane & 1u) ? tb : ta;
    }
    {   // output non-linearity, loss gradient and loss term of the eight rows, in lanes 0..7
        const float out = o_mine + bias2;
        const float z = a.loss_kind == 0 ? 1.0f / (1.0f + expf(-out)) : out;
        // of each (fwd, rev) row pair only the larger prediction trains; ties keep the first row
        const float zo = lane_move<0xB1>(z);
        float dA = 0.0f, lterm = 0.0f;
        if (live_mine) {
            bool use = use_mine;
            if (a.revcomp) use = use && ((r_mine & 1) ? !(zo >= z) : (z >= zo));
            if (use) {
                dA = dbk::loss_grad(a.loss_kind, z, y_mine) * inv_n;
                lterm = dbk::loss_term(a.loss_kind, z, y_mine);
            }
            a.Z[zi_mine] = z;
        }
        if (lane < 8u) { dAs[8u * wave + lane] = dA; lss[8u * wave + lane] = lterm; }
    }
    wave_lds_sync();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const unsigned row = 8u * wave + 2u * i + half;
        D1s[row * H + j] = sv[i] > 0.0f ? dAs[row] * w2v : 0.0f;
    }
    wave_lds_sync();

    // ---------------- gradient back to the pooled features: lane = input j of the half wave's row
    float gv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int q = 0; q < H / 4; ++q) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 d4 = reinterpret_cast<const float4*>(D1s + (8u * wave + 2u * i + half) * H)[q];
            gv[i] += d4.x * wr[4 * q];
            gv[i] += d4.y * wr[4 * q + 1];
            gv[i] += d4.z * wr[4 * q + 2];
            gv[i] += d4.w * wr[4 * q + 3];
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const unsigned row = 8u * wave + 2u * i + half;
        const size_t r = r0 + row;
        if (r < a.n && j < (unsigned)k) a.dpooled[r * ncol + (size_t)b * k + j] = kept[row * KT + j] ? gv[i] : 0.0f;
    }
    __syncthreads();

    // ---------------- this chunk's share of the parameter gradients, rows ascending
    float* part_out = a.partial + ((size_t)chunk * a.nblock + b) * a.pstride;
    constexpr int PER = KT / 8;                                       // consecutive inputs per thread
    const unsigned kk0 = (unsigned)PER * (2u * wave + half);
    float acc[PER], gb1 = 0.0f;
#pragma unroll
    for (int c = 0; c < PER; ++c) acc[c] = 0.0f;
#pragma unroll 16
    for (int rr = 0; rr < RB; ++rr) {
        const float d = D1s[rr * H + j];
#pragma unroll
        for (int c = 0; c < PER; ++c) acc[c] += xs[rr * KT + kk0 + c] * d;
        gb1 += d;
    }
#pragma unroll
    for (int c = 0; c < PER; ++c) part_out[(kk0 + c) * H + j] = acc[c];
    // the small sums, one per wave (the wave's number is a scalar: no lane masks, the reads of a loop in flight together)
    if (wave == 0) {
        if (half == 0) part_out[KT * H + j] = gb1;
    } else if (wave == 1) {
        float gW2 = 0.0f;
#pragma unroll 16
        for (int rr = 0; rr < RB; ++rr) gW2 += H1s[rr * H + j] * dAs[rr];
        if (half == 0) part_out[KT * H + H + j] = gW2;
    } else {
        const float* src = wave == 2 ? dAs : lss;
        float sum = 0.0f;
#pragma unroll 16
        for (int rr = 0; rr < RB; ++rr) sum += src[rr];
        if (lane == 0) part_out[KT * H + 2 * H + (wave == 2 ? 0 : 1)] = sum;
    }
}

// b: model of the group, chunk: which RB rows
__device__ __forceinline__ void head_train_body(const head_args& a, const unsigned b, const unsigned chunk)
{
    if (a.hidden == 32 && !a.U && (a.k & 3) == 0 && (((size_t)a.k * a.nblock) & 3) == 0 && ((uintptr_t)a.pooled & 15) == 0 &&
        (a.k + a.kf == 16 || a.k + a.kf == 32)) {
        if (a.k + a.kf == 32) head_train_h32<32>(a, b, chunk);
        else head_train_h32<16>(a, b, chunk);
        return;
    }
    extern __shared__ float hs[];
    // kt inputs per model: its k pooled features, then the kf shared feature columns (no dropout, no gradient back)
    const int k = a.k, kt = a.k + a.kf, hidden = a.hidden, h1 = hidden > 0 ? hidden : 1;
    const unsigned tid = threadIdx.x;
    const size_t r0 = (size_t)chunk * RB;
    const int row = tid / NP, part = tid % NP;
    const size_t r = r0 + row;
    const bool live = r < a.n;
    const size_t ncol = (size_t)k * a.nblock;
    // per-row strides are odd so that lanes holding different rows hit distinct LDS banks; the weight rows too:
    // in the backward pass the eight lanes of a row read eight different inputs' weights for the same hidden unit
    const int ks = kt | 1, hst = h1 | 1, wst = hidden > 0 ? (hidden | 1) : 1;
    float* w1s = hs;                        // [kt][wst]
    float* b1s = w1s + kt * wst;            // [h1]
    float* w2s = b1s + h1;                  // [h1] (unused when hidden == 0)
    float* H0s = w2s + h1;                  // [RB][ks]  inputs after dropout
    float* H1s = H0s + RB * ks;             // [RB][hst] hidden activations (hidden > 0)
    float* D1s = H1s + RB * hst;            // [RB][hst] gradient at the hidden pre-activations
    float* dAs = D1s + RB * hst;            // [RB]      gradient at the output pre-activation
    float* lss = dAs + RB;                  // [RB]      loss terms
    unsigned char* kept = reinterpret_cast<unsigned char*>(lss + RB);   // [RB][k] dropout keep flags
    const dbk::small_div by_h1((unsigned)h1), by_k((unsigned)k), by_kf((unsigned)a.kf);      // (all dividends below are < 2^20)

    // four loads in flight per thread and round (a plain strided loop waits for each load before the next)
    for (int e0 = tid; e0 < kt * h1; e0 += 4 * NT) {
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = e0 + j * NT < kt * h1 ? a.W1[(size_t)b * kt * h1 + e0 + j * NT] : 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = e0 + j * NT;
            if (e < kt * h1) { const unsigned kk = by_h1.quot(e); w1s[kk * wst + by_h1.rem(e, kk)] = v[j]; }
        }
    }
    for (int e = tid; e < h1; e += NT) {                          // both vectors' loads are issued before either is stored
        const float vb = a.b1[(size_t)b * h1 + e];
        const float vw = e < hidden ? a.W2[(size_t)b * hidden + e] : 0.0f;
        b1s[e] = vb;
        if (e < hidden) w2s[e] = vw;
    }
    const float bias2 = hidden > 0 ? a.b2[b] : 0.0f;
    // this row's target and mask are needed only after the forward pass: requested now, they arrive meanwhile
    const size_t zi = live ? r * a.nblock + b : 0;
    const float y_row = live ? a.Y[zi] : 0.0f;
    const bool use_row = (live && a.Ymask) ? a.Ymask[zi] != 0 : true;
    const float p_drop = a.rate ? a.rate[b] : 0.0f;
    const unsigned long long off = a.counter ? a.counter[0] : a.offset;
    const float inv_n = 1.0f / (float)a.n;

    // ---------------- inputs of the chunk, dropout applied (same element numbering as the stand-alone dropout kernels)
    if (!a.U && (k & 3) == 0 && (ncol & 3) == 0 && ((uintptr_t)a.pooled & 15) == 0) {
        // four consecutive features of a row per thread: one 16-byte load and ONE call of the generator for their four
        // uniforms (flat elements 4q .. 4q+3 share a counter value)
        const unsigned kq = (unsigned)k >> 2;
        const dbk::small_div by_kq(kq);
        for (unsigned e = tid; e < RB * kq; e += NT) {
            const unsigned er = by_kq.quot(e), kk = 4u * by_kq.rem(e, er);
            const size_t rr = r0 + er, col = (size_t)b * k + kk;
            float4 xv = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            float u[4] = {1.0f, 1.0f, 1.0f, 1.0f};
            const bool in = rr < a.n;
            if (in) {
                xv = *reinterpret_cast<const float4*>(a.pooled + rr * ncol + col);
                if (a.rate) dbk_rng::uniform4_at(a.seed, off, ((a.revcomp ? (rr >> 1) : rr) * ncol + col) >> 2, u);
            }
            const float x4[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool kp = !(in && a.rate) || u[j] >= p_drop;
                H0s[er * ks + kk + j] = kp ? x4[j] : 0.0f;
                kept[er * k + kk + j] = kp;
            }
        }
    } else {
        for (int e0 = tid; e0 < RB * k; e0 += 4 * NT) {
            float xv[4], uv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {                              // the loads of a round first
                const int e = e0 + j * NT, er = (int)by_k.quot((unsigned)e), kk = e - er * k;
                const size_t rr = r0 + er, col = (size_t)b * k + kk;
                const bool in = e < RB * k && rr < a.n;
                xv[j] = in ? a.pooled[rr * ncol + col] : 0.0f;
                uv[j] = (in && a.rate && a.U) ? a.U[(a.revcomp ? (rr & ~(size_t)1) : rr) * ncol + col] : 1.0f;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e = e0 + j * NT, er = (int)by_k.quot((unsigned)e), kk = e - er * k;
                if (e >= RB * k) break;
                const size_t rr = r0 + er, col = (size_t)b * k + kk;
                bool kp = true;
                if (rr < a.n && a.rate) {
                    const float u = a.U ? uv[j] : dbk_rng::uniform_at(a.seed, off, a.revcomp ? (rr >> 1) * ncol + col : rr * ncol + col);
                    kp = u >= p_drop;
                }
                H0s[er * ks + kk] = kp ? xv[j] : 0.0f;
                kept[e] = kp;
            }
        }
    }
    // the shared feature columns follow the model's own inputs in the row (a null pointer stands for all zeros)
    for (int e = tid; e < RB * a.kf; e += NT) {
        const int er = (int)by_kf.quot((unsigned)e), kk = e - er * a.kf;
        const size_t rr = r0 + er;
        H0s[er * ks + k + kk] = (a.feats && rr < a.n) ? a.feats[rr * a.kf + kk] : 0.0f;
    }
    __syncthreads();

    // ---------------- forward: the row's eight lanes split the hidden units (or, without a hidden layer, the inputs)
    const float* x = H0s + row * ks;
    float outp = 0.0f;
    if (hidden > 0) {
        for (int h = part; h < hidden; h += NP) {
            float s = 0.0f;
#pragma unroll 8
            for (int kk = 0; kk < kt; ++kk) s += x[kk] * w1s[kk * wst + h];
            s += b1s[h];
            s = s > 0.0f ? s : 0.0f;
            H1s[row * hst + h] = s;
            outp += s * w2s[h];
        }
    } else {
#pragma unroll 4
        for (int kk = part; kk < kt; kk += NP) outp += x[kk] * w1s[kk];
    }
    // butterfly over the row's lanes: every lane ends with the same bits
    outp += __shfl_xor(outp, 1, 64);
    outp += __shfl_xor(outp, 2, 64);
    outp += __shfl_xor(outp, 4, 64);
    const float out = outp + (hidden > 0 ? bias2 : b1s[0]);
    const float z = a.loss_kind == 0 ? 1.0f / (1.0f + expf(-out)) : out;
    // of each (fwd, rev) row pair only the larger prediction trains; ties keep the first row
    const float zo = __shfl_xor(z, NP, 64);
    float dA = 0.0f, lterm = 0.0f;
    if (live) {
        const float y = y_row;
        bool use = use_row;
        if (a.revcomp) use = use && ((r & 1) ? !(zo >= z) : (z >= zo));
        if (use) {
            dA = dbk::loss_grad(a.loss_kind, z, y) * inv_n;
            lterm = dbk::loss_term(a.loss_kind, z, y);
        }
        if (part == 0) a.Z[zi] = z;
    }
    if (part == 0) {
        dAs[row] = dA;
        lss[row] = lterm;
    }
    // gradient at the hidden pre-activations, once: the loops below then run without branches, so that their
    // LDS reads can be issued back to back
    if (hidden > 0)
        for (int h = part; h < hidden; h += NP) D1s[row * hst + h] = H1s[row * hst + h] > 0.0f ? dA * w2s[h] : 0.0f;
    __syncthreads();

    // ---------------- gradient back to the pooled features: the row's lanes split the inputs
    if (live) {
        float* pd = a.dpooled + r * ncol + (size_t)b * k;
        for (int kk = part; kk < k; kk += NP) {
            float g;
            if (hidden > 0) {
                g = 0.0f;
#pragma unroll 8
                for (int h = 0; h < hidden; ++h) g += D1s[row * hst + h] * w1s[kk * wst + h];
            } else {
                g = dA * w1s[kk];
            }
            pd[kk] = kept[row * k + kk] ? g : 0.0f;
        }
    }

    // ---------------- this chunk's share of the parameter gradients, rows ascending
    float* part_out = a.partial + ((size_t)chunk * a.nblock + b) * a.pstride;
    for (int pidx = tid; pidx < kt * h1; pidx += NT) {
        const int kk = (int)by_h1.quot((unsigned)pidx), h = pidx - kk * h1;
        float s = 0.0f;
        if (hidden > 0) {
#pragma unroll 8
            for (int rr = 0; rr < RB; ++rr) s += H0s[rr * ks + kk] * D1s[rr * hst + h];
        } else {
#pragma unroll 8
            for (int rr = 0; rr < RB; ++rr) s += H0s[rr * ks + kk] * dAs[rr];
        }
        part_out[pidx] = s;
    }
    for (int h = tid; h < h1; h += NT) {
        float gb1 = 0.0f, gW2 = 0.0f;
        if (hidden > 0) {
#pragma unroll 8
            for (int rr = 0; rr < RB; ++rr) {
                gb1 += D1s[rr * hst + h];
                gW2 += H1s[rr * hst + h] * dAs[rr];
            }
        } else {
            for (int rr = 0; rr < RB; ++rr) gb1 += dAs[rr];
        }
        part_out[kt * h1 + h] = gb1;
        part_out[kt * h1 + h1 + h] = gW2;
    }
    if (tid == NT - 1) {
        float gb2 = 0.0f, ls = 0.0f;
        for (int rr = 0; rr < RB; ++rr) {
            gb2 += dAs[rr];
            ls += lss[rr];
        }
        part_out[kt * h1 + 2 * h1] = gb2;
        part_out[kt * h1 + 2 * h1 + 1] = ls;
    }
}

__global__ __launch_bounds__(NT) void k_head_train(head_args a) { head_train_body(a, blockIdx.x, blockIdx.y); }

// The heads of several model groups in one launch: workgroups first[g] .. first[g+1]-1 are group g's grid of
// (models, row chunks), models fastest.
struct head_multi_args {
    unsigned n;
    unsigned first[dbk::MULTI_MAX + 1];
    head_args g[dbk::MULTI_MAX];
};
__global__ __launch_bounds__(NT) void k_head_train_multi(const head_multi_args m)
{
    unsigned g = 0;
    while (g + 1 < m.n && blockIdx.x >= m.first[g + 1]) ++g;
    const head_args& a = m.g[g];
    const unsigned local = blockIdx.x - m.first[g];
    head_train_body(a, local % (unsigned)a.nblock, local / (unsigned)a.nblock);
}

// Adds the row chunks in ascending order and writes each gradient to its place.
__global__ void k_head_reduce(head_args a)
{
    const int kt = a.k + a.kf, hidden = a.hidden, h1 = hidden > 0 ? hidden : 1;
    const unsigned nW1 = kt * h1;
    const size_t total = (size_t)a.nblock * a.pstride;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const unsigned b = (unsigned)(e / a.pstride), idx = (unsigned)(e % a.pstride);
        float s = 0.0f;
        // eight chunks in flight per round, added in ascending order
        for (unsigned c0 = 0; c0 < a.nchunk; c0 += 8) {
            float v[8];
#pragma unroll
            for (unsigned t = 0; t < 8; ++t) v[t] = c0 + t < a.nchunk ? a.partial[((size_t)(c0 + t) * a.nblock + b) * a.pstride + idx] : 0.0f;
#pragma unroll
            for (unsigned t = 0; t < 8; ++t)
                if (c0 + t < a.nchunk) s += v[t];
        }
        if (idx < nW1) a.dW1[(size_t)b * nW1 + idx] = s;
        else if (idx < nW1 + h1) a.db1[(size_t)b * h1 + (idx - nW1)] = s;
        else if (idx < nW1 + 2 * h1) { if (hidden > 0) a.dW2[(size_t)b * hidden + (idx - nW1 - h1)] = s; }
        else if (idx == nW1 + 2 * h1) { if (hidden > 0) a.db2[b] = s; }
        else if (a.loss) a.loss[b] = dbk::loss_mean(a.loss_kind, s, (float)a.n);
    }
    // every workgroup of the forward/backward kernel has read the generator position by now: move it on
    if (a.counter && a.counter_advance && blockIdx.x == 0 && threadIdx.x == 0) a.counter[0] += a.counter_advance;
}

inline size_t head_smem(int k, int kf, int h1)
{
    const int kt = k + kf;
    const size_t general = ((size_t)kt * (h1 | 1) + 2 * h1 + (size_t)RB * (kt | 1) + 2 * (size_t)RB * (h1 | 1) + 2 * RB) * sizeof(float) + (size_t)RB * k;
    const size_t h32 = ((size_t)kt * 36 + (size_t)RB * kt + 2 * (size_t)RB * 32 + 2 * RB) * sizeof(float) + (size_t)RB * kt;      // head_train_h32's carve-up
    return general > h32 ? general : h32;
}

}  // namespace

// The chunk sums are left in the stream's second scratch buffer, group after group, for the step's last kernel.
int dbk::head_train_multi(hipStream_t st, size_t nrow, unsigned n, dbk::head_group* g)
{
    DBK_CHECK(n >= 1 && n <= dbk::MULTI_MAX && nrow >= 1, "ValueError: 1 to %u groups of at least one row", dbk::MULTI_MAX);
    const size_t nchunk = (nrow + RB - 1) / RB;
    head_multi_args m;
    m.n = n;
    m.first[0] = 0;
    size_t smem = 0, total = 0;
    for (unsigned i = 0; i < n; ++i) {
        const int h1 = g[i].hidden > 0 ? g[i].hidden : 1;
        DBK_CHECK(g[i].nblock >= 1 && g[i].k >= 1 && g[i].kf >= 0 && g[i].hidden >= 0, "ValueError: bad head shape (nblock=%d, k=%d, nfeat=%d, hidden=%d)", g[i].nblock, g[i].k, g[i].kf, g[i].hidden);
        DBK_CHECK(g[i].loss_kind >= 0 && g[i].loss_kind <= 2, "ValueError: loss kind must be 0 (logistic + nll), 1 (linear + mse) or 2 (linear + hinge), got %d", g[i].loss_kind);
        DBK_CHECK(!g[i].revcomp || nrow % 2 == 0, "ValueError: reverse-complement rows come in pairs, got %zu rows", nrow);
        const size_t need = head_smem(g[i].k, g[i].kf, h1);
        DBK_CHECK(need <= dbk_scan::lds_limit(), "ValueError: head of %d inputs x %d hidden units needs %zu bytes of LDS", g[i].k + g[i].kf, g[i].hidden, need);
        smem = need > smem ? need : smem;
        g[i].nchunk = (unsigned)nchunk;
        g[i].pstride = (unsigned)((g[i].k + g[i].kf) * h1 + 2 * h1 + 2);
        total += nchunk * (size_t)g[i].nblock * g[i].pstride;
        m.first[i + 1] = m.first[i] + (unsigned)(g[i].nblock * nchunk);
    }
    float* partial = (float*)dbk::workspace(total * sizeof(float), st, 1);
    DBK_CHECK(partial != nullptr, "MemoryError: could not allocate %zu bytes of scratch (%s)", total * sizeof(float), dbk::workspace_error());
    for (unsigned i = 0; i < n; ++i) {
        g[i].partial = partial;
        partial += nchunk * (size_t)g[i].nblock * g[i].pstride;
        head_args& a = m.g[i];
        a.n = nrow; a.nblock = g[i].nblock; a.k = g[i].k; a.kf = g[i].kf; a.feats = g[i].feats; a.hidden = g[i].hidden; a.loss_kind = g[i].loss_kind; a.revcomp = g[i].revcomp;
        a.pooled = g[i].pooled; a.rate = g[i].rate; a.U = nullptr; a.seed = g[i].seed; a.offset = 0;
        a.counter = (unsigned long long*)g[i].counter; a.counter_advance = 0;
        a.W1 = g[i].W1; a.b1 = g[i].b1; a.W2 = g[i].W2; a.b2 = g[i].b2; a.Y = g[i].Y; a.Ymask = g[i].Ymask;
        a.Z = g[i].Z; a.dpooled = g[i].dpooled; a.dW1 = a.db1 = a.dW2 = a.db2 = a.loss = nullptr;
        a.partial = g[i].partial; a.nchunk = g[i].nchunk; a.pstride = g[i].pstride;
    }
    DBK_HIP(hipFuncSetAttribute((const void*)k_head_train_multi, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(k_head_train_multi, dim3(m.first[n]), dim3(NT), smem, st, m);
    DBK_LAUNCH_OK();
}

extern "C" int dbk_head_train(dbk_stream_t stream, size_t n, int nblock, int k, int hidden, int loss_kind, int reverse_complement,
                              const float* pooled, int nfeat, const float* feats, const float* rate, const float* U, uint64_t seed, uint64_t offset,
                              uint64_t* counter, uint64_t counter_advance,
                              const float* W1, const float* b1, const float* W2, const float* b2,
                              const float* Y, const uint8_t* Ymask,
                              float* Z, float* dpooled, float* dW1, float* db1, float* dW2, float* db2, float* loss)
{
    DBK_CHECK(nblock >= 1 && k >= 1 && nfeat >= 0 && hidden >= 0, "ValueError: bad head shape (nblock=%d, k=%d, nfeat=%d, hidden=%d)", nblock, k, nfeat, hidden);
    DBK_CHECK(loss_kind >= 0 && loss_kind <= 2, "ValueError: loss kind must be 0 (logistic + nll), 1 (linear + mse) or 2 (linear + hinge), got %d", loss_kind);
    const int h1 = hidden > 0 ? hidden : 1;
    DBK_CHECK(!reverse_complement || n % 2 == 0, "ValueError: reverse-complement rows come in pairs, got %zu rows", n);
    if (n == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(pooled && W1 && b1 && Y && Z && dpooled && dW1 && db1, "ValueError: null pointer argument");
    DBK_CHECK(hidden == 0 || (W2 && b2 && dW2 && db2), "ValueError: hidden layer requested but W2/b2/dW2/db2 are null");
    const size_t smem = head_smem(k, nfeat, h1);
    DBK_CHECK(smem <= dbk_scan::lds_limit(), "ValueError: head of %d inputs x %d hidden units needs %zu bytes of LDS", k + nfeat, hidden, smem);
    const size_t nchunk = (n + RB - 1) / RB;
    DBK_CHECK(nchunk <= 65535, "ValueError: the fused head takes at most %d rows per call (got %zu)", 65535 * RB, n);
    head_args a;
    a.n = n; a.nblock = nblock; a.k = k; a.kf = nfeat; a.feats = feats; a.hidden = hidden; a.loss_kind = loss_kind; a.revcomp = reverse_complement;
    a.pooled = pooled; a.rate = rate; a.U = U; a.seed = seed; a.offset = offset; a.counter = (unsigned long long*)counter; a.counter_advance = counter_advance;
    a.W1 = W1; a.b1 = b1; a.W2 = W2; a.b2 = b2; a.Y = Y; a.Ymask = Ymask;
    a.Z = Z; a.dpooled = dpooled; a.dW1 = dW1; a.db1 = db1; a.dW2 = dW2; a.db2 = db2; a.loss = loss;
    a.nchunk = (unsigned)nchunk;
    a.pstride = (unsigned)((k + nfeat) * h1 + 2 * h1 + 2);
    const size_t pbytes = nchunk * (size_t)nblock * a.pstride * sizeof(float);
    dbk::deferred_sums* later = dbk::deferred();                   // inside dbk_train_step: the chunk sums are taken by its last kernel
    a.partial = (float*)dbk::workspace(pbytes, dbk::as_stream(stream), later ? 1 : 0);
    DBK_CHECK(a.partial != nullptr, "MemoryError: could not allocate %zu bytes of scratch (%s)", pbytes, dbk::workspace_error());
    DBK_HIP(hipFuncSetAttribute((const void*)k_head_train, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(k_head_train, dim3(nblock, (unsigned)nchunk), dim3(NT), smem, dbk::as_stream(stream), a);
    if (later) {
        later->head_partial = a.partial;
        later->head_nchunk = a.nchunk;
        later->head_pstride = a.pstride;
    } else {
        hipLaunchKernelGGL(k_head_reduce, dim3(dbk::ew_grid((size_t)nblock * a.pstride)), dim3(256), 0, dbk::as_stream(stream), a);
    }
    DBK_LAUNCH_OK();
}

// Forward + backward of the per-model dense head in ONE launch: one workgroup per model.
//
// At training sizes (a few hundred rows, 16-64 inputs, 0-64 hidden units per model) the head is a few
// hundred kFLOP per model: the cost of running it layer by layer is the ~20 kernel launches, not the
// arithmetic. Here a workgroup keeps its model's weights in LDS and walks the batch in chunks of 256
// rows. Phase A: one thread per row does dropout, both layers, the output non-linearity, the loss
// gradient and the gradient back to the pooled features, all in registers, and leaves the row's
// (dropped-out) inputs, hidden activations and output gradient in LDS. Phase B: one thread per weight
// sums its gradient over the chunk's rows in ascending order. No atomics; the summation order depends
// only on the shapes, so results are bit-reproducible.
//
// Replaces, per step: dropout_fp_train -> blockwise_dot(_combined) -> bias -> relu -> blockwise_dot -> bias
// -> logistic -> loss bprop -> maskout (Ymask, Zmask) -> bias bprop -> blockwise_dot_tn/_nt -> relu bprop -> ... ->
// dropout_bp_tr (reference: deepity/std/elemwise.py:71-180, full.py:78-119, softmax.py:58-77, loss.py:98-119,
// deepity_smat/dropout.cu:41-109, blockwise_dot.cu:77-153, maskout.cu:41-67).
#include "dbk_common.h"
#include "rng.h"
#include "scan_common.h"

namespace {

constexpr int RC = 256;            // rows per chunk = threads per workgroup
constexpr int MAXPAIR = 16;        // first-layer weights owned per thread (k*h1 <= 4096)

struct head_args {
    size_t n;
    int nblock, k, hidden, loss_kind, revcomp;
    const float *pooled, *rate, *U;
    unsigned long long seed, offset;
    const unsigned long long* counter;
    const float *W1, *b1, *W2, *b2, *Y;
    const uint8_t* Ymask;
    float *Z, *dpooled, *dW1, *db1, *dW2, *db2, *loss;
};

template <int KMAX>
__global__ __launch_bounds__(RC) void k_head_train(head_args a)
{
    extern __shared__ float hs[];
    const int k = a.k, hidden = a.hidden, h1 = hidden > 0 ? hidden : 1;
    const unsigned b = blockIdx.x, tid = threadIdx.x;
    const size_t ncol = (size_t)k * a.nblock;
    float* w1s = hs;                        // [k][h1]
    float* b1s = w1s + k * h1;              // [h1]
    float* w2s = b1s + h1;                  // [h1] (unused when hidden == 0)
    float* H0s = w2s + h1;                  // [RC][k]   inputs after dropout
    float* H1s = H0s + RC * k;              // [RC][h1]  hidden activations (hidden > 0)
    float* dAs = H1s + RC * h1;             // [RC]      gradient at the output pre-activation
    float* red = dAs + RC;                  // [RC]      loss reduction

    for (int e = tid; e < k * h1; e += RC) w1s[e] = a.W1[(size_t)b * k * h1 + e];
    for (int e = tid; e < h1; e += RC) b1s[e] = a.b1[(size_t)b * h1 + e];
    for (int e = tid; e < hidden; e += RC) w2s[e] = a.W2[(size_t)b * hidden + e];
    const float bias2 = hidden > 0 ? a.b2[b] : 0.0f;
    const float p_drop = a.rate ? a.rate[b] : 0.0f;
    const unsigned long long off = a.counter ? a.counter[0] : a.offset;
    const float inv_n = 1.0f / (float)a.n;

    float gW1[MAXPAIR];
#pragma unroll
    for (int i = 0; i < MAXPAIR; ++i) gW1[i] = 0.0f;
    float gb1 = 0.0f, gW2 = 0.0f, gb2 = 0.0f, lsum = 0.0f;     // thread t owns b1[t], W2[t]; thread 0 owns b2
    __syncthreads();

    for (size_t r0 = 0; r0 < a.n; r0 += RC) {
        const size_t r = r0 + tid;
        const bool live = r < a.n;
        // ---------------- phase A: this thread's row
        float dA = 0.0f;
        if (live) {
            float x[KMAX];
            unsigned long long keep = 0;
            const float* px = a.pooled + r * ncol + (size_t)b * k;
#pragma unroll
            for (int kk = 0; kk < KMAX; ++kk) {
                if (kk < k) {
                    bool kp = true;
                    if (a.rate) {
                        // same element numbering as the stand-alone dropout kernels
                        const size_t col = (size_t)b * k + kk;
                        float u;
                        if (a.U) u = a.U[(a.revcomp ? (r & ~(size_t)1) : r) * ncol + col];
                        else u = dbk_rng::uniform_at(a.seed, off, a.revcomp ? (r >> 1) * ncol + col : r * ncol + col);
                        kp = u >= p_drop;
                    }
                    keep |= (unsigned long long)kp << kk;
                    x[kk] = kp ? px[kk] : 0.0f;
                    H0s[tid * k + kk] = x[kk];
                } else {
                    x[kk] = 0.0f;
                }
            }
            float out = 0.0f;
            if (hidden > 0) {
                for (int h = 0; h < hidden; ++h) {
                    float s = 0.0f;
#pragma unroll
                    for (int kk = 0; kk < KMAX; ++kk)
                        if (kk < k) s += x[kk] * w1s[kk * hidden + h];
                    s += b1s[h];
                    s = s > 0.0f ? s : 0.0f;
                    H1s[tid * hidden + h] = s;
                    out += s * w2s[h];
                }
                out += bias2;
            } else {
#pragma unroll
                for (int kk = 0; kk < KMAX; ++kk)
                    if (kk < k) out += x[kk] * w1s[kk];
                out += b1s[0];
            }
            const float z = a.loss_kind == 0 ? 1.0f / (1.0f + expf(-out)) : out;
            const size_t zi = r * a.nblock + b;
            a.Z[zi] = z;
            const float y = a.Y[zi];
            bool use = a.Ymask ? a.Ymask[zi] != 0 : true;
            if (a.revcomp) {
                // of each (fwd, rev) row pair only the larger prediction trains; ties keep the first row
                const float zo = __shfl_xor(z, 1, 64);
                use = use && ((r & 1) ? !(zo >= z) : (z >= zo));
            }
            dA = use ? (z - y) * inv_n : 0.0f;
            if (use) {
                if (a.loss_kind == 0)
                    lsum += logf(fmaxf(1e-15f, z)) * y + logf(fmaxf(1e-15f, 1.0f - z)) * (1.0f - y);
                else
                    lsum += (z - y) * (z - y);
            }
            // gradient back to the pooled features
            float* pd = a.dpooled + r * ncol + (size_t)b * k;
#pragma unroll
            for (int kk = 0; kk < KMAX; ++kk) {
                if (kk < k) {
                    float g = 0.0f;
                    if (hidden > 0) {
                        for (int h = 0; h < hidden; ++h) {
                            const float d1 = H1s[tid * hidden + h] > 0.0f ? dA * w2s[h] : 0.0f;
                            g += d1 * w1s[kk * hidden + h];
                        }
                    } else {
                        g = dA * w1s[kk];
                    }
                    pd[kk] = ((keep >> kk) & 1ull) ? g : 0.0f;
                }
            }
        }
        dAs[tid] = dA;
        __syncthreads();
        // ---------------- phase B: parameter gradients over the chunk's rows, ascending
        const int rows = (int)((a.n - r0) < (size_t)RC ? (a.n - r0) : RC);
#pragma unroll
        for (int i = 0; i < MAXPAIR; ++i) {
            const int pidx = tid + i * RC;
            if (pidx < k * h1) {
                const int kk = pidx / h1, h = pidx % h1;
                float s = gW1[i];
                if (hidden > 0) {
                    const float w2 = w2s[h];
                    for (int rr = 0; rr < rows; ++rr) {
                        const float d1 = H1s[rr * hidden + h] > 0.0f ? dAs[rr] * w2 : 0.0f;
                        s += H0s[rr * k + kk] * d1;
                    }
                } else {
                    for (int rr = 0; rr < rows; ++rr) s += H0s[rr * k + kk] * dAs[rr];
                }
                gW1[i] = s;
            }
        }
        if ((int)tid < h1) {
            if (hidden > 0) {
                const float w2 = w2s[tid];
                for (int rr = 0; rr < rows; ++rr) {
                    const float hv = H1s[rr * hidden + tid], d = dAs[rr];
                    gb1 += hv > 0.0f ? d * w2 : 0.0f;
                    gW2 += hv * d;
                }
            } else {
                for (int rr = 0; rr < rows; ++rr) gb1 += dAs[rr];
            }
        }
        if (tid == 0 && hidden > 0)
            for (int rr = 0; rr < rows; ++rr) gb2 += dAs[rr];
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < MAXPAIR; ++i) {
        const int pidx = tid + i * RC;
        if (pidx < k * h1) a.dW1[(size_t)b * k * h1 + pidx] = gW1[i];
    }
    if ((int)tid < h1) {
        a.db1[(size_t)b * h1 + tid] = gb1;
        if (hidden > 0) a.dW2[(size_t)b * hidden + tid] = gW2;
    }
    if (tid == 0 && hidden > 0) a.db2[b] = gb2;
    if (a.loss) {
        red[tid] = lsum;
        __syncthreads();
        for (int s = RC / 2; s > 0; s >>= 1) {
            if ((int)tid < s) red[tid] += red[tid + s];
            __syncthreads();
        }
        if (tid == 0) a.loss[b] = a.loss_kind == 0 ? -red[0] * inv_n : 0.5f * red[0] * inv_n;
    }
}

}  // namespace

extern "C" int dbk_head_train(dbk_stream_t stream, size_t n, int nblock, int k, int hidden, int loss_kind, int reverse_complement,
                              const float* pooled, const float* rate, const float* U, uint64_t seed, uint64_t offset,
                              const uint64_t* counter,
                              const float* W1, const float* b1, const float* W2, const float* b2,
                              const float* Y, const uint8_t* Ymask,
                              float* Z, float* dpooled, float* dW1, float* db1, float* dW2, float* db2, float* loss)
{
    DBK_CHECK(nblock >= 1 && k >= 1 && hidden >= 0, "ValueError: bad head shape (nblock=%d, k=%d, hidden=%d)", nblock, k, hidden);
    DBK_CHECK(loss_kind == 0 || loss_kind == 1, "ValueError: loss kind must be 0 (logistic + nll) or 1 (linear + mse), got %d", loss_kind);
    DBK_CHECK(k <= 64, "ValueError: the fused head takes at most 64 inputs per model (got %d)", k);
    const int h1 = hidden > 0 ? hidden : 1;
    DBK_CHECK(k * h1 <= RC * MAXPAIR, "ValueError: first layer too large for the fused head (%d x %d weights per model)", k, h1);
    DBK_CHECK(h1 <= RC, "ValueError: at most %d hidden units per model (got %d)", RC, hidden);
    DBK_CHECK(!reverse_complement || n % 2 == 0, "ValueError: reverse-complement rows come in pairs, got %zu rows", n);
    if (n == 0) { dbk::clear_error(); return 0; }
    DBK_CHECK(pooled && W1 && b1 && Y && Z && dpooled && dW1 && db1, "ValueError: null pointer argument");
    DBK_CHECK(hidden == 0 || (W2 && b2 && dW2 && db2), "ValueError: hidden layer requested but W2/b2/dW2/db2 are null");
    size_t smem = ((size_t)k * h1 + 2 * h1 + (size_t)RC * k + (size_t)RC * h1 + 2 * RC) * sizeof(float);
    DBK_CHECK(smem <= dbk_scan::lds_limit(), "ValueError: head of %d inputs x %d hidden units needs %zu bytes of LDS", k, hidden, smem);
    head_args a;
    a.n = n; a.nblock = nblock; a.k = k; a.hidden = hidden; a.loss_kind = loss_kind; a.revcomp = reverse_complement;
    a.pooled = pooled; a.rate = rate; a.U = U; a.seed = seed; a.offset = offset; a.counter = (const unsigned long long*)counter;
    a.W1 = W1; a.b1 = b1; a.W2 = W2; a.b2 = b2; a.Y = Y; a.Ymask = Ymask;
    a.Z = Z; a.dpooled = dpooled; a.dW1 = dW1; a.db1 = db1; a.dW2 = dW2; a.db2 = db2; a.loss = loss;
    auto kern = k <= 16 ? k_head_train<16> : (k <= 32 ? k_head_train<32> : k_head_train<64>);
    DBK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3(nblock), dim3(RC), smem, dbk::as_stream(stream), a);
    DBK_LAUNCH_OK();
}

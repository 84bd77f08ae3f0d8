// Shared host-side plumbing for libdeepbind_hip.so: error reporting, argument checks,
// launch checks and the per-device scratch workspace.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstddef>
#include "../../include/deepbind_hip.h"

namespace dbk {

// Thread-local text of the last failure; polled by the host language after every call.
void set_error(const char* fmt, ...);
void clear_error();

// Device scratch that grows on demand and lives until the process ends. One buffer per (device, stream):
// launches are ordered within a stream, so consecutive calls on it can share the buffer, and calls on
// different streams never do. 64 stream slots per device; when all are taken the slot used longest ago
// passes to the new stream (after draining the device). Growing a buffer or recycling a slot synchronises
// the device, which a stream under capture does not allow: null then, and when memory runs out, with the
// reason in workspace_error(). A buffer handed out DURING a capture is in a graph from then on: its slot is never
// recycled and the buffer never freed (a later, larger eager call on that stream sets it aside for the graph's replays
// and allocates a new one for the stream).
// `which` selects one of four independent buffers of the stream: 0 and 1 hold kernels' partial results (a call
// that must keep one kernel's partial results while another kernel fills its own uses the second), 2 and 3 the
// whole maps of the unfused scan + pool chain, whose kernels use buffer 0 themselves.
void* workspace(size_t bytes, hipStream_t stream, int which = 0);
const char* workspace_error();

// While dbk_train_step runs, dbk_head_train and dbk_scanpool_bprop leave their partial results unreduced and
// describe them here instead: the step's last kernel adds them up (in the order the stand-alone reduction
// kernels use) and applies the parameter update in the same pass. Thread-local; null outside such a step.
struct deferred_sums {
    const float* head_partial = nullptr;    // [chunk][model][pstride] (see head_train.hip)
    unsigned head_nchunk = 0, head_pstride = 0;
    const float* slabs = nullptr;           // [slab][stride]: 4m*F filter gradients then F bias gradients
    size_t slab_stride = 0;
    unsigned nslab = 0;
};
deferred_sums*& deferred();

// One launch per phase for several model groups that step on the same batch (dbk_train_steps): every group
// keeps the grid, the kernel body and the partial-sum layout it has in a launch of its own, so the results are
// the same bits; the launch just holds all the grids side by side.
constexpr unsigned MULTI_MAX = 8;           // groups per launch
struct scan_group {                         // the scan side of one group
    const float *W, *bias;                  // look-ahead weights: (4m, F) and (F)
    unsigned F;                             // filters of all the group's models
    int ptype;
    const uint8_t* X;                       // the batch, or the group's own copy after input dropout
    float *pooled, *dpooled;
    uint32_t* argmax;
    unsigned long long* act;                // activity masks (null with max pooling)
    // filled in by scan_bprop_multi: where the group's partial gradient sums lie
    float* slabs; size_t slab_stride; unsigned nslab;
};
struct head_group {                         // the dense head of one group (arguments of dbk_head_train)
    int nblock, k, kf, hidden, loss_kind, revcomp;   // kf: feature columns shared by all models (after each model's k inputs)
    const float *pooled, *feats, *rate;
    uint64_t seed; uint64_t* counter;
    const float *W1, *b1, *W2, *b2, *Y;
    const uint8_t* Ymask;
    float *Z, *dpooled;
    // filled in by head_train_multi
    float* partial; unsigned nchunk, pstride;
};
// true when every group's shape is one the multi-group launches take (else the groups are stepped one by one)
bool scan_multi_takes(size_t m, size_t N, size_t P, unsigned n, const scan_group* g);
int scan_fprop_multi(hipStream_t st, size_t m, size_t N, const uint32_t* R, size_t P, unsigned n, const scan_group* g);
int scan_bprop_multi(hipStream_t st, size_t m, size_t N, const uint32_t* R, size_t P, unsigned n, scan_group* g);
int head_train_multi(hipStream_t st, size_t nrow, unsigned n, head_group* g);

// dbk_set_exact_scan: the drop-in scan operators keep to the kernels that add in the reference's order at every size
bool exact_scan();

inline hipStream_t as_stream(dbk_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline unsigned divup(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

// Grid size for grid-stride elementwise kernels: enough workgroups to fill 256 CUs several times.
inline unsigned ew_grid(size_t n, unsigned block = 256)
{
    size_t g = (n + block - 1) / block;
    if (g > 256u * 16u) g = 256u * 16u;
    if (g < 1) g = 1;
    return (unsigned)g;
}


// Quotient of small numbers without the integer division sequence: for e < 2^20 and any divisor, (e + 0.5) / d is at
// least 0.5 / d away from a whole number while the reciprocal's and the product's rounding move it by less than
// e / d * 2^-21, so truncating gives floor(e / d) exactly.
struct small_div {
    float inv; unsigned d;
    __device__ __forceinline__ explicit small_div(unsigned d_) : inv(__builtin_amdgcn_rcpf((float)d_)), d(d_) {}
    __device__ __forceinline__ unsigned quot(unsigned e) const
    {
        if (__builtin_constant_p(d) && d == 1u) return e;
        return (unsigned)(((float)e + 0.5f) * inv);
    }
    __device__ __forceinline__ unsigned rem(unsigned e, unsigned q) const { return e - q * d; }
};

// The three losses of the path (deepity/deepity/std/loss.py:98-174): kind 0 = logistic output + negative log-likelihood,
// 1 = linear output + squared error, 2 = linear output + bidirectional hinge. loss_grad is dLoss/d(output) before the
// masks and the 1/rows factor (loss.py:98-112; hinge: 1 - 2Y where (1-Y)Z + Y(1-Z) > 0, loss.py:165-169), loss_term the
// per-row term that is summed, loss_mean what the reported loss makes of the sum (-mean, mean/2, mean).
constexpr int LOSS_NLL = 0, LOSS_MSE = 1, LOSS_HINGE = 2;
__device__ __forceinline__ float loss_grad(int kind, float z, float y)
{
    if (kind == LOSS_HINGE) return ((1.0f - y) * z + y * (1.0f - z)) > 0.0f ? 1.0f - 2.0f * y : 0.0f;
    return z - y;
}
__device__ __forceinline__ float loss_term(int kind, float z, float y)
{
    if (kind == LOSS_NLL) return logf(fmaxf(1e-15f, z)) * y + logf(fmaxf(1e-15f, 1.0f - z)) * (1.0f - y);
    if (kind == LOSS_MSE) return (z - y) * (z - y);
    return fmaxf(0.0f, (1.0f - y) * z + y * (1.0f - z));
}
__device__ __forceinline__ float loss_mean(int kind, float s, float n)
{
    return kind == LOSS_NLL ? -s / n : (kind == LOSS_MSE ? 0.5f * s / n : s / n);
}

}  // namespace dbk

#define DBK_CHECK(cond, ...)                                  \
    do {                                                      \
        if (!(cond)) {                                        \
            dbk::set_error(__VA_ARGS__);                      \
            return 1;                                         \
        }                                                     \
    } while (0)

#define DBK_HIP(expr)                                                                      \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) {                                                            \
            dbk::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
            return 2;                                                                      \
        }                                                                                  \
    } while (0)

// After a kernel launch: surface launch-configuration errors synchronously, like the reference's
// validate-at-emit convention.
#define DBK_LAUNCH_OK()                                                                    \
    do {                                                                                   \
        hipError_t e_ = hipGetLastError();                                                 \
        if (e_ != hipSuccess) {                                                            \
            dbk::set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(e_), __FILE__, __LINE__); \
            return 2;                                                                      \
        }                                                                                  \
        dbk::clear_error();                                                                \
        return 0;                                                                          \
    } while (0)

#define DBK_DTYPE_OK(dtype) DBK_CHECK((dtype) == DBK_F32 || (dtype) == DBK_F64, "TypeError: dtype must be DBK_F32 or DBK_F64, got %d", (int)(dtype))

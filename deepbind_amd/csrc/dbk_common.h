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
// different streams never do. At most 64 distinct streams per device; null when that is exceeded or
// when memory runs out. Growing a buffer synchronises the device (and so cannot happen under capture).
// `which` selects one of two independent buffers of the stream (a call that must keep one kernel's partial
// results while another kernel fills its own uses the second).
void* workspace(size_t bytes, hipStream_t stream, int which = 0);

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

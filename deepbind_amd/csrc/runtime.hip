// Error state, version, device count, sync and the scratch workspace.
#include <atomic>
#include "dbk_common.h"
#include <cstring>
#include <mutex>

namespace dbk {

static thread_local char g_err[512] = {0};

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

void clear_error() { g_err[0] = 0; }

constexpr int WS_BUFFERS = 4;   // 0, 1: partial sums of the kernels; 2, 3: whole maps of the unfused scan + pool chain
// pinned: a capture has taken a buffer's address into a graph, which may be replayed for as long as the process lives,
// so the slot never changes hands again and its buffers are never freed
struct ws_t { hipStream_t stream = nullptr; void* ptr[WS_BUFFERS] = {}; size_t bytes[WS_BUFFERS] = {}; bool used = false, pinned = false; uint64_t tick = 0; };
constexpr int WS_DEVICES = 64, WS_STREAMS = 64;
static ws_t g_ws[WS_DEVICES][WS_STREAMS];
static uint64_t g_ws_tick = 0;
static std::mutex g_ws_mutex;
static thread_local char g_ws_why[160] = {0};

const char* workspace_error() { return g_ws_why; }

static bool capturing(hipStream_t stream)
{
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) { (void)hipGetLastError(); return false; }
    return status != hipStreamCaptureStatusNone;
}

void* workspace(size_t bytes, hipStream_t stream, int which)
{
    int dev = 0;
    g_ws_why[0] = 0;
    if (which < 0 || which >= WS_BUFFERS) return nullptr;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= WS_DEVICES) {
        snprintf(g_ws_why, sizeof(g_ws_why), "no current device below %d", WS_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    ws_t *w = nullptr, *vacant = nullptr, *oldest = nullptr;
    for (int i = 0; i < WS_STREAMS && !w; ++i) {
        ws_t& c = g_ws[dev][i];
        if (c.used && c.stream == stream) w = &c;
        else if (!c.used) { if (!vacant) vacant = &c; }
        else if (!c.pinned && (!oldest || c.tick < oldest->tick)) oldest = &c;
    }
    if (!w) w = vacant;
    if (!w) {
        // Every slot belongs to some stream: the one used longest ago changes hands, buffers included. Its stream
        // may have been destroyed (a graph capture's) or may still run work that reads the buffers, so the whole
        // device is drained first, which a capture in progress does not allow.
        if (capturing(stream)) {
            snprintf(g_ws_why, sizeof(g_ws_why), "all %d stream slots are taken and one cannot be recycled while the stream is capturing", WS_STREAMS);
            return nullptr;
        }
        if (hipDeviceSynchronize() != hipSuccess) {
            (void)hipGetLastError();
            snprintf(g_ws_why, sizeof(g_ws_why), "could not drain the device to recycle a stream slot");
            return nullptr;
        }
        if (!oldest) {
            snprintf(g_ws_why, sizeof(g_ws_why), "all %d stream slots hold scratch that captured graphs refer to", WS_STREAMS);
            return nullptr;
        }
        w = oldest;
    }
    w->used = true;
    w->stream = stream;
    w->tick = ++g_ws_tick;
    const bool under_capture = capturing(stream);
    if (w->bytes[which] >= bytes && w->ptr[which]) {
        if (under_capture) w->pinned = true;
        return w->ptr[which];
    }
    if (under_capture) {
        snprintf(g_ws_why, sizeof(g_ws_why), "scratch cannot grow while the stream is capturing: run the call once eagerly on this stream first");
        return nullptr;
    }
    if (w->ptr[which] && w->pinned) {
        // A captured graph refers to this buffer and may be replayed as long as the process lives: it is set aside, never
        // freed, and the stream gets a larger one for its eager calls and later captures.
        w->ptr[which] = nullptr;
        w->bytes[which] = 0;
    }
    if (w->ptr[which]) {
        // earlier launches may still be reading the old buffer
        if (hipDeviceSynchronize() != hipSuccess) {
            (void)hipGetLastError();
            snprintf(g_ws_why, sizeof(g_ws_why), "could not drain the device before growing the buffer");
            return nullptr;
        }
        (void)hipFree(w->ptr[which]);
        w->ptr[which] = nullptr;
        w->bytes[which] = 0;
    }
    size_t want = bytes < (size_t(1) << 20) ? (size_t(1) << 20) : bytes + bytes / 4;
    if (hipMalloc(&w->ptr[which], want) != hipSuccess) {
        (void)hipGetLastError();
        w->ptr[which] = nullptr;
        snprintf(g_ws_why, sizeof(g_ws_why), "hipMalloc of %zu bytes failed", want);
        return nullptr;
    }
    w->bytes[which] = want;
    return w->ptr[which];
}

static thread_local deferred_sums* g_deferred = nullptr;
deferred_sums*& deferred() { return g_deferred; }

static std::atomic<int> g_exact_scan{0};
bool exact_scan() { return g_exact_scan.load(std::memory_order_relaxed) != 0; }

}  // namespace dbk

extern "C" {

const char* dbk_last_error(void) { return dbk::g_err; }

int dbk_version(void) { return 3; }

int dbk_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return -1;
    return n;
}

int dbk_set_exact_scan(int on)
{
    return dbk::g_exact_scan.exchange(on ? 1 : 0, std::memory_order_relaxed);
}

int dbk_sync(dbk_stream_t stream)
{
    DBK_HIP(hipStreamSynchronize(dbk::as_stream(stream)));
    dbk::clear_error();
    return 0;
}

}  // extern "C"

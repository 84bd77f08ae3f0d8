// Error state, version, device count, sync and the scratch workspace.
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

struct ws_t { hipStream_t stream = nullptr; void* ptr[2] = {nullptr, nullptr}; size_t bytes[2] = {0, 0}; bool used = false; };
constexpr int WS_DEVICES = 64, WS_STREAMS = 64;
static ws_t g_ws[WS_DEVICES][WS_STREAMS];
static std::mutex g_ws_mutex;

void* workspace(size_t bytes, hipStream_t stream, int which)
{
    int dev = 0;
    if (which < 0 || which > 1) return nullptr;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= WS_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    ws_t* w = nullptr;
    for (int i = 0; i < WS_STREAMS && !w; ++i) {
        ws_t& c = g_ws[dev][i];
        if (c.used ? c.stream == stream : true) w = &c;        // this stream's slot, or the first free one
    }
    if (!w) return nullptr;
    w->used = true;
    w->stream = stream;
    if (w->bytes[which] >= bytes && w->ptr[which]) return w->ptr[which];
    if (w->ptr[which]) {
        // earlier launches may still be reading the old buffer
        if (hipDeviceSynchronize() != hipSuccess) return nullptr;
        (void)hipFree(w->ptr[which]);
        w->ptr[which] = nullptr;
        w->bytes[which] = 0;
    }
    size_t want = bytes < (size_t(1) << 20) ? (size_t(1) << 20) : bytes + bytes / 4;
    if (hipMalloc(&w->ptr[which], want) != hipSuccess) { w->ptr[which] = nullptr; return nullptr; }
    w->bytes[which] = want;
    return w->ptr[which];
}

static thread_local deferred_sums* g_deferred = nullptr;
deferred_sums*& deferred() { return g_deferred; }

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

int dbk_sync(dbk_stream_t stream)
{
    DBK_HIP(hipStreamSynchronize(dbk::as_stream(stream)));
    dbk::clear_error();
    return 0;
}

}  // extern "C"

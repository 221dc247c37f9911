// Error reporting and version for libflashnn_hip.so.
#include "fnn_common.h"

#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <set>
#include <string>
#include <tuple>

namespace fnn {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

Call::Call(const char* fn) : fn(fn), prior(hipPeekAtLastError()) {}

int Call::done() const {
    const hipError_t e = hipPeekAtLastError();
    if (e == prior) return FNN_OK;     // nothing new; an error the caller's own HIP calls left stays theirs
    (void)hipGetLastError();           // ours: take it off the thread
    set_error("%s: HIP launch failed: %s", fn, hipGetErrorString(e));
    return FNN_ERR_HIP;
}

void allow_large_lds(const void* kernel, std::atomic<uint64_t>& raised) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;          // the launch that follows reports it
    const uint64_t bit = 1ull << (dev & 63);
    if (raised.load(std::memory_order_acquire) & bit) return;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess)
        raised.fetch_or(bit, std::memory_order_release);
}

// ---- which kernel ran ----------------------------------------------------------------------------
struct KernelNote { const char* name; int a, b, c; };
static thread_local KernelNote g_note = {"", 0, 0, 0};
static thread_local char g_note_text[160] = "";

static void format_note(const KernelNote& n, char* out, size_t cap) {
    if (n.a == 0 && n.b == 0 && n.c == 0) snprintf(out, cap, "%s", n.name);
    else snprintf(out, cap, "%s<%d,%d,%d>", n.name, n.a, n.b, n.c);
}

static bool log_enabled() {
    static const bool on = [] {
        const char* v = getenv("FLASHNN_HIP_LOG");
        return v && v[0] && strcmp(v, "0") != 0;
    }();
    return on;
}

void note_kernel(const char* name, int a, int b, int c) {
    g_note = KernelNote{name, a, b, c};
    if (!log_enabled()) return;
    // one line per kernel variant and process, the first time it is launched
    static std::mutex mu;
    static std::set<std::tuple<std::string, int, int, int>> seen;
    std::lock_guard<std::mutex> lock(mu);
    if (!seen.emplace(name, a, b, c).second) return;
    char text[160];
    format_note(g_note, text, sizeof(text));
    fprintf(stderr, "[flashnn_hip] first launch of %s\n", text);
}

}  // namespace fnn

extern "C" int fnn_version(void) { return 2; }
extern "C" const char* fnn_last_error(void) { return fnn::g_err; }
extern "C" const char* fnn_last_kernel(void) {
    fnn::format_note(fnn::g_note, fnn::g_note_text, sizeof(fnn::g_note_text));
    return fnn::g_note_text;
}

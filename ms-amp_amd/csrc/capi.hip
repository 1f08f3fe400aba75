// Library-wide pieces of the C ABI: version and the thread-local error string.
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "common.cuh"

namespace msamp {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return MSAMP_ERR_HIP - static_cast<int>(e);
}

// ---- kernels whose workgroups wait for each other ---------------------------------------------
// Two such kernels half-resident on one chip could wait for each other forever, so at any time they are kept to
// one stream per device, out of stream capture (a replay would reuse the token), and can be switched off
// altogether with MSAMP_INTIME_MODE=0 in the environment.  The stream that holds a device keeps it while it has
// work in flight; another stream that asks takes the device over once the holder has gone idle (or no longer
// exists), so a warm-up on a side stream does not tie the device to that stream for the life of the process.
static std::atomic<uint32_t> g_token{0};
static std::mutex g_owner_mutex;
static hipStream_t g_owner_stream[64];
static bool g_owner_set[64];
static int g_waiting_kernels = -1;

bool waiting_kernels_allowed(hipStream_t st) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    // a capturing stream never runs them, and must not take the device from the stream that does
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone) return false;
    std::lock_guard<std::mutex> lock(g_owner_mutex);
    if (g_waiting_kernels < 0) {
        const char* e = getenv("MSAMP_INTIME_MODE");
        g_waiting_kernels = e ? (atoi(e) != 0) : 1;
    }
    if (!g_waiting_kernels) return false;
    if (!g_owner_set[dev]) {
        g_owner_set[dev] = true;
        g_owner_stream[dev] = st;
        return true;
    }
    if (g_owner_stream[dev] == st) return true;
    // Another stream holds the device.  hipSuccess: everything it was given has completed, so none of its waiting
    // kernels is on the chip.  hipErrorNotReady: busy, the caller takes the two-pass kernels.  Anything else (the
    // handle was destroyed, the holder is being captured): its kernels cannot be running either way, but leave the
    // error out of the caller's sight.
    const hipError_t q = hipStreamQuery(g_owner_stream[dev]);
    if (q == hipErrorNotReady) return false;
    if (q != hipSuccess) (void)hipGetLastError();
    if (q == hipErrorStreamCaptureUnsupported || q == hipErrorStreamCaptureImplicit) return false;
    g_owner_stream[dev] = st;
    return true;
}

static std::atomic<uint32_t> g_spin_limit{1u << 20};    // a fraction of a second of polling

uint32_t collector_spin_limit() { return g_spin_limit.load(std::memory_order_relaxed); }

uint32_t next_tokens(uint32_t count) {
    for (;;) {
        const uint32_t first = g_token.fetch_add(count) + 1;
        if (first != 0 && first + count - 1 >= first) return first;    // skip 0 and a range that wraps
    }
}

}    // namespace msamp

extern "C" {

int msamp_hip_version(void) { return 100; }

const char* msamp_last_error(void) { return msamp::g_err; }

void msamp_set_spin_limit(uint32_t polls) { msamp::g_spin_limit.store(polls, std::memory_order_relaxed); }

int msamp_check_async_error(void* workspace, msamp_stream_t stream) {
    // a null workspace stands for the library's own (msamp_cast_to_fp8_intime_static) on the current device
    if (workspace == nullptr) {
        const int rc = msamp::static_workspace(&workspace);
        if (rc != MSAMP_OK) return rc;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint32_t* word = static_cast<uint32_t*>(workspace) + msamp::kWsErrorWord;
    uint32_t code = 0;
    hipError_t e = hipMemcpyAsync(&code, word, sizeof(code), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return msamp::hip_fail(e, "msamp_check_async_error: reading the error word");
    if (code == 0) return MSAMP_OK;
    const uint32_t zero = 0;
    e = hipMemcpyAsync(word, &zero, sizeof(zero), hipMemcpyHostToDevice, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return msamp::hip_fail(e, "msamp_check_async_error: clearing the error word");
    msamp::set_error("a kernel whose workgroups wait for each other gave up waiting (code %u: %s%s): the tensor and meta it "
                     "wrote are invalid; repeat the call with MSAMP_FLAG_TWO_PASS",
                     code, (code & msamp::kErrCollectorGaveUp) ? "collecting workgroup " : "",
                     (code & msamp::kErrFollowerGaveUp) ? "waiting workgroup" : "");
    return MSAMP_ERR_TIMEOUT;
}

}    // extern "C"

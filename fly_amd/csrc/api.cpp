// Process-wide pieces of the C ABI: version and the thread-local error string.
#include "common.h"

namespace flyhip {
char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

namespace {
constexpr int MAX_DEVICES = 64;
Machine g_machine[MAX_DEVICES + 1];
std::atomic<int> g_machine_ready[MAX_DEVICES + 1];
}  // namespace

const Machine& machine() {
    int dev = 0;
    const bool have = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < MAX_DEVICES;
    const int slot = have ? dev : MAX_DEVICES;
    if (!g_machine_ready[slot].load(std::memory_order_acquire)) {
        Machine m{256, 8, 512};
        int v = 0;
        if (have && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) m.cus = v;
        if (have && hipDeviceGetAttribute(&v, hipDeviceAttributeNumberOfXccs, dev) == hipSuccess && v > 0) m.xcds = v;
        if (!have) (void)hipGetLastError();                 // (no device: leave no sticky error behind)
        m.slots = 2 * m.cus;
        g_machine[slot] = m;                                 // (racing threads write the same values)
        g_machine_ready[slot].store(1, std::memory_order_release);
    }
    return g_machine[slot];
}

int ensure_dynamic_lds(const void* kernel, size_t bytes, std::atomic<unsigned long long>& done, const char* what) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    const unsigned long long bit = 1ull << dev;
    if (done.load(std::memory_order_acquire) & bit) return OK;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return fail(ERR_LAUNCH, "%s: LDS attribute: %s", what, hipGetErrorString(e));
    done.fetch_or(bit, std::memory_order_release);
    return OK;
}

int refuse_capture(hipStream_t st) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    const hipError_t e = hipStreamIsCapturing(st, &status);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(ERR_UNSUPPORTED, "the stream cannot be launched on (%s): another stream of this process is under graph "
                                     "capture, and calls of this library are not capturable", hipGetErrorString(e));
    }
    if (status != hipStreamCaptureStatusNone)
        return fail(ERR_UNSUPPORTED, "the stream is under graph capture: calls of this library are not capturable "
                                     "(run them eagerly, outside the capture)");
    return OK;
}
}  // namespace flyhip

extern "C" int flyhip_version(void) { return 100; }
extern "C" const char* flyhip_last_error(void) { return flyhip::error_buffer(); }

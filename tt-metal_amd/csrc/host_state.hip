// Host-side state of libttmi that outlives a call: the library's own device scratch, the per-device error word that
// kernels raise when a bounded wait gives up, and the knobs of the test entry point.
#include <atomic>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "ttmi_internal.h"

namespace ttmi {

// ---------------------------------------------------------------------------------------------------------
// Scratch.  One buffer per (purpose, device, stream): launches on one stream run in stream order, so they may share a
// buffer; launches on different streams may overlap, so they never do.  A buffer that has become too small is replaced
// by a larger one and RETIRED, not freed: a kernel queued by another host thread may still be about to use it, and
// hipFree would have to wait for the whole device.  Retired buffers are kept until the process ends (sizes grow
// geometrically, so they add up to less than the live buffer).
// ---------------------------------------------------------------------------------------------------------
namespace {
struct Buffer { void *ptr = nullptr; size_t bytes = 0; uint64_t generation = 0; };
struct Key {
    int kind, device; hipStream_t stream;
    bool operator<(const Key &o) const {
        if (kind != o.kind) return kind < o.kind;
        if (device != o.device) return device < o.device;
        return stream < o.stream;
    }
};
std::mutex g_guard;
std::atomic<uint64_t> g_allocations{0};          // hipMalloc / hipHostMalloc calls this library has made (a test reads it)
std::map<Key, Buffer> g_live;
struct Retired { void *ptr; size_t bytes; int device; };
std::vector<Retired> g_retired;
uint64_t g_generation[SCRATCH_KINDS] = {};       // raised by scratch_invalidate: contents of every buffer of that kind are suspect
}  // namespace

size_t scratch_grown_size(size_t have, size_t need) {
    if (need <= have) return have;
    const size_t doubled = have * 2;
    const size_t want = doubled > need ? doubled : need;
    return (want + 255) & ~(size_t)255;
}

int scratch_get(int kind, hipStream_t stream, size_t bytes, void **ptr, bool *fresh, size_t *capacity) {
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    std::lock_guard<std::mutex> lock(g_guard);
    Buffer &b = g_live[Key{kind, dev, stream}];
    *fresh = false;
    if (b.bytes < bytes) {
        const size_t size = scratch_grown_size(b.bytes, bytes);
        void *p = nullptr;
        if (int rc = check_hip(hipMalloc(&p, size), "hipMalloc(library scratch)")) return rc;
        ++g_allocations;
        if (b.ptr) g_retired.push_back(Retired{b.ptr, b.bytes, dev});
        b.ptr = p; b.bytes = size;
        *fresh = true;
    }
    if (b.generation != g_generation[kind]) { b.generation = g_generation[kind]; *fresh = true; }
    *ptr = b.ptr;
    if (capacity) *capacity = b.bytes;
    return TTMI_OK;
}

uint64_t scratch_generation(int kind) {
    std::lock_guard<std::mutex> lock(g_guard);
    return g_generation[kind];
}

// after this, scratch_get reports every buffer of that kind as fresh once (its owner initialises it again)
void scratch_invalidate(int kind) {
    std::lock_guard<std::mutex> lock(g_guard);
    ++g_generation[kind];
}

// ---------------------------------------------------------------------------------------------------------
// Error word: four bytes of pinned host memory per device that kernels can write (a plain vector store through the
// device's mapping of it) and the host can read without synchronising.  A kernel raises it when a bounded wait gives up;
// the next call on that device reports it.
// ---------------------------------------------------------------------------------------------------------
namespace {
struct ErrorWord { volatile uint32_t *host = nullptr; uint32_t *device = nullptr; };
ErrorWord g_error_word[64];
}  // namespace

int error_word(uint32_t **device_ptr, volatile uint32_t **host_ptr) {
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (dev < 0 || dev >= 64) return fail(TTMI_ERR_UNSUPPORTED, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_guard);
    ErrorWord &w = g_error_word[dev];
    if (!w.host) {
        void *h = nullptr, *d = nullptr;
        if (int rc = check_hip(hipHostMalloc(&h, 64, hipHostMallocMapped), "hipHostMalloc(error word)")) return rc;
        ++g_allocations;
        *reinterpret_cast<volatile uint32_t *>(h) = 0;
        if (int rc = check_hip(hipHostGetDevicePointer(&d, h, 0), "hipHostGetDevicePointer(error word)")) return rc;
        w.host = reinterpret_cast<volatile uint32_t *>(h);
        w.device = reinterpret_cast<uint32_t *>(d);
    }
    if (device_ptr) *device_ptr = w.device;
    if (host_ptr) *host_ptr = w.host;
    return TTMI_OK;
}

// The same without creating it: false when this device has no error word yet.
bool error_word_if_exists(uint32_t **device_ptr, volatile uint32_t **host_ptr) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    std::lock_guard<std::mutex> lock(g_guard);
    const ErrorWord &w = g_error_word[dev];
    if (!w.host) return false;
    if (device_ptr) *device_ptr = w.device;
    if (host_ptr) *host_ptr = w.host;
    return true;
}

#ifdef TTMI_TEST_HOOKS
// ---------------------------------------------------------------------------------------------------------
// Test knobs (ttmi_test_set_knob): which kernel, how many workgroups, which block form, the spin limit of the bounded
// waits, and whether producers keep their partial sums to themselves.  Product code never sets them.
// ---------------------------------------------------------------------------------------------------------
namespace {
std::atomic<uint32_t> g_knob[TTMI_KNOB_COUNT];
std::atomic<bool> g_knob_set[TTMI_KNOB_COUNT];
}  // namespace

bool knob(int which, uint32_t *value) {
    if (which < 0 || which >= TTMI_KNOB_COUNT || !g_knob_set[which].load(std::memory_order_relaxed)) return false;
    *value = g_knob[which].load(std::memory_order_relaxed);
    return true;
}

uint32_t knob_or(int which, uint32_t fallback) {
    uint32_t v;
    return knob(which, &v) ? v : fallback;
}

#endif

}  // namespace ttmi

using namespace ttmi;

extern "C" {

#ifdef TTMI_TEST_HOOKS
// Test entry point (not declared in include/ttmi.h): sets knob `which` to `value`, or clears it when `set` is 0.
__attribute__((visibility("default"))) int ttmi_test_set_knob(int which, uint32_t value, int set) {
    if (which < 0 || which >= TTMI_KNOB_COUNT) return fail(TTMI_ERR_INVALID_ARGUMENT, "unknown test knob %d", which);
    g_knob[which].store(value, std::memory_order_relaxed);
    g_knob_set[which].store(set != 0, std::memory_order_relaxed);
    return TTMI_OK;
}
#endif

// What a kernel has reported since the last query on the current device: TTMI_OK, or TTMI_ERR_HIP with the message in
// ttmi_last_error().  Clears the report.
int ttmi_device_status(void) {
    volatile uint32_t *host = nullptr;
    if (int rc = error_word(nullptr, &host)) return rc;
    const uint32_t raised = *host;
    if (!raised) return TTMI_OK;
    *host = 0;
    scratch_invalidate(SCRATCH_SLOTS);
    return fail(TTMI_ERR_HIP, "a matmul kernel gave up waiting for the partial sums of another workgroup (code %u): the output of every matmul "
                "launched on this device since the last status check is suspect", raised);
}

int ttmi_release_scratch(size_t *freed_bytes) {
    int dev = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (int rc = check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize")) return rc;      // nothing queued may still be about to use a buffer
    size_t freed = 0;
    std::lock_guard<std::mutex> lock(g_guard);
    for (auto it = g_live.begin(); it != g_live.end();) {
        if (it->first.device == dev) {
            if (it->second.ptr) { (void)hipFree(it->second.ptr); freed += it->second.bytes; }
            it = g_live.erase(it);
        } else {
            ++it;
        }
    }
    for (size_t i = 0; i < g_retired.size();) {
        if (g_retired[i].device == dev) {
            (void)hipFree(g_retired[i].ptr); freed += g_retired[i].bytes;
            g_retired[i] = g_retired.back(); g_retired.pop_back();
        } else {
            ++i;
        }
    }
    if (freed_bytes) *freed_bytes = freed;
    return TTMI_OK;
}

#ifdef TTMI_TEST_HOOKS
// Test entry point: how many allocations (device scratch, the pinned error word) the library has made in this process.
__attribute__((visibility("default"))) uint64_t ttmi_test_allocations(void) { return g_allocations.load(); }

// Test entry point: the size a library buffer of `have` bytes grows to when `need` bytes are asked for.
__attribute__((visibility("default"))) size_t ttmi_test_scratch_grown_size(size_t have, size_t need) { return scratch_grown_size(have, need); }
#endif

}  // extern "C"

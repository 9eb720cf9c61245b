// The library's per-GPU launch status word, the bound of the kernels' waits, and the calls that
// set a process up ahead of time (qmoe_init) and read the word back (qmoe_check_status).
#include <atomic>
#include <mutex>

#include "qmoe_common.hpp"

namespace qmoe {

// Its name is a host-side stand-in, not a device address: the address is asked for once per device,
// with that device current, and only that pointer reaches kernels and copies.
static __device__ __align__(16) uint32_t launch_status[4];

int launch_status_word(uint32_t** out) {
    static constexpr int MAX_DEVICES = 64;
    static std::mutex lock;
    static uint32_t* per_device[MAX_DEVICES] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
        return fail(QMOE_ELAUNCH, "launch status word: no current HIP device");
    std::lock_guard<std::mutex> guard(lock);
    if (!per_device[dev]) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(launch_status));
        if (e != hipSuccess || !ptr) return fail(QMOE_ELAUNCH, "launch status word: %s", hipGetErrorString(e));
        per_device[dev] = (uint32_t*)ptr;
    }
    *out = per_device[dev];
    return QMOE_OK;
}

// One second of the 100 MHz counter: a launch that streams all of a GPU's memory takes a twentieth of it.
static constexpr int64_t DEFAULT_WAIT_TICKS = 100 * 1000 * 1000;
static std::atomic<int64_t> g_wait_ticks{DEFAULT_WAIT_TICKS};
int64_t wait_limit_ticks() { return g_wait_ticks.load(std::memory_order_relaxed); }

}  // namespace qmoe

using namespace qmoe;

extern "C" {

int qmoe_init(void) {
    uint32_t* word = nullptr;
    if (int rc = launch_status_word(&word)) return rc;
    void* area = nullptr;
    return static_scratch(&area);
}

int qmoe_check_status(void* stream) {
    uint32_t* word = nullptr;
    if (int rc = launch_status_word(&word)) return rc;
    hipStream_t s = (hipStream_t)stream;
    uint32_t seen[4] = {0, 0, 0, 0};
    hipError_t e = hipMemcpyAsync(seen, word, sizeof(seen), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) return fail(QMOE_ELAUNCH, "qmoe_check_status: %s", hipGetErrorString(e));
    if (!seen[0]) return QMOE_OK;
    const uint32_t zero[4] = {0, 0, 0, 0};
    e = hipMemcpyAsync(word, zero, sizeof(zero), hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) return fail(QMOE_ELAUNCH, "qmoe_check_status: clearing the word: %s", hipGetErrorString(e));
    return fail(QMOE_ELAUNCH, "a streaming launch gave up a bounded wait for the other waves of its workgroup (status %u): "
                "that launch's outputs are incomplete", seen[0]);
}

void qmoe_set_wait_limit(long long ticks) { g_wait_ticks.store(ticks ? (int64_t)ticks : DEFAULT_WAIT_TICKS, std::memory_order_relaxed); }

}  // extern "C"

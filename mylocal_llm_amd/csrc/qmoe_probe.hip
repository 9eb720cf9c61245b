// A pure streaming read of a device buffer: the ceiling against which the weight-streaming
// kernels are read.  Every byte is loaded once with 16-byte loads into registers, folded into a
// checksum and dropped; nothing is decoded and nothing is written (the checksum leaves only when
// it equals a value the caller chooses, so the loads cannot be optimised away).  The launch has
// the shape of the streaming kernels: one workgroup of eight waves per CU, each wave walking
// 4 KB items (four 1 KB requests of 64 lanes x 16 bytes) with the next item already in flight.
#include "qmoe_common.hpp"

namespace qmoe {

__global__ __launch_bounds__(512, 1) void read_probe_kernel(const uint8_t* __restrict__ base, long items, uint32_t match,
                                                            uint32_t* __restrict__ sink) {
    const int lane = threadIdx.x & 63;
    const long waves = (long)gridDim.x * 8, me = (long)blockIdx.x * 8 + (threadIdx.x >> 6);
    u32x4_t now[4], next[4];
    uint32_t sum = 0;
    auto fetch = [&](long item, u32x4_t* r) {
        const uint8_t* p = base + (item < items ? item : items - 1) * 4096 + lane * 16;
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = ldg_u32x4<16>(p + j * 1024);
    };
    fetch(me, now);
    for (long item = me; item < items; item += waves) {
        fetch(item + waves, next);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            sum ^= now[j][0] ^ now[j][1] ^ now[j][2] ^ now[j][3];
            now[j] = next[j];
        }
    }
    if (sum == match) sink[0] = sum;
}

}  // namespace qmoe

using namespace qmoe;

extern "C" int qmoe_read_probe(const void* buffer, size_t bytes, uint32_t match, uint32_t* sink, void* stream) {
    if (!buffer || !sink) return fail(QMOE_EINVAL, "qmoe_read_probe: null pointer");
    if (bytes < 4096 || bytes % 4096 || (uintptr_t)buffer % 16)
        return fail(QMOE_EINVAL, "qmoe_read_probe: %zu bytes: a positive multiple of 4096 from a 16-byte aligned address", bytes);
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus < 1)
        return fail(QMOE_ELAUNCH, "qmoe_read_probe: cannot read the device's CU count");
    hipLaunchKernelGGL(read_probe_kernel, dim3(cus), dim3(512), 0, (hipStream_t)stream, (const uint8_t*)buffer,
                       (long)(bytes / 4096), match, sink);
    return check_launch("qmoe_read_probe");
}

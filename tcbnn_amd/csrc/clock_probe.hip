// Shader clock actually running, for reading a measured rate against peaks that are quoted at the nominal clock:
// one wave counts shader cycles (s_memtime) over a stretch of the constant-rate wall clock (s_memrealtime) while
// whatever else the caller has queued runs beside it.  No counterpart in the reference.
#include "common.h"

namespace tcbnn {
namespace {

__global__ __launch_bounds__(64) void clock_probe_kernel(unsigned long long* __restrict__ out, unsigned long long ticks) {
    const unsigned long long t0 = wall_clock64();
    const unsigned long long c0 = clock64();
    unsigned long long t1 = t0;
    // bounded: the wall clock always advances
    while (t1 - t0 < ticks) {
        __builtin_amdgcn_s_sleep(64);
        t1 = wall_clock64();
    }
    const unsigned long long c1 = clock64();
    t1 = wall_clock64();
    if (threadIdx.x == 0) {
        out[0] = c1 - c0;
        out[1] = t1 - t0;
    }
}

}  // namespace
}  // namespace tcbnn

using namespace tcbnn;

extern "C" int tcbnn_shader_clock_probe(unsigned long long* counts, int microseconds, int* wall_clock_khz, void* stream) {
    TCBNN_NOTNULL(counts);
    TCBNN_NOTNULL(wall_clock_khz);
    TCBNN_REQUIRE(microseconds > 0 && microseconds <= 1000000, "shader_clock_probe: 1 .. 1000000 microseconds");
    int dev = 0, khz = 0;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (int rc = check_hip(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev),
                           "hipDeviceGetAttribute(WallClockRate)"))
        return rc;
    TCBNN_REQUIRE(khz > 0, "shader_clock_probe: the device reports no wall clock rate");
    *wall_clock_khz = khz;
    const unsigned long long ticks = (unsigned long long)khz * (unsigned long long)microseconds / 1000ull;
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, counts, ticks);
    TCBNN_LAUNCH_CHECK("clock_probe_kernel");
    return TCBNN_OK;
}

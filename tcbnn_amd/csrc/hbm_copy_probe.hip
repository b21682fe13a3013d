// hbm_copy_probe: a plain device copy kernel of known size.
//
// Hardware counters of HBM traffic (FETCH_SIZE, WRITE_SIZE of the L2/TCC block) are read per
// dispatch by a profiler.  This program gives them a dispatch whose traffic is known exactly --
// `bytes` read once and `bytes` written once, in 16-byte accesses, far larger than the caches --
// so that the counter readings of the library's kernels can be scaled by the same factor.
// It also prints the copy's bandwidth, the practical HBM ceiling of the device.
//
//   hbm_copy_probe [MiB=1024] [launches=5]
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

#define CHECK(x)                                                                              \
    do {                                                                                      \
        hipError_t e_ = (x);                                                                  \
        if (e_ != hipSuccess) {                                                               \
            fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
            return 1;                                                                         \
        }                                                                                     \
    } while (0)

__global__ __launch_bounds__(256) void hbm_copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                       size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

int main(int argc, char** argv) {
    const size_t mib = argc > 1 ? strtoull(argv[1], nullptr, 10) : 1024;
    const int launches = argc > 2 ? atoi(argv[2]) : 5;
    if (mib == 0 || mib > 16384 || launches < 1 || launches > 1000) {
        fprintf(stderr, "usage: hbm_copy_probe [MiB 1..16384] [launches 1..1000]\n");
        return 2;
    }
    const size_t bytes = mib << 20, n16 = bytes / 16;
    uint4 *src = nullptr, *dst = nullptr;
    CHECK(hipMalloc(&src, bytes));
    CHECK(hipMalloc(&dst, bytes));
    CHECK(hipMemset(src, 0x5a, bytes));
    CHECK(hipMemset(dst, 0, bytes));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    const int grid = 256 * 16;
    hbm_copy_kernel<<<grid, 256>>>(dst, src, n16);  // warm-up
    CHECK(hipDeviceSynchronize());
    float best = 1e30f, sum = 0.f;
    for (int i = 0; i < launches; ++i) {
        CHECK(hipEventRecord(e0));
        hbm_copy_kernel<<<grid, 256>>>(dst, src, n16);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        best = ms < best ? ms : best;
        sum += ms;
    }
    CHECK(hipGetLastError());
    printf("{\"kernel\": \"hbm_copy_kernel\", \"bytes_read_per_launch\": %zu, \"bytes_written_per_launch\": %zu, "
           "\"launches\": %d, \"avg_ms\": %.4f, \"best_ms\": %.4f, \"read_plus_write_gbs_avg\": %.1f}\n",
           bytes, bytes, launches + 1, sum / launches, best, 2.0 * bytes / (sum / launches * 1e-3) / 1e9);
    CHECK(hipFree(src));
    CHECK(hipFree(dst));
    return 0;
}

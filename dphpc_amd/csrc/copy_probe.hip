// Plain copy kernel of known size: the yardstick for rocprofv3's FETCH_SIZE /
// WRITE_SIZE counters.  usage: copy_probe [bytes] [reps]
// Reads `bytes` and writes `bytes` per launch, 16 bytes per lane, grid-stride.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

__global__ __launch_bounds__(256) void copy_probe_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); return 1; } } while (0)

int main(int argc, char **argv) {
    const size_t bytes = argc > 1 ? strtoull(argv[1], nullptr, 10) : (size_t)1 << 30;
    const int reps = argc > 2 ? atoi(argv[2]) : 5;
    const size_t n = bytes / sizeof(uint4);
    uint4 *src = nullptr, *dst = nullptr;
    CHECK(hipMalloc((void **)&src, n * sizeof(uint4)));
    CHECK(hipMalloc((void **)&dst, n * sizeof(uint4)));
    CHECK(hipMemset(src, 1, n * sizeof(uint4)));
    CHECK(hipMemset(dst, 0, n * sizeof(uint4)));
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a));
    CHECK(hipEventCreate(&b));
    float best = 1e30f;
    for (int r = 0; r < reps; ++r) {
        CHECK(hipEventRecord(a, 0));
        hipLaunchKernelGGL(copy_probe_kernel, dim3(256 * 16), dim3(256), 0, 0, src, dst, n);
        CHECK(hipEventRecord(b, 0));
        CHECK(hipEventSynchronize(b));
        float ms = 0.f;
        CHECK(hipEventElapsedTime(&ms, a, b));
        if (ms < best) best = ms;
    }
    printf("copy_probe bytes_read=%zu bytes_written=%zu best_ms=%.4f GBps=%.1f\n", n * sizeof(uint4), n * sizeof(uint4), best,
           2.0 * n * sizeof(uint4) / (best * 1e-3) / 1e9);
    CHECK(hipFree(src));
    CHECK(hipFree(dst));
    return 0;
}

// Calibration of rocprofv3's FETCH_SIZE / WRITE_SIZE counters: one plain copy kernel that reads
// MiB and writes MiB per launch (16-byte integer vectors, non-temporal, nothing else), so that the
// ratio of the counter readings to the known sizes turns the same counters, read for a scan kernel,
// into bytes of HBM traffic. Not part of the library: `make calib` builds build/copy_calib.
//   copy_calib [MiB = 1024] [launches = 20]
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

typedef unsigned u4 __attribute__((ext_vector_type(4)));

#define CHECK(call)                                                        \
    do {                                                                   \
        const hipError_t e_ = (call);                                      \
        if (e_ != hipSuccess) {                                            \
            fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));     \
            return 1;                                                      \
        }                                                                  \
    } while (0)

// A workgroup of 256 lanes moves 1024 consecutive vectors, four per lane.
__global__ __launch_bounds__(256) void copy_calib_kernel(const u4 *__restrict__ in, u4 *__restrict__ out, size_t n)
{
    size_t i = (size_t)blockIdx.x * 1024 + threadIdx.x;
#pragma unroll
    for (int k = 0; k < 4; k++, i += 256)
        if (i < n) __builtin_nontemporal_store(__builtin_nontemporal_load(in + i), out + i);
}

int main(int argc, char **argv)
{
    const size_t mib = argc > 1 ? (size_t)atol(argv[1]) : 1024;
    const int launches = argc > 2 ? atoi(argv[2]) : 20;
    if (mib < 1 || mib > 65536 || launches < 1) {
        fprintf(stderr, "usage: %s [MiB] [launches]\n", argv[0]);
        return 2;
    }
    const size_t bytes = mib << 20, n = bytes / sizeof(u4);
    u4 *in = nullptr, *out = nullptr;
    CHECK(hipMalloc(&in, bytes));
    CHECK(hipMalloc(&out, bytes));
    CHECK(hipMemset(in, 1, bytes));
    CHECK(hipMemset(out, 0, bytes));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    const dim3 grid((unsigned)((n + 1023) / 1024)), block(256);
    hipLaunchKernelGGL(copy_calib_kernel, grid, block, 0, 0, in, out, n);  // warm-up
    CHECK(hipEventRecord(e0, 0));
    for (int i = 0; i < launches; i++) hipLaunchKernelGGL(copy_calib_kernel, grid, block, 0, 0, in, out, n);
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    ms /= launches;
    printf("copy_calib: %zu MiB read + %zu MiB written per launch, %d launches, %.1f us per launch, %.1f GB/s\n", mib,
           mib, launches + 1, ms * 1e3, 2.0 * bytes / (ms * 1e-3) / 1e9);
    CHECK(hipDeviceSynchronize());
    CHECK(hipFree(in));
    CHECK(hipFree(out));
    return 0;
}

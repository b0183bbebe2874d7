// Plain copy kernel of known size, used only to calibrate the FETCH_SIZE and
// WRITE_SIZE counters of rocprofv3 (what they read for N bytes in, N bytes out).
//   hipcc -O3 --offload-arch=gfx950 copy_calib.hip -o copy_calib && ./copy_calib [MiB]
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

typedef unsigned u4 __attribute__((ext_vector_type(4)));

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
    const size_t bytes = mib << 20, n = bytes / 16;
    u4 *in, *out;
    if (hipMalloc(&in, bytes) != hipSuccess || hipMalloc(&out, bytes) != hipSuccess) return 1;
    hipMemset(in, 1, bytes);
    hipMemset(out, 0, bytes);
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    const int reps = 20;
    for (int r = 0; r < reps + 3; r++) {
        if (r == 3) hipEventRecord(e0, 0);
        hipLaunchKernelGGL(copy_calib_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, 0, in, out, n);
    }
    hipEventRecord(e1, 0);
    hipEventSynchronize(e1);
    float ms = 0;
    hipEventElapsedTime(&ms, e0, e1);
    printf("copy_calib: %zu MiB read + %zu MiB written per launch, %.1f us per launch, %.1f GB/s\n", mib, mib,
           ms * 1e3 / reps, 2.0 * bytes * reps / (ms * 1e-3) / 1e9);
    return hipDeviceSynchronize() == hipSuccess ? 0 : 1;
}

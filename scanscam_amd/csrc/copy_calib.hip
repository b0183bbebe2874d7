// Calibration of rocprofv3's FETCH_SIZE / WRITE_SIZE counters: one plain copy kernel that reads
// MiB and writes MiB per launch (16-byte integer vectors, non-temporal, nothing else), so that the
// ratio of the counter readings to the known sizes turns the same counters, read for a scan kernel,
// into bytes of HBM traffic. Not part of the library: `make calib` builds build/copy_calib.
//   copy_calib [MiB = 1024] [launches = 20]
// Two further modes stream without scanning, in the scan kernels' access shapes, to show what the memory
// system gives those shapes when no scan, no ticket and no carry chain is involved:
//   copy_calib mix      each mix of read and write streams (1R0W ... 3R2W; forward scan = 2R1W, backward = 3R2W),
//                       67 108 864 fp32 per stream, and each workgroup shape (W waves x U 16-byte accesses per lane
//                       and stream, all loads issued before the first store), 4 rotated buffer sets;
//   copy_calib order    the look-back tile (8 waves x 4 accesses) in the look-back kernel's tile-major order of
//                       work: the stream is cut into R rows and workgroup k takes tile k / R of row k % R, so tiles
//                       of all R rows are in flight together (R = 1 is one linear sweep).
//   copy_calib cl       channels-last tensors [B, T, C]: a workgroup's waves are `side` channel spans side by side
//                       (64 lanes x the lane's bytes each) times `spans` spans of S time steps, tiles of time handed
//                       out over workgroups as in the time-split kernel. side = 1 is that kernel's shape (a wave
//                       reads pieces of a time step, one row of C apart); side = all spans of a time step makes a
//                       workgroup's tile one contiguous block of memory.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

typedef unsigned u4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));

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

// READS input and WRITES output streams in the scan kernels' shape: workgroup k covers W * U consecutive 1 KiB
// spans of every stream (wave w its U spans), or, with R > 1, tile k / R of row k % R of a stream cut into R rows.
template <int READS, int WRITES, int U, int W>
__global__ __launch_bounds__(W * 64) void stream_kernel(const f4 *__restrict__ a, const f4 *__restrict__ b,
                                                         const f4 *__restrict__ c, f4 *__restrict__ o0,
                                                         f4 *__restrict__ o1, unsigned R, size_t row_vecs, float never)
{
    const size_t base = (size_t)(blockIdx.x % R) * row_vecs + (size_t)(blockIdx.x / R) * (W * U * 64) +
                        (threadIdx.x / 64) * (U * 64) + (threadIdx.x % 64);
    f4 va[U], vb[U], vc[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        va[u] = __builtin_nontemporal_load(a + base + u * 64);
        if (READS > 1) vb[u] = __builtin_nontemporal_load(b + base + u * 64);
        if (READS > 2) vc[u] = __builtin_nontemporal_load(c + base + u * 64);
    }
    if (WRITES == 0) {  // the sum of what was read is compared with a value it never takes, so the loads stay
        f4 s = 0;
#pragma unroll
        for (int u = 0; u < U; u++) {
            s += va[u];
            if (READS > 1) s += vb[u];
            if (READS > 2) s += vc[u];
        }
        if (s.x + s.y + s.z + s.w == never) o0[base] = s;
        return;
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        f4 r = va[u];
        if (READS > 1) r += vb[u];
        if (READS > 2) r *= vc[u];
        __builtin_nontemporal_store(r, o0 + base + u * 64);
        if (WRITES > 1) __builtin_nontemporal_store(r + 1.0f, o1 + base + u * 64);
    }
}

// Channels-last shapes: lane vector V (4, 8 or 16 bytes), S time steps per wave. Workgroup k covers tile
// k / (batch * blocks) of (batch element, channel block) k % (batch * blocks); wave w is channel span w % side of
// the block and time span w / side of the tile.
template <typename V, int S, int READS, int WRITES>
__global__ __launch_bounds__(1024) void cl_stream_kernel(const char *__restrict__ a, const char *__restrict__ b,
                                                         const char *__restrict__ c, char *__restrict__ o0,
                                                         char *__restrict__ o1, int batch, int T, int row_bytes, int side)
{
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, spans = blockDim.x / 64 / side;
    const int span_bytes = 64 * (int)sizeof(V), blocks = (row_bytes + side * span_bytes - 1) / (side * span_bytes);
    const int pairs = batch * blocks, pair = blockIdx.x % pairs, tile = blockIdx.x / pairs;
    const int col = ((pair % blocks) * side + wave % side) * span_bytes + lane * (int)sizeof(V);
    const int t0 = (tile * spans + wave / side) * S;
    const size_t base = ((size_t)(pair / blocks) * T + t0) * row_bytes + col;
    const bool live = col + (int)sizeof(V) <= row_bytes;
    V va[S], vb[S], vc[S];
#pragma unroll
    for (int k = 0; k < S; k++) {
        const bool ok = live && t0 + k < T;
        const size_t at = ok ? base + (size_t)k * row_bytes : 0;
        va[k] = __builtin_nontemporal_load(reinterpret_cast<const V *>(a + at));
        if (READS > 1) vb[k] = __builtin_nontemporal_load(reinterpret_cast<const V *>(b + at));
        if (READS > 2) vc[k] = __builtin_nontemporal_load(reinterpret_cast<const V *>(c + at));
    }
#pragma unroll
    for (int k = 0; k < S; k++) {
        if (!(live && t0 + k < T)) continue;
        V r = va[k];
        if (READS > 1) r += vb[k];
        if (READS > 2) r *= vc[k];
        __builtin_nontemporal_store(r, reinterpret_cast<V *>(o0 + base + (size_t)k * row_bytes));
        if (WRITES > 1) __builtin_nontemporal_store(r + r, reinterpret_cast<V *>(o1 + base + (size_t)k * row_bytes));
    }
}

static const size_t kStreamElems = (size_t)16384 * 4096;  // fp32 per stream
static f4 *g_sets[4][5];

template <int READS, int WRITES, int U, int W> static int stream_case(unsigned R)
{
    const size_t vecs = kStreamElems / 4, tile_vecs = (size_t)W * U * 64;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    const int launches = 40;
    for (int i = -4; i < launches; i++) {
        f4 **s = g_sets[(i + 4) % 4];
        if (i == 0) CHECK(hipEventRecord(e0, 0));
        hipLaunchKernelGGL((stream_kernel<READS, WRITES, U, W>), dim3((unsigned)(vecs / tile_vecs)), dim3(W * 64), 0, 0,
                           s[0], s[1], s[2], s[3], s[4], R, vecs / R, -12345.0f);
    }
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    ms /= launches;
    const double bytes = (double)(READS + WRITES) * kStreamElems * 4;
    printf("  %dR%dW  %2d waves x %d accesses  %5u rows  %7.1f us  %7.1f GB/s  %4.1f %% of 8 TB/s\n", READS, WRITES, W, U, R,
           ms * 1e3, bytes / (ms * 1e-3) / 1e9, bytes / (ms * 1e-3) / 8e12 * 100);
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return 0;
}

template <typename V, int S, int READS, int WRITES> static int cl_case(int batch, int T, int row_bytes, int side, int spans)
{
    const int span_bytes = 64 * (int)sizeof(V), blocks = (row_bytes + side * span_bytes - 1) / (side * span_bytes);
    const int tiles = (T + spans * S - 1) / (spans * S);
    const size_t bytes_per_stream = (size_t)batch * T * row_bytes;
    if (bytes_per_stream > kStreamElems * 4 || side * spans > 16) return 1;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    const int launches = 40;
    for (int i = -4; i < launches; i++) {
        f4 **s = g_sets[(i + 4) % 4];
        if (i == 0) CHECK(hipEventRecord(e0, 0));
        hipLaunchKernelGGL((cl_stream_kernel<V, S, READS, WRITES>), dim3((unsigned)(batch * blocks * tiles)),
                           dim3(side * spans * 64), 0, 0, (const char *)s[0], (const char *)s[1], (const char *)s[2],
                           (char *)s[3], (char *)s[4], batch, T, row_bytes, side);
    }
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    ms /= launches;
    const double bytes = (double)(READS + WRITES) * bytes_per_stream;
    printf("  %dR%dW  %2d-byte lanes  %2d side by side x %2d spans x %2d steps  %5d workgroups  %7.1f us  %4.1f %%\n", READS, WRITES,
           (int)sizeof(V), side, spans, S, batch * blocks * tiles, ms * 1e3, bytes / (ms * 1e-3) / 8e12 * 100);
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return 0;
}

typedef float f2 __attribute__((ext_vector_type(2)));

template <typename V, int S> static int cl_both(int batch, int T, int row_bytes, int side, int spans)
{
    return cl_case<V, S, 2, 1>(batch, T, row_bytes, side, spans) | cl_case<V, S, 3, 2>(batch, T, row_bytes, side, spans);
}

static int run_cl()
{
    for (auto &set : g_sets)
        for (auto &p : set) {
            CHECK(hipMalloc(&p, kStreamElems * 4));
            CHECK(hipMemset(p, 0, kStreamElems * 4));
        }
    int rc = 0;
    printf("channels-last tile shapes, scan-free (forward mix 2R1W, backward mix 3R2W), 4 rotated buffer sets, %% of 8 TB/s:\n");
    printf("fp32 [8, 4096, 512] (time steps of 2048 bytes):\n");
    rc |= cl_both<f2, 16>(8, 4096, 2048, 1, 8) | cl_both<f2, 16>(8, 4096, 2048, 2, 4) | cl_both<f2, 16>(8, 4096, 2048, 4, 2) |
          cl_both<f2, 16>(8, 4096, 2048, 4, 4) | cl_both<f4, 8>(8, 4096, 2048, 1, 8) | cl_both<f4, 8>(8, 4096, 2048, 2, 4) |
          cl_both<f4, 8>(8, 4096, 2048, 2, 8) | cl_both<float, 16>(8, 4096, 2048, 1, 8) | cl_both<float, 16>(8, 4096, 2048, 8, 1) |
          cl_both<float, 16>(8, 4096, 2048, 8, 2);
    printf("16-bit [8, 4096, 512] (time steps of 1024 bytes):\n");
    rc |= cl_both<float, 16>(8, 4096, 1024, 1, 8) | cl_both<float, 16>(8, 4096, 1024, 4, 2) | cl_both<float, 16>(8, 4096, 1024, 4, 4) |
          cl_both<f2, 16>(8, 4096, 1024, 1, 8) | cl_both<f2, 16>(8, 4096, 1024, 2, 4) | cl_both<f2, 16>(8, 4096, 1024, 2, 8);
    printf("fp32 [8, 4096, 2048] (time steps of 8192 bytes):\n");
    rc |= cl_both<f2, 16>(8, 4096, 8192, 1, 8) | cl_both<f2, 16>(8, 4096, 8192, 4, 2) | cl_both<f2, 16>(8, 4096, 8192, 8, 1) |
          cl_both<f2, 16>(8, 4096, 8192, 16, 1) | cl_both<f4, 8>(8, 4096, 8192, 8, 1) | cl_both<f4, 8>(8, 4096, 8192, 8, 2);
    printf("fp32 [32, 2048, 1001] (time steps of 4004 bytes, no whole lines):\n");
    rc |= cl_both<float, 16>(32, 2048, 4004, 1, 8) | cl_both<float, 16>(32, 2048, 4004, 1, 16) | cl_both<float, 16>(32, 2048, 4004, 16, 1) |
          cl_both<float, 16>(32, 2048, 4004, 8, 2) | cl_both<float, 16>(32, 2048, 4004, 4, 4) | cl_both<float, 8>(32, 2048, 4004, 16, 1);
    printf("16-bit [90, 2048, 514] (time steps of 1028 bytes, no whole lines):\n");
    rc |= cl_both<float, 16>(90, 2048, 1028, 1, 8) | cl_both<float, 16>(90, 2048, 1028, 5, 1) | cl_both<float, 16>(90, 2048, 1028, 5, 2) |
          cl_both<float, 16>(90, 2048, 1028, 5, 3);
    printf("fp32 [32, 2048, 1024] (time steps of 4096 bytes; tiles only, a workgroup that walks all of T is not modelled):\n");
    rc |= cl_both<f2, 8>(32, 2048, 4096, 1, 8) | cl_both<f2, 8>(32, 2048, 4096, 8, 1) | cl_both<f2, 8>(32, 2048, 4096, 8, 2) |
          cl_both<f4, 8>(32, 2048, 4096, 4, 2) | cl_both<f4, 8>(32, 2048, 4096, 4, 4);
    CHECK(hipDeviceSynchronize());
    return rc;
}

static int run_streams(bool order)
{
    for (auto &set : g_sets)
        for (auto &p : set) {
            CHECK(hipMalloc(&p, kStreamElems * 4));
            CHECK(hipMemset(p, 0, kStreamElems * 4));
        }
    int rc = 0;
    if (!order) {
        printf("stream mixes, 67 108 864 fp32 per stream, non-temporal 16-byte accesses, 4 rotated buffer sets:\n");
        rc |= stream_case<1, 0, 4, 4>(1) | stream_case<2, 0, 4, 4>(1) | stream_case<3, 0, 4, 4>(1);
        rc |= stream_case<0 + 1, 1, 4, 4>(1) | stream_case<2, 1, 4, 4>(1) | stream_case<3, 2, 4, 4>(1);
        printf("forward mix (2 reads + 1 write) by workgroup shape:\n");
        rc |= stream_case<2, 1, 2, 4>(1) | stream_case<2, 1, 8, 4>(1) | stream_case<2, 1, 2, 8>(1) | stream_case<2, 1, 4, 8>(1) |
              stream_case<2, 1, 8, 8>(1) | stream_case<2, 1, 2, 16>(1) | stream_case<2, 1, 4, 16>(1);
        printf("backward mix (3 reads + 2 writes) by workgroup shape:\n");
        rc |= stream_case<3, 2, 2, 4>(1) | stream_case<3, 2, 2, 8>(1) | stream_case<3, 2, 4, 8>(1) | stream_case<3, 2, 2, 16>(1) |
              stream_case<3, 2, 4, 16>(1);
    } else {
        printf("order of work, 8 waves x 4 accesses (8192-element tiles), workgroup k -> tile k / R of row k %% R:\n");
        for (unsigned R : {1u, 8u, 32u, 64u, 128u, 256u, 1024u}) rc |= stream_case<2, 1, 4, 8>(R);
        for (unsigned R : {1u, 8u, 32u, 64u, 128u, 256u, 1024u}) rc |= stream_case<3, 2, 4, 8>(R);
    }
    CHECK(hipDeviceSynchronize());
    return rc;
}

int main(int argc, char **argv)
{
    if (argc > 1 && argv[1][0] == 'c') return run_cl();
    if (argc > 1 && (argv[1][0] == 'm' || argv[1][0] == 'o')) return run_streams(argv[1][0] == 'o');
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

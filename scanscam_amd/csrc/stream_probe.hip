// Measurement aid, not part of the library: plain streaming kernels of known size.
//
//   stream_probe copy [MiB]   one kernel that reads MiB and writes MiB: what rocprofv3's FETCH_SIZE and
//                             WRITE_SIZE counters read for a known number of bytes (their scale factors)
//   stream_probe ceiling [rows]  scan-free kernels with the access shape of the scan kernels at
//                             rows (default 16384) x 4096 fp32 (one 256-thread workgroup per row, four 16-byte
//                             non-temporal loads per lane per stream): 2 reads + 1 write like the
//                             forward scan, 3 reads + 2 writes like the backward scan. What the memory
//                             system gives that access shape when no scan is done at all.
//   stream_probe policy [rows]   the same two shapes with every combination of the sc0 / sc1 / nt cache-policy bits on
//                             the loads or on the stores, over 8 rotated buffer sets so that no cache level can
//                             hold an output between launches. Shows which policy the kernels should use.
//   stream_probe mix             what the memory system gives each mix of read and write streams (1R0W ... 3R2W,
//                             268 MB per stream, 4 rotated buffer sets) and each workgroup shape (W waves x U
//                             16-byte accesses per lane per stream): the ceilings the scan kernels are measured
//                             against.
//   stream_probe order           the look-back kernel's tile shape (8 waves x 4 accesses) with its order of work:
//                             the 67 108 864 elements of a stream are cut into R rows, and workgroup k takes tile
//                             k / R of row k % R, so that tiles of all rows are in flight together. R = 1 is the
//                             plain linear order. What the memory system gives that order with no scan, no tickets
//                             and no carry chain.
//   stream_probe cl              the channels-last kernels' access shape with no scan: tensors [B, T, C] fp32, a
//                             workgroup owns 64 * VEC channels of one batch element and walks all of T in tiles of
//                             W waves x S time steps; per step a wave reads one span of 64 * VEC channels. With and
//                             without the kernels' one barrier per tile; and the same spans with one tile per
//                             workgroup (the shape of the kernel that also splits time over workgroups).
//   stream_probe misaligned      a copy with 16-byte accesses that start 2, 4, 6 or 8 bytes after a 16-byte border, in
//                             every lane or in one lane per wave: what element-aligned vectors cost.
//
//   hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops stream_probe.hip -o stream_probe
//   (or `make -C scanscam_amd/csrc`, which builds build/stream_probe)
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef unsigned u4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));

#define CHECK(call)                                                                   \
    do {                                                                              \
        hipError_t e_ = (call);                                                       \
        if (e_ != hipSuccess) {                                                       \
            fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));                \
            exit(1);                                                                  \
        }                                                                             \
    } while (0)

__global__ __launch_bounds__(256) void copy_calib_kernel(const u4 *__restrict__ in, u4 *__restrict__ out, size_t n)
{
    size_t i = (size_t)blockIdx.x * 1024 + threadIdx.x;
#pragma unroll
    for (int k = 0; k < 4; k++, i += 256)
        if (i < n) __builtin_nontemporal_store(__builtin_nontemporal_load(in + i), out + i);
}

// READS input streams, WRITES output streams; workgroup b covers vectors [b*1024, (b+1)*1024), wave w its
// quarter, four consecutive 1 KiB spans per wave -- the layout of scan_row_kernel<float, 4, 4>.
template <int READS, int WRITES>
__global__ __launch_bounds__(256) void stream_shape_kernel(const f4 *__restrict__ a, const f4 *__restrict__ b,
                                                           const f4 *__restrict__ c, f4 *__restrict__ o0,
                                                           f4 *__restrict__ o1)
{
    const size_t base = (size_t)blockIdx.x * 1024 + (threadIdx.x / 64) * 256 + (threadIdx.x % 64);
    f4 va[4], vb[4], vc[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        va[u] = __builtin_nontemporal_load(a + base + u * 64);
        if (READS > 1) vb[u] = __builtin_nontemporal_load(b + base + u * 64);
        if (READS > 2) vc[u] = __builtin_nontemporal_load(c + base + u * 64);
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
        f4 r = va[u];
        if (READS > 1) r += vb[u];
        if (READS > 2) r *= vc[u];
        __builtin_nontemporal_store(r, o0 + base + u * 64);
        if (WRITES > 1) __builtin_nontemporal_store(r + 1.0f, o1 + base + u * 64);
    }
}

// The same for any mix of streams and any workgroup shape: W waves, U consecutive 1 KiB spans per wave and
// stream, all loads issued before the first store. With no output stream the sum of what was read is
// compared with a value it never takes, so the loads stay.
template <int READS, int WRITES, int U, int W>
__global__ __launch_bounds__(W * 64) void stream_mix_kernel(const f4 *__restrict__ a, const f4 *__restrict__ b,
                                                            const f4 *__restrict__ c, f4 *__restrict__ o0,
                                                            f4 *__restrict__ o1, float never)
{
    const size_t base = (size_t)blockIdx.x * (W * U * 64) + (threadIdx.x / 64) * (U * 64) + (threadIdx.x % 64);
    f4 va[U], vb[U], vc[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (READS > 0) va[u] = __builtin_nontemporal_load(a + base + u * 64);
        if (READS > 1) vb[u] = __builtin_nontemporal_load(b + base + u * 64);
        if (READS > 2) vc[u] = __builtin_nontemporal_load(c + base + u * 64);
    }
    if (WRITES == 0) {
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
        f4 r = never;
        if (READS > 0) r = va[u];
        if (READS > 1) r += vb[u];
        if (READS > 2) r *= vc[u];
        __builtin_nontemporal_store(r, o0 + base + u * 64);
        if (WRITES > 1) __builtin_nontemporal_store(r + 1.0f, o1 + base + u * 64);
    }
}

// stream_mix_kernel with the look-back kernel's order of work: workgroup k works on tile k / R of row k % R.
template <int READS, int WRITES, int U, int W>
__global__ __launch_bounds__(W * 64) void stream_order_kernel(const f4 *__restrict__ a, const f4 *__restrict__ b,
                                                              const f4 *__restrict__ c, f4 *__restrict__ o0,
                                                              f4 *__restrict__ o1, unsigned R, size_t row_vecs)
{
    const size_t base = (size_t)(blockIdx.x % R) * row_vecs + (size_t)(blockIdx.x / R) * (W * U * 64) +
                        (threadIdx.x / 64) * (U * 64) + (threadIdx.x % 64);
    f4 va[U], vb[U], vc[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        va[u] = __builtin_nontemporal_load(a + base + u * 64);
        vb[u] = __builtin_nontemporal_load(b + base + u * 64);
        if (READS > 2) vc[u] = __builtin_nontemporal_load(c + base + u * 64);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        f4 r = va[u] + vb[u];
        if (READS > 2) r *= vc[u];
        __builtin_nontemporal_store(r, o0 + base + u * 64);
        if (WRITES > 1) __builtin_nontemporal_store(r + 1.0f, o1 + base + u * 64);
    }
}

// Cache-policy variants: the builtins only reach "nt", so the instruction is written out. POLICY 0..6 =
// nt | sc1 nt | sc0 sc1 nt | sc0 nt | sc1 | sc0 sc1 | none.
#define PROBE_POLICY(OP, ...)                                                          \
    switch (POLICY) {                                                                  \
    case 0: asm volatile(OP " nt" __VA_ARGS__); break;                                 \
    case 1: asm volatile(OP " sc1 nt" __VA_ARGS__); break;                             \
    case 2: asm volatile(OP " sc0 sc1 nt" __VA_ARGS__); break;                         \
    case 3: asm volatile(OP " sc0 nt" __VA_ARGS__); break;                             \
    case 4: asm volatile(OP " sc1" __VA_ARGS__); break;                                \
    case 5: asm volatile(OP " sc0 sc1" __VA_ARGS__); break;                            \
    default: asm volatile(OP __VA_ARGS__); break;                                      \
    }
static const char *const kPolicyName[7] = {"nt", "sc1 nt", "sc0 sc1 nt", "sc0 nt", "sc1", "sc0 sc1", "(none)"};

template <int POLICY> __device__ __forceinline__ f4 policy_load(const f4 *p)
{
    f4 r;
    PROBE_POLICY("global_load_dwordx4 %0, %1, off", : "=v"(r) : "v"(p) : "memory")
    return r;
}
template <int POLICY> __device__ __forceinline__ void policy_store(f4 *p, f4 v)
{
    PROBE_POLICY("global_store_dwordx4 %0, %1, off", : : "v"(p), "v"(v) : "memory")
}

template <int READS, int WRITES, int LOAD_POLICY, int STORE_POLICY>
__global__ __launch_bounds__(256) void stream_policy_kernel(const f4 *__restrict__ a, const f4 *__restrict__ b,
                                                            const f4 *__restrict__ c, f4 *__restrict__ o0,
                                                            f4 *__restrict__ o1)
{
    const size_t base = (size_t)blockIdx.x * 1024 + (threadIdx.x / 64) * 256 + (threadIdx.x % 64);
    f4 va[4], vb[4], vc[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        va[u] = policy_load<LOAD_POLICY>(a + base + u * 64);
        if (READS > 1) vb[u] = policy_load<LOAD_POLICY>(b + base + u * 64);
        if (READS > 2) vc[u] = policy_load<LOAD_POLICY>(c + base + u * 64);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the compiler does not track loads issued from asm
#pragma unroll
    for (int u = 0; u < 4; u++) {
        f4 r = va[u];
        if (READS > 1) r += vb[u];
        if (READS > 2) r *= vc[u];
        policy_store<STORE_POLICY>(o0 + base + u * 64, r);
        if (WRITES > 1) policy_store<STORE_POLICY>(o1 + base + u * 64, r + 1.0f);
    }
}

template <typename F> static float mean_ms(F launch, int reps)
{
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int i = 0; i < 3; i++) launch();
    CHECK(hipEventRecord(e0, 0));
    for (int i = 0; i < reps; i++) launch();
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    return ms / reps;
}

static int run_copy(size_t mib)
{
    const size_t bytes = mib << 20, n = bytes / 16;
    u4 *in, *out;
    CHECK(hipMalloc(&in, bytes));
    CHECK(hipMalloc(&out, bytes));
    CHECK(hipMemset(in, 1, bytes));
    CHECK(hipMemset(out, 0, bytes));
    const float ms = mean_ms(
        [&] { hipLaunchKernelGGL(copy_calib_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, 0, in, out, n); }, 20);
    printf("copy_calib: %zu MiB read + %zu MiB written per launch, %.1f us per launch, %.1f GB/s\n", mib, mib,
           ms * 1e3, 2.0 * bytes / (ms * 1e-3) / 1e9);
    return hipDeviceSynchronize() == hipSuccess ? 0 : 1;
}

static int run_ceiling(size_t rows)
{
    const size_t T = 4096, n = rows * T, bytes = n * 4;
    f4 *buf[5];
    for (auto &p : buf) {
        CHECK(hipMalloc(&p, bytes));
        CHECK(hipMemset(p, 0, bytes));
    }
    const dim3 grid((unsigned)rows), block(256);
    const float fwd = mean_ms([&] { hipLaunchKernelGGL((stream_shape_kernel<2, 1>), grid, block, 0, 0, buf[0], buf[1], buf[2], buf[3], buf[4]); }, 30);
    const float bwd = mean_ms([&] { hipLaunchKernelGGL((stream_shape_kernel<3, 2>), grid, block, 0, 0, buf[0], buf[1], buf[2], buf[3], buf[4]); }, 30);
    printf("stream ceiling, %zu x 4096 fp32, one workgroup per row:\n", rows);
    printf("  2 reads + 1 write (forward shape):  %7.1f us  %7.1f GB/s  %4.1f %% of 8 TB/s\n", fwd * 1e3,
           3.0 * bytes / (fwd * 1e-3) / 1e9, 3.0 * bytes / (fwd * 1e-3) / 8e12 * 100);
    printf("  3 reads + 2 writes (backward shape): %7.1f us  %7.1f GB/s  %4.1f %% of 8 TB/s\n", bwd * 1e3,
           5.0 * bytes / (bwd * 1e-3) / 1e9, 5.0 * bytes / (bwd * 1e-3) / 8e12 * 100);
    return hipDeviceSynchronize() == hipSuccess ? 0 : 1;
}

static f4 *g_sets[8][5];

template <int READS, int WRITES, int LP, int SP> static void policy_case(size_t rows)
{
    int i = 0;
    const float ms = mean_ms(
        [&] {
            f4 **s = g_sets[i++ % 8];
            hipLaunchKernelGGL((stream_policy_kernel<READS, WRITES, LP, SP>), dim3((unsigned)rows), dim3(256), 0, 0,
                               s[0], s[1], s[2], s[3], s[4]);
        },
        32);
    const double bytes = (double)(READS + WRITES) * rows * 4096 * 4;
    printf("  %dR%dW  loads %-11s stores %-11s %7.1f us  %4.1f %% of 8 TB/s\n", READS, WRITES, kPolicyName[LP],
           kPolicyName[SP], ms * 1e3, bytes / (ms * 1e-3) / 8e12 * 100);
}
template <int LP, int SP> static void policy_pair(size_t rows)
{
    policy_case<2, 1, LP, SP>(rows);
    policy_case<3, 2, LP, SP>(rows);
}

static int run_policy(size_t rows)
{
    const size_t bytes = rows * 4096 * 4;
    for (auto &set : g_sets)
        for (auto &p : set) {
            CHECK(hipMalloc(&p, bytes));
            CHECK(hipMemset(p, 0, bytes));
        }
    printf("cache policy, %zu x 4096 fp32, one workgroup per row, 8 rotated buffer sets:\n", rows);
    policy_pair<0, 0>(rows);
    policy_pair<1, 0>(rows);
    policy_pair<2, 0>(rows);
    policy_pair<3, 0>(rows);
    policy_pair<4, 0>(rows);
    policy_pair<5, 0>(rows);
    policy_pair<6, 0>(rows);
    policy_pair<0, 1>(rows);
    policy_pair<0, 2>(rows);
    policy_pair<0, 3>(rows);
    policy_pair<0, 4>(rows);
    policy_pair<0, 5>(rows);
    policy_pair<0, 6>(rows);
    return hipDeviceSynchronize() == hipSuccess ? 0 : 1;
}

static f4 *g_mix[4][5];

template <int READS, int WRITES, int U, int W> static void mix_case()
{
    const size_t n = (size_t)16384 * 4096;  // elements per stream
    int i = 0;
    const float ms = mean_ms(
        [&] {
            f4 **s = g_mix[i++ % 4];
            hipLaunchKernelGGL((stream_mix_kernel<READS, WRITES, U, W>), dim3((unsigned)(n / 4 / (W * U * 64))),
                               dim3(W * 64), 0, 0, s[0], s[1], s[2], s[3], s[4], 12345.678f);
        },
        40);
    const double bytes = (double)(READS + WRITES) * n * 4;
    printf("  %dR%dW  %2d waves x %d accesses  %7.1f us  %7.1f GB/s  %4.1f %% of 8 TB/s\n", READS, WRITES, W, U, ms * 1e3,
           bytes / (ms * 1e-3) / 1e9, bytes / (ms * 1e-3) / 8e12 * 100);
}

static int run_mix()
{
    const size_t bytes = (size_t)16384 * 4096 * 4;
    for (auto &set : g_mix)
        for (auto &p : set) {
            CHECK(hipMalloc(&p, bytes));
            CHECK(hipMemset(p, 0, bytes));
        }
    printf("stream mixes, 67 108 864 fp32 per stream, non-temporal 16-byte accesses, 4 rotated buffer sets:\n");
    mix_case<1, 0, 4, 4>();
    mix_case<1, 0, 1, 16>();
    mix_case<2, 0, 4, 4>();
    mix_case<3, 0, 4, 4>();
    mix_case<0, 1, 4, 4>();
    mix_case<0, 2, 4, 4>();
    mix_case<1, 1, 4, 4>();
    printf("forward mix (2 reads + 1 write) by workgroup shape:\n");
    mix_case<2, 1, 1, 4>();
    mix_case<2, 1, 2, 4>();
    mix_case<2, 1, 4, 4>();
    mix_case<2, 1, 8, 4>();
    mix_case<2, 1, 2, 8>();
    mix_case<2, 1, 4, 8>();
    mix_case<2, 1, 1, 16>();
    mix_case<2, 1, 4, 16>();
    printf("backward mix (3 reads + 2 writes) by workgroup shape:\n");
    mix_case<3, 2, 1, 4>();
    mix_case<3, 2, 2, 4>();
    mix_case<3, 2, 4, 4>();
    mix_case<3, 2, 2, 8>();
    mix_case<3, 2, 4, 8>();
    mix_case<3, 2, 1, 16>();
    mix_case<3, 2, 4, 16>();
    return hipDeviceSynchronize() == hipSuccess ? 0 : 1;
}

template <int READS, int WRITES> static void order_case(unsigned R)
{
    constexpr int U = 4, W = 8;
    const size_t n = (size_t)16384 * 4096, vecs = n / 4, tile_vecs = W * U * 64;  // R divides vecs / tile_vecs
    int i = 0;
    const float ms = mean_ms(
        [&] {
            f4 **s = g_mix[i++ % 4];
            hipLaunchKernelGGL((stream_order_kernel<READS, WRITES, U, W>), dim3((unsigned)(vecs / tile_vecs)), dim3(W * 64),
                               0, 0, s[0], s[1], s[2], s[3], s[4], R, vecs / R);
        },
        40);
    const double bytes = (double)(READS + WRITES) * n * 4;
    printf("  %dR%dW  %5u rows of %8zu  %7.1f us  %7.1f GB/s  %4.1f %% of 8 TB/s\n", READS, WRITES, R, n / R, ms * 1e3,
           bytes / (ms * 1e-3) / 1e9, bytes / (ms * 1e-3) / 8e12 * 100);
}

static int run_order()
{
    const size_t bytes = (size_t)16384 * 4096 * 4;
    for (auto &set : g_mix)
        for (auto &p : set) {
            CHECK(hipMalloc(&p, bytes));
            CHECK(hipMemset(p, 0, bytes));
        }
    printf("order of work, 67 108 864 fp32 per stream, 8 waves x 4 accesses (8192-element tiles), workgroup k -> tile k / R of row k %% R:\n");
    for (unsigned R : {1u, 8u, 64u, 256u, 1024u}) order_case<2, 1>(R);
    for (unsigned R : {1u, 8u, 64u, 256u, 1024u}) order_case<3, 2>(R);
    return hipDeviceSynchronize() == hipSuccess ? 0 : 1;
}

// Channels-last access shape (scan_cl_kernel): see `stream_probe cl` above. T is a multiple of W * S.
template <int VEC> struct ClVec { typedef f4 type; };
template <> struct ClVec<1> { typedef float type; };

template <int READS, int WRITES, int VEC, int S, bool SYNC>
__global__ void cl_stream_kernel(const float *__restrict__ a, const float *__restrict__ b, const float *__restrict__ c,
                                 float *__restrict__ o0, float *__restrict__ o1, int T, int C)
{
    typedef typename ClVec<VEC>::type V;
    const int W = blockDim.x / 64, wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int groups = C / (64 * VEC);
    const size_t col = (size_t)(blockIdx.x / groups) * T * C + (size_t)(blockIdx.x % groups) * 64 * VEC + lane * VEC;
    for (int t0 = wave * S; t0 < T; t0 += W * S) {
        V va[S], vb[S], vc[S];
#pragma unroll
        for (int k = 0; k < S; k++) {
            const size_t at = col + (size_t)(t0 + k) * C;
            va[k] = __builtin_nontemporal_load(reinterpret_cast<const V *>(a + at));
            vb[k] = __builtin_nontemporal_load(reinterpret_cast<const V *>(b + at));
            if (READS > 2) vc[k] = __builtin_nontemporal_load(reinterpret_cast<const V *>(c + at));
        }
        if (SYNC) __syncthreads();
#pragma unroll
        for (int k = 0; k < S; k++) {
            const size_t at = col + (size_t)(t0 + k) * C;
            V r = va[k] + vb[k];
            if (READS > 2) r *= vc[k];
            __builtin_nontemporal_store(r, reinterpret_cast<V *>(o0 + at));
            if (WRITES > 1) __builtin_nontemporal_store(r + 1.0f, reinterpret_cast<V *>(o1 + at));
        }
    }
}

static float *g_cl[2][5];
static const size_t kClElements = (size_t)1 << 28;  // per stream: the largest case below

template <int READS, int WRITES, int VEC, int S, bool SYNC> static void cl_case(int B, int T, int C, int W)
{
    const size_t n = (size_t)B * T * C;
    if (n > kClElements || T % (W * S) != 0 || C % (64 * VEC) != 0 || W < 1 || W > 16) {
        fprintf(stderr, "cl_case: [%d, %d, %d] with %d waves x %d steps does not fit the buffers or the kernel\n", B, T, C, W, S);
        exit(1);
    }
    int i = 0;
    const float ms = mean_ms(
        [&] {
            float **s = g_cl[i++ % 2];
            hipLaunchKernelGGL((cl_stream_kernel<READS, WRITES, VEC, S, SYNC>), dim3((unsigned)(B * (C / (64 * VEC)))),
                               dim3(W * 64), 0, 0, s[0], s[1], s[2], s[3], s[4], T, C);
        },
        30);
    const double bytes = (double)(READS + WRITES) * n * 4;
    printf("  %dR%dW  [%4d, %5d, %5d]  %2d-byte lanes  %2d waves x %2d steps  %-10s %5d workgroups  %7.1f us  %4.1f %% of 8 TB/s\n",
           READS, WRITES, B, T, C, VEC * 4, W, S, SYNC ? "barrier" : "no barrier", B * (C / (64 * VEC)), ms * 1e3,
           bytes / (ms * 1e-3) / 8e12 * 100);
}

// The same spans taken one tile of W x S steps per workgroup (scan_cl_lookback_kernel's shape, with no tickets and
// no carry chain): workgroup k takes tile k / RG of row-group k % RG (ROW_MAJOR = false: tiles of all row-groups in
// flight together) or tile k % tiles of row-group k / tiles (ROW_MAJOR = true).
template <int READS, int WRITES, int VEC, int S, bool ROW_MAJOR>
__global__ void cl_tile_kernel(const float *__restrict__ a, const float *__restrict__ b, const float *__restrict__ c,
                               float *__restrict__ o0, float *__restrict__ o1, int T, int C, int rowgroups, int tiles)
{
    typedef typename ClVec<VEC>::type V;
    const int W = blockDim.x / 64, wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int groups = C / (64 * VEC);
    const int rg = ROW_MAJOR ? blockIdx.x / tiles : blockIdx.x % rowgroups;
    const int tile = ROW_MAJOR ? blockIdx.x % tiles : blockIdx.x / rowgroups;
    const size_t col = (size_t)(rg / groups) * T * C + (size_t)(rg % groups) * 64 * VEC + lane * VEC;
    const int t0 = (tile * W + wave) * S;
    V va[S], vb[S], vc[S];
#pragma unroll
    for (int k = 0; k < S; k++) {
        const size_t at = col + (size_t)(t0 + k) * C;
        va[k] = __builtin_nontemporal_load(reinterpret_cast<const V *>(a + at));
        vb[k] = __builtin_nontemporal_load(reinterpret_cast<const V *>(b + at));
        if (READS > 2) vc[k] = __builtin_nontemporal_load(reinterpret_cast<const V *>(c + at));
    }
#pragma unroll
    for (int k = 0; k < S; k++) {
        const size_t at = col + (size_t)(t0 + k) * C;
        V r = va[k] + vb[k];
        if (READS > 2) r *= vc[k];
        __builtin_nontemporal_store(r, reinterpret_cast<V *>(o0 + at));
        if (WRITES > 1) __builtin_nontemporal_store(r + 1.0f, reinterpret_cast<V *>(o1 + at));
    }
}

template <int READS, int WRITES, int VEC, int S, bool ROW_MAJOR> static void cl_tile_case(int B, int T, int C, int W)
{
    const size_t n = (size_t)B * T * C;
    if (n > kClElements || T % (W * S) != 0 || C % (64 * VEC) != 0 || W < 1 || W > 16) {
        fprintf(stderr, "cl_tile_case: [%d, %d, %d] with %d waves x %d steps does not fit the buffers or the kernel\n", B, T, C, W, S);
        exit(1);
    }
    const int rowgroups = B * (C / (64 * VEC)), tiles = T / (W * S);
    int i = 0;
    const float ms = mean_ms(
        [&] {
            float **s = g_cl[i++ % 2];
            hipLaunchKernelGGL((cl_tile_kernel<READS, WRITES, VEC, S, ROW_MAJOR>), dim3((unsigned)(rowgroups * tiles)),
                               dim3(W * 64), 0, 0, s[0], s[1], s[2], s[3], s[4], T, C, rowgroups, tiles);
        },
        30);
    const double bytes = (double)(READS + WRITES) * n * 4;
    printf("  %dR%dW  [%4d, %5d, %5d]  %2d-byte lanes  one tile of %2d waves x %2d steps per workgroup, %-10s %6d workgroups  %7.1f us  %4.1f %% of 8 TB/s\n",
           READS, WRITES, B, T, C, VEC * 4, W, S, ROW_MAJOR ? "row-major" : "tile-major", rowgroups * tiles, ms * 1e3,
           bytes / (ms * 1e-3) / 8e12 * 100);
}

template <int READS, int WRITES> static void cl_tile_cases()
{
    cl_tile_case<READS, WRITES, 4, 4, false>(64, 2048, 1024, 4);
    cl_tile_case<READS, WRITES, 4, 4, true>(64, 2048, 1024, 4);
    cl_tile_case<READS, WRITES, 4, 4, false>(64, 2048, 1024, 8);
    cl_tile_case<READS, WRITES, 4, 8, false>(64, 2048, 1024, 8);
    cl_tile_case<READS, WRITES, 4, 8, false>(8, 4096, 2048, 8);
    cl_tile_case<READS, WRITES, 4, 8, true>(8, 4096, 2048, 8);
    cl_tile_case<READS, WRITES, 4, 8, false>(8, 4096, 2048, 4);
    cl_tile_case<READS, WRITES, 4, 4, false>(8, 4096, 2048, 4);
    cl_tile_case<READS, WRITES, 1, 16, false>(8, 4096, 2048, 8);
    cl_tile_case<READS, WRITES, 1, 8, false>(8, 4096, 2048, 4);
    cl_tile_case<READS, WRITES, 1, 16, false>(8, 4096, 512, 8);
    cl_tile_case<READS, WRITES, 4, 8, false>(8, 4096, 512, 8);
}

template <int READS, int WRITES> static void cl_cases()
{
    cl_case<READS, WRITES, 4, 4, true>(64, 2048, 1024, 16);
    cl_case<READS, WRITES, 4, 4, false>(64, 2048, 1024, 16);
    cl_case<READS, WRITES, 4, 8, true>(64, 2048, 1024, 8);
    cl_case<READS, WRITES, 4, 4, true>(64, 2048, 1024, 4);
    cl_case<READS, WRITES, 4, 4, true>(256, 1024, 1024, 16);
    cl_case<READS, WRITES, 4, 4, false>(256, 1024, 1024, 16);
    cl_case<READS, WRITES, 4, 4, true>(256, 1024, 1024, 4);
    cl_case<READS, WRITES, 4, 4, true>(512, 1024, 256, 16);
    cl_case<READS, WRITES, 4, 4, false>(512, 1024, 256, 16);
    cl_case<READS, WRITES, 1, 8, true>(8, 4096, 2048, 16);
    cl_case<READS, WRITES, 1, 8, false>(8, 4096, 2048, 16);
    cl_case<READS, WRITES, 1, 16, true>(8, 4096, 2048, 8);
    cl_case<READS, WRITES, 1, 16, true>(8, 4096, 2048, 16);
    cl_case<READS, WRITES, 1, 8, true>(64, 2048, 512, 16);
    cl_case<READS, WRITES, 1, 8, true>(32, 2048, 1024, 16);
}

static int run_cl()
{
    const size_t bytes = kClElements * sizeof(float);
    for (auto &set : g_cl)
        for (auto &p : set) {
            CHECK(hipMalloc(&p, bytes));
            CHECK(hipMemset(p, 0, bytes));
        }
    printf("channels-last access shape, fp32, 2 rotated buffer sets of 1 GiB per stream:\n");
    cl_cases<2, 1>();
    cl_cases<3, 2>();
    printf("one tile per workgroup:\n");
    cl_tile_cases<2, 1>();
    cl_tile_cases<3, 2>();
    return hipDeviceSynchronize() == hipSuccess ? 0 : 1;
}

// 16-byte accesses that start OFFSET bytes after a 16-byte border (element-aligned vectors of rows that start
// anywhere), in every lane (EVERY = true) or in lane 0 of each wave only. Copy of 2^26 floats.
typedef f4 f4_unaligned __attribute__((aligned(2)));

template <bool LOADS, bool STORES, bool EVERY>
__global__ __launch_bounds__(256) void misaligned_kernel(const char *__restrict__ in, char *__restrict__ out, int offset)
{
    const size_t i = ((size_t)blockIdx.x * 1024 + (threadIdx.x / 64) * 256 + (threadIdx.x % 64)) * 16;
    const bool mine = EVERY || (threadIdx.x % 64) == 0;
    f4 v[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
        v[u] = __builtin_nontemporal_load(reinterpret_cast<const f4_unaligned *>(in + i + u * 1024 + ((LOADS && mine) ? offset : 0)));
#pragma unroll
    for (int u = 0; u < 4; u++)
        __builtin_nontemporal_store(v[u], reinterpret_cast<f4_unaligned *>(out + i + u * 1024 + ((STORES && mine) ? offset : 0)));
}

template <bool LOADS, bool STORES, bool EVERY> static void misaligned_case(char *in, char *out, size_t bytes, int offset)
{
    const float ms = mean_ms(
        [&] {
            hipLaunchKernelGGL((misaligned_kernel<LOADS, STORES, EVERY>), dim3((unsigned)(bytes / 16384)), dim3(256), 0, 0, in, out, offset);
        },
        20);
    printf("  offset %2d bytes in %-22s of %-6s  %7.1f us  %4.1f %% of 8 TB/s\n", offset, EVERY ? "every lane" : "lane 0 of each wave",
           LOADS && STORES ? "both" : (LOADS ? "loads" : "stores"), ms * 1e3, 2.0 * bytes / (ms * 1e-3) / 8e12 * 100);
}

static int run_misaligned()
{
    const size_t bytes = (size_t)1 << 28;  // the kernels touch up to 16 bytes beyond: allocate one block more
    char *in, *out;
    CHECK(hipMalloc(&in, bytes + 16384));
    CHECK(hipMalloc(&out, bytes + 16384));
    CHECK(hipMemset(in, 0, bytes + 16384));
    CHECK(hipMemset(out, 0, bytes + 16384));
    printf("copy of 256 MiB with 16-byte accesses that start off a 16-byte border:\n");
    for (int offset : {0, 2, 4, 8, 6}) {
        misaligned_case<true, false, true>(in, out, bytes, offset);
        misaligned_case<false, true, true>(in, out, bytes, offset);
        misaligned_case<true, false, false>(in, out, bytes, offset);
        misaligned_case<false, true, false>(in, out, bytes, offset);
    }
    return hipDeviceSynchronize() == hipSuccess ? 0 : 1;
}

int main(int argc, char **argv)
{
    if (argc > 1 && strcmp(argv[1], "misaligned") == 0) return run_misaligned();
    if (argc > 1 && strcmp(argv[1], "cl") == 0) return run_cl();
    if (argc > 1 && strcmp(argv[1], "order") == 0) return run_order();
    if (argc > 1 && strcmp(argv[1], "mix") == 0) return run_mix();
    if (argc > 1 && strcmp(argv[1], "ceiling") == 0) return run_ceiling(argc > 2 ? (size_t)atol(argv[2]) : 16384);
    if (argc > 1 && strcmp(argv[1], "copy") == 0) return run_copy(argc > 2 ? (size_t)atol(argv[2]) : 1024);
    if (argc > 1 && strcmp(argv[1], "policy") == 0) return run_policy(argc > 2 ? (size_t)atol(argv[2]) : 16384);
    fprintf(stderr, "usage: %s copy [MiB] | ceiling [rows] | policy [rows] | mix | order | cl | misaligned\n", argv[0]);
    return 2;
}

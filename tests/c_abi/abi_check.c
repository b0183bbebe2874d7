/*
 * A consumer of libscanscam_hip.so written in plain C99: no C++, no torch, no Python. It shows that
 * the boundary is what include/scanscam_hip.h says (device pointers, sizes, a caller-owned workspace,
 * a stream, integer error codes) and checks each entry point against a sequential loop on the host.
 *
 *   make -C tests/c_abi        (needs scanscam_amd/libscanscam_hip.so)
 *   tests/c_abi/abi_check      exits 0 and prints "abi_check: ok" when every case agrees
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "scanscam_hip.h"

#define HIP_OK(call)                                                                       \
    do {                                                                                   \
        hipError_t e_ = (call);                                                            \
        if (e_ != hipSuccess) {                                                            \
            fprintf(stderr, "abi_check: %s failed: %s\n", #call, hipGetErrorString(e_));   \
            exit(2);                                                                       \
        }                                                                                  \
    } while (0)

static unsigned long long rng_state = 88172645463325252ull;
static float uniform01(void)
{
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return (float)((rng_state >> 40) & 0xffffff) / 16777216.0f;
}

static float *device_copy(const float *host, size_t n)
{
    float *d;
    HIP_OK(hipMalloc((void **)&d, n * sizeof(float)));
    HIP_OK(hipMemcpy(d, host, n * sizeof(float), hipMemcpyHostToDevice));
    return d;
}

static double worst(const float *got, const float *want, size_t n)
{
    double w = 0.0;
    for (size_t i = 0; i < n; i++) {
        double den = fabs((double)want[i]) > 1.0 ? fabs((double)want[i]) : 1.0;
        double e = fabs((double)got[i] - (double)want[i]) / den;
        if (!(e <= w)) w = e; /* also catches NaN */
    }
    return w;
}

/* rows x T tensors; channels_last = 0: [rows, T]; 1: [batch = rows / C, T, C] with C given. */
static int check_case(const char *name, long rows, long T, long C, int channels_last, hipStream_t stream)
{
    const size_t n = (size_t)rows * (size_t)T;
    float *a = malloc(n * 4), *b = malloc(n * 4), *gh = malloc(n * 4), *h = malloc(n * 4), *ga = malloc(n * 4),
          *gb = malloc(n * 4), *got = malloc(n * 4);
    const long batch = channels_last ? rows / C : 0;
    /* Element (row r, time t) lives at idx(r, t). */
#define IDX(r, t) (channels_last ? ((size_t)((r) / C) * T + (t)) * C + (r) % C : (size_t)(r) * T + (t))
    for (size_t i = 0; i < n; i++) {
        a[i] = uniform01();
        b[i] = 2.0f * uniform01() - 1.0f;
        gh[i] = 2.0f * uniform01() - 1.0f;
    }
    for (long r = 0; r < rows; r++) {
        float acc = 0.0f;
        for (long t = 0; t < T; t++) {
            acc = acc * a[IDX(r, t)] + b[IDX(r, t)];
            h[IDX(r, t)] = acc;
        }
        float d = 0.0f;
        for (long t = T - 1; t >= 0; t--) {
            d += gh[IDX(r, t)];
            gb[IDX(r, t)] = d;
            ga[IDX(r, t)] = d * (t > 0 ? h[IDX(r, t - 1)] : 0.0f);
            d *= a[IDX(r, t)];
        }
    }
#undef IDX
    float *da = device_copy(a, n), *db = device_copy(b, n), *dgh = device_copy(gh, n), *dh = device_copy(h, n);
    float *o0, *o1;
    HIP_OK(hipMalloc((void **)&o0, n * 4));
    HIP_OK(hipMalloc((void **)&o1, n * 4));

    size_t ws_bytes = 0;
    for (int dir = 0; dir < 2; dir++) {
        size_t need = channels_last ? scanscam_workspace_bytes_cl(batch, T, C, SCANSCAM_F32, dir, NULL)
                                    : scanscam_workspace_bytes(rows, T, SCANSCAM_F32, dir);
        if (need > ws_bytes) ws_bytes = need;
    }
    void *ws = NULL;
    if (ws_bytes) HIP_OK(hipMalloc(&ws, ws_bytes));

    int failures = 0;
    int rc = channels_last
                 ? scanscam_scan_fwd_cl(da, db, o0, batch, T, C, SCANSCAM_F32, ws, ws_bytes, stream, NULL)
                 : scanscam_scan_fwd(da, db, o0, rows, T, SCANSCAM_F32, ws, ws_bytes, stream);
    if (rc != SCANSCAM_OK) {
        fprintf(stderr, "abi_check: %s forward: %s\n", name, scanscam_strerror(rc));
        failures++;
    }
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(got, o0, n * 4, hipMemcpyDeviceToHost));
    const double eh = worst(got, h, n);

    rc = channels_last
             ? scanscam_scan_bwd_cl(da, dh, dgh, o1, o0, batch, T, C, SCANSCAM_F32, ws, ws_bytes, stream, NULL)
             : scanscam_scan_bwd(da, dh, dgh, o1, o0, rows, T, SCANSCAM_F32, ws, ws_bytes, stream);
    if (rc != SCANSCAM_OK) {
        fprintf(stderr, "abi_check: %s backward: %s\n", name, scanscam_strerror(rc));
        failures++;
    }
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(got, o0, n * 4, hipMemcpyDeviceToHost));
    const double egb = worst(got, gb, n);
    HIP_OK(hipMemcpy(got, o1, n * 4, hipMemcpyDeviceToHost));
    const double ega = worst(got, ga, n);

    printf("abi_check: %-28s workspace %8zu B  worst relative error h %.2e  grad_b %.2e  grad_a %.2e\n", name,
           ws_bytes, eh, egb, ega);
    /* gates and values in [0,1) x [-1,1): |h|, |grad_b| stay small, so 1e-5 (2e-5 for the product) is ample */
    if (!(eh <= 1e-5) || !(egb <= 1e-5) || !(ega <= 2e-5)) failures++;

    if (channels_last) {
        /* The plan the channels-last call resolves to, handed back in: bit-identical output, no larger workspace. */
        scanscam_plan plan;
        float *again = (float *)malloc(n * 4);
        if (scanscam_resolve_plan_cl(batch, T, C, SCANSCAM_F32, SCANSCAM_FORWARD, NULL, &plan) != SCANSCAM_OK) failures++;
        if (scanscam_workspace_bytes_cl(batch, T, C, SCANSCAM_F32, SCANSCAM_FORWARD, &plan) > ws_bytes) failures++;
        HIP_OK(hipMemset(o0, 0, n * 4));
        if (scanscam_scan_fwd_cl(da, db, o0, batch, T, C, SCANSCAM_F32, ws, ws_bytes, stream, NULL) != SCANSCAM_OK) failures++;
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(again, o0, n * 4, hipMemcpyDeviceToHost));
        HIP_OK(hipMemset(o0, 0, n * 4));
        if (scanscam_scan_fwd_cl(da, db, o0, batch, T, C, SCANSCAM_F32, ws, ws_bytes, stream, &plan) != SCANSCAM_OK) failures++;
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(got, o0, n * 4, hipMemcpyDeviceToHost));
        if (memcmp(got, again, n * 4) != 0 || worst(got, h, n) > 1e-5) failures++;
        free(again);
    }
    if (!channels_last) {
        /* The same launch through the _plan and _timed variants: a resolved plan handed back in gives
         * bit-identical output, and the caller's events hold the kernel's own duration. */
        scanscam_plan plan;
        hipEvent_t ev0, ev1;
        float ms = -1.0f;
        HIP_OK(hipEventCreate(&ev0));
        HIP_OK(hipEventCreate(&ev1));
        float *again = (float *)malloc(n * 4);
        if (scanscam_resolve_plan(rows, T, SCANSCAM_F32, SCANSCAM_FORWARD, NULL, &plan) != SCANSCAM_OK) failures++;
        if (scanscam_workspace_bytes_plan(rows, T, SCANSCAM_F32, SCANSCAM_FORWARD, &plan) > ws_bytes) failures++;
        HIP_OK(hipMemset(o0, 0, n * 4));
        if (scanscam_scan_fwd_plan(da, db, o0, rows, T, SCANSCAM_F32, ws, ws_bytes, stream, &plan) != SCANSCAM_OK) failures++;
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(again, o0, n * 4, hipMemcpyDeviceToHost));
        HIP_OK(hipMemset(o0, 0, n * 4));
        if (scanscam_scan_fwd_timed(da, db, o0, rows, T, SCANSCAM_F32, ws, ws_bytes, stream, &plan, ev0, ev1) != SCANSCAM_OK)
            failures++;
        HIP_OK(hipEventSynchronize(ev1));
        HIP_OK(hipEventElapsedTime(&ms, ev0, ev1));
        HIP_OK(hipMemcpy(got, o0, n * 4, hipMemcpyDeviceToHost));
        if (memcmp(got, again, n * 4) != 0 || worst(got, h, n) > 1e-5 || !(ms > 0.0f && ms < 100.0f)) failures++;
        /* And without a workspace: the entry point for callers that cannot allocate gives the same bits. */
        HIP_OK(hipMemset(o0, 0, n * 4));
        if (scanscam_scan_fwd_noalloc(da, db, o0, rows, T, SCANSCAM_F32, stream) != SCANSCAM_OK) failures++;
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(got, o0, n * 4, hipMemcpyDeviceToHost));
        if (memcmp(got, again, n * 4) != 0) failures++;
        {
            int expired = -1;
            if (scanscam_noalloc_timed_out(stream, &expired) != SCANSCAM_OK || expired != 0) failures++;
            if (scanscam_noalloc_timed_out(stream, NULL) != SCANSCAM_EINVAL) failures++;
        }
        if (scanscam_scan_bwd_plan(da, dh, dgh, o1, o0, rows, T, SCANSCAM_F32, ws, ws_bytes, stream, NULL) != SCANSCAM_OK)
            failures++;
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipMemcpy(again, o0, n * 4, hipMemcpyDeviceToHost));
        if (scanscam_scan_bwd_timed(da, dh, dgh, o1, o0, rows, T, SCANSCAM_F32, ws, ws_bytes, stream, NULL, ev0, ev1) !=
            SCANSCAM_OK)
            failures++;
        HIP_OK(hipEventSynchronize(ev1));
        HIP_OK(hipMemcpy(got, o0, n * 4, hipMemcpyDeviceToHost));
        if (memcmp(got, again, n * 4) != 0 || worst(got, gb, n) > 1e-5) failures++;
        printf("abi_check: %-28s _plan and _timed variants agree; forward kernel %.1f us\n", name, ms * 1e3);
        free(again);
        HIP_OK(hipEventDestroy(ev0));
        HIP_OK(hipEventDestroy(ev1));
    }

    hipFree(da); hipFree(db); hipFree(dgh); hipFree(dh); hipFree(o0); hipFree(o1);
    if (ws) hipFree(ws);
    free(a); free(b); free(gh); free(h); free(ga); free(gb); free(got);
    return failures;
}

/*
 * Strided entry points on the two halves of one buffer x: row layout x[B][2C][T] with a = x[:, :C],
 * b = x[:, C:]; channels-last x[B][T][2C] with a = x[..., :C], b = x[..., C:]. Outputs are dense.
 */
static int check_strided(const char *name, long B, long C, long T, int channels_last, hipStream_t stream)
{
    const size_t n = (size_t)B * C * T;
    float *x = malloc(2 * n * 4), *gh = malloc(n * 4), *h = malloc(n * 4), *ga = malloc(n * 4), *gb = malloc(n * 4),
          *got = malloc(n * 4);
    /* element (batch i, channel c, time t): in a half of x, and in a dense tensor of the same layout */
#define XIDX(i, c, t) (channels_last ? ((size_t)(i) * T + (t)) * 2 * C + (c) : ((size_t)(i) * 2 * C + (c)) * T + (t))
#define DIDX(i, c, t) (channels_last ? ((size_t)(i) * T + (t)) * C + (c) : ((size_t)(i) * C + (c)) * T + (t))
    const size_t b_off = channels_last ? (size_t)C : (size_t)C * T; /* where the second half starts */
    for (size_t i = 0; i < 2 * n; i++) x[i] = uniform01();
    for (size_t i = 0; i < n; i++) gh[i] = 2.0f * uniform01() - 1.0f;
    for (long i = 0; i < B; i++)
        for (long c = 0; c < C; c++) {
            float acc = 0.0f;
            for (long t = 0; t < T; t++) {
                acc = acc * x[XIDX(i, c, t)] + x[XIDX(i, c, t) + b_off];
                h[DIDX(i, c, t)] = acc;
            }
            float d = 0.0f;
            for (long t = T - 1; t >= 0; t--) {
                d += gh[DIDX(i, c, t)];
                gb[DIDX(i, c, t)] = d;
                ga[DIDX(i, c, t)] = d * (t > 0 ? h[DIDX(i, c, t - 1)] : 0.0f);
                d *= x[XIDX(i, c, t)];
            }
        }
#undef XIDX
#undef DIDX
    float *dx = device_copy(x, 2 * n), *dgh = device_copy(gh, n), *dh = device_copy(h, n);
    float *o0, *o1;
    HIP_OK(hipMalloc((void **)&o0, n * 4));
    HIP_OK(hipMalloc((void **)&o1, n * 4));
    size_t ws_bytes = 0;
    for (int dir = 0; dir < 2; dir++) {
        size_t need = channels_last ? scanscam_workspace_bytes_cl(B, T, C, SCANSCAM_F32, dir, NULL)
                                    : scanscam_workspace_bytes(B * C, T, SCANSCAM_F32, dir);
        if (need > ws_bytes) ws_bytes = need;
    }
    void *ws = NULL;
    if (ws_bytes) HIP_OK(hipMalloc(&ws, ws_bytes));

    /* both halves have the strides of x; NULL = dense */
    const scanscam_strides sx = {2 * C * T, channels_last ? 2 * C : T};
    int failures = 0;
    int rc = channels_last ? scanscam_scan_fwd_cl_strided(dx, dx + b_off, o0, &sx, &sx, NULL, B, T, C, SCANSCAM_F32, ws,
                                                          ws_bytes, stream, NULL)
                           : scanscam_scan_fwd_strided(dx, dx + b_off, o0, &sx, &sx, NULL, B, C, T, SCANSCAM_F32, ws,
                                                       ws_bytes, stream, NULL);
    if (rc != SCANSCAM_OK) {
        fprintf(stderr, "abi_check: %s forward: %s\n", name, scanscam_strerror(rc));
        failures++;
    }
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(got, o0, n * 4, hipMemcpyDeviceToHost));
    const double eh = worst(got, h, n);
    rc = channels_last ? scanscam_scan_bwd_cl_strided(dx, dh, dgh, o1, o0, &sx, NULL, NULL, NULL, NULL, B, T, C,
                                                      SCANSCAM_F32, ws, ws_bytes, stream, NULL)
                       : scanscam_scan_bwd_strided(dx, dh, dgh, o1, o0, &sx, NULL, NULL, NULL, NULL, B, C, T,
                                                   SCANSCAM_F32, ws, ws_bytes, stream, NULL);
    if (rc != SCANSCAM_OK) {
        fprintf(stderr, "abi_check: %s backward: %s\n", name, scanscam_strerror(rc));
        failures++;
    }
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(got, o0, n * 4, hipMemcpyDeviceToHost));
    const double egb = worst(got, gb, n);
    HIP_OK(hipMemcpy(got, o1, n * 4, hipMemcpyDeviceToHost));
    const double ega = worst(got, ga, n);
    printf("abi_check: %-28s workspace %8zu B  worst relative error h %.2e  grad_b %.2e  grad_a %.2e\n", name,
           ws_bytes, eh, egb, ega);
    if (!(eh <= 1e-5) || !(egb <= 1e-5) || !(ega <= 2e-5)) failures++;
    hipFree(dx); hipFree(dgh); hipFree(dh); hipFree(o0); hipFree(o1);
    if (ws) hipFree(ws);
    free(x); free(gh); free(h); free(ga); free(gb); free(got);
    return failures;
}

int main(void)
{
    if (scanscam_abi_version() != 3) {
        fprintf(stderr, "abi_check: unexpected ABI version %d\n", scanscam_abi_version());
        return 1;
    }
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    int failures = 0;
    failures += check_case("rows [512, 4096]", 512, 4096, 0, 0, stream);
    failures += check_case("short rows [3000, 64]", 3000, 64, 0, 0, stream);
    failures += check_case("odd length [33, 1025]", 33, 1025, 0, 0, stream);
    failures += check_case("long rows [3, 300000]", 3, 300000, 0, 0, stream);
    failures += check_case("channels-last [4, 999, 320]", 4 * 320, 999, 320, 1, stream);
    failures += check_case("channels-last [1, 2048, 64]", 64, 2048, 64, 1, stream);
    failures += check_strided("halves of x[6][2*40][1000]", 6, 40, 1000, 0, stream);
    failures += check_strided("halves of x[2][2*3][200000]", 2, 3, 200000, 0, stream);
    failures += check_strided("halves of x[5][777][2*192]", 5, 192, 777, 1, stream);
    /* Argument errors come back as codes, with nothing launched. */
    if (scanscam_scan_fwd(NULL, NULL, NULL, 4, 8, SCANSCAM_F32, NULL, 0, stream) != SCANSCAM_EINVAL) failures++;
    if (scanscam_scan_fwd(NULL, NULL, NULL, 0, 8, SCANSCAM_F32, NULL, 0, stream) != SCANSCAM_OK) failures++;
    HIP_OK(hipStreamDestroy(stream));
    if (failures) {
        fprintf(stderr, "abi_check: %d failure(s)\n", failures);
        return 1;
    }
    printf("abi_check: ok\n");
    return 0;
}

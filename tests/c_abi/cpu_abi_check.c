/*
 * A plain-C99 consumer of libscanscam_cpu.so (include/scanscam_cpu.h): calls the
 * four entry points on host arrays and compares every result, bit for bit, with
 * the textbook loop written out here (one row at a time, multiply then add;
 * build with -ffp-contract=off so that this file rounds twice as well).
 * Prints "cpu_abi_check: ok" and returns 0 when everything matches.
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "scanscam_cpu.h"

static uint64_t state = 0x9E3779B97F4A7C15ull;
static double uniform(void) /* xorshift64*, in (-1, 1) */
{
    state ^= state >> 12;
    state ^= state << 25;
    state ^= state >> 27;
    return (double)((state * 0x2545F4914F6CDD1Dull) >> 11) / 4503599627370496.0 - 1.0;
}

#define CHECK_TYPE(T, SUFFIX)                                                                              \
    static int check_##SUFFIX(int64_t rows, int64_t len)                                                   \
    {                                                                                                      \
        const size_t n = (size_t)(rows * len), bytes = (n ? n : 1) * sizeof(T);                            \
        T *a = malloc(bytes), *b = malloc(bytes), *gh = malloc(bytes), *h = malloc(bytes),                 \
          *ga = malloc(bytes), *gb = malloc(bytes), *wh = malloc(bytes), *wga = malloc(bytes),             \
          *wgb = malloc(bytes);                                                                            \
        for (size_t i = 0; i < n; i++) {                                                                   \
            a[i] = (T)uniform();                                                                           \
            b[i] = (T)uniform();                                                                           \
            gh[i] = (T)uniform();                                                                          \
        }                                                                                                  \
        for (int64_t r = 0; r < rows; r++) {                                                               \
            T acc = 0;                                                                                     \
            for (int64_t t = 0; t < len; t++) {                                                            \
                acc = acc * a[r * len + t];                                                                \
                acc = acc + b[r * len + t];                                                                \
                wh[r * len + t] = acc;                                                                     \
            }                                                                                              \
            T d = 0;                                                                                       \
            for (int64_t t = len - 1; t >= 0; t--) {                                                       \
                const T prev = t > 0 ? wh[r * len + t - 1] : (T)0;                                         \
                d = d + gh[r * len + t];                                                                   \
                wgb[r * len + t] = d;                                                                      \
                wga[r * len + t] = d * prev;                                                               \
                d = d * a[r * len + t];                                                                    \
            }                                                                                              \
        }                                                                                                  \
        int bad = scanscam_cpu_fwd_##SUFFIX(a, b, h, rows, len);                                           \
        bad |= scanscam_cpu_bwd_##SUFFIX(a, h, gh, ga, gb, rows, len);                                     \
        bad |= memcmp(h, wh, n * sizeof(T)) != 0;                                                          \
        bad |= memcmp(ga, wga, n * sizeof(T)) != 0;                                                        \
        bad |= memcmp(gb, wgb, n * sizeof(T)) != 0;                                                        \
        if (bad) fprintf(stderr, "cpu_abi_check: %s [%lld, %lld] differs\n", #SUFFIX, (long long)rows,     \
                         (long long)len);                                                                  \
        free(a); free(b); free(gh); free(h); free(ga); free(gb); free(wh); free(wga); free(wgb);           \
        return bad;                                                                                        \
    }

CHECK_TYPE(float, f32)
CHECK_TYPE(double, f64)

int main(void)
{
    static const int64_t shapes[][2] = {{1, 1}, {3, 5}, {8, 16}, {9, 15}, {17, 129}, {32, 1025}, {5, 4096}, {0, 7}, {7, 0}};
    int bad = 0;
    for (size_t i = 0; i < sizeof(shapes) / sizeof(shapes[0]); i++) {
        bad |= check_f32(shapes[i][0], shapes[i][1]);
        bad |= check_f64(shapes[i][0], shapes[i][1]);
    }
    bad |= scanscam_cpu_fwd_f32(NULL, NULL, NULL, 2, 3) != 1; /* null pointers with work to do */
    bad |= scanscam_cpu_bwd_f64(NULL, NULL, NULL, NULL, NULL, -1, 3) != 1;
    if (bad) return 1;
    printf("cpu_abi_check: ok\n");
    return 0;
}

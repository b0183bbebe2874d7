/*
 * CPU oracle for the first-order gated linear scan. TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the HIP kernels are compared against. It is
 * never linked into, imported by, or called from the shipped library or the
 * Python package; only tests, the smoke check and the cpu_baseline leg of the
 * benchmark may load it.
 *
 * Each loop restates, operation for operation, the single-threaded CPU
 * implementation of the reference:
 *   forward   src/scanscam_cpu.hpp:9-28   (acc *= g; acc += v; store)
 *   backward  src/scanscam_cpu.hpp:54-78  (d += gh; gb = d; ga = d * h[j-1]; d *= a)
 * The multiply and the add are kept as two separately rounded operations
 * (compile with -ffp-contract=off) so that results are bit-identical to the
 * reference built without FMA contraction. Row offsets are 64-bit here (the
 * reference indexes with int; the results are the same below 2^31 elements).
 *
 * How each function is pinned (none is "parity unpinned"):
 *   oracle_fwd_f32 / _f64, oracle_bwd_f32 / _f64:
 *     - bit-exact against the reference's own C++ loop compiled from its
 *       sources into oracle/_ref (tests/test_oracle.py, golden fixtures under
 *       tests/golden/ written from that build);
 *     - closed forms (a==1 -> cumsum, a==0 -> copy, geometric series),
 *       brute-force sum-of-products on tiny inputs, torch.autograd through an
 *       independent tensor-level loop for the backward pair.
 *   oracle_fwd_f32_acc64 / oracle_bwd_f32_acc64: the same recurrences carried
 *     in double, used only to report reassociation error; pinned by the same
 *     closed forms and by agreement with the f64 functions on upcast inputs.
 */
#include <stddef.h>
#include <stdint.h>

#define DEFINE_FWD(NAME, T)                                                   \
    void NAME(const T *gate, const T *value, T *output, int64_t rows,         \
              int64_t len)                                                    \
    {                                                                         \
        for (int64_t i = 0; i < rows; i++) {                                  \
            const T *g = gate + i * len;                                      \
            const T *v = value + i * len;                                     \
            T *o = output + i * len;                                          \
            T acc = (T)0.0;                                                   \
            for (int64_t j = 0; j < len; j++) {                               \
                acc *= g[j];                                                  \
                acc += v[j];                                                  \
                o[j] = acc;                                                   \
            }                                                                 \
        }                                                                     \
    }

#define DEFINE_BWD(NAME, T)                                                   \
    void NAME(const T *gate, const T *output, const T *out_grad,              \
              T *gate_grad, T *value_grad, int64_t rows, int64_t len)         \
    {                                                                         \
        for (int64_t i = 0; i < rows; i++) {                                  \
            const int64_t base = i * len;                                     \
            T d = (T)0.0;                                                     \
            for (int64_t j = len - 1; j >= 0; j--) {                          \
                T prev = (T)0.0;                                              \
                if (j > 0) {                                                  \
                    prev = output[base + j - 1];                              \
                }                                                             \
                d += out_grad[base + j];                                      \
                T g = gate[base + j];                                         \
                value_grad[base + j] = d;                                     \
                gate_grad[base + j] = d * prev;                               \
                d *= g;                                                       \
            }                                                                 \
        }                                                                     \
    }

DEFINE_FWD(oracle_fwd_f32, float)
DEFINE_FWD(oracle_fwd_f64, double)
DEFINE_BWD(oracle_bwd_f32, float)
DEFINE_BWD(oracle_bwd_f64, double)

/* fp32 inputs, recurrence carried in double, double outputs: the yardstick
 * for "how far is an fp32 result from the exactly-carried recurrence". */
void oracle_fwd_f32_acc64(const float *gate, const float *value, double *output,
                          int64_t rows, int64_t len)
{
    for (int64_t i = 0; i < rows; i++) {
        const float *g = gate + i * len;
        const float *v = value + i * len;
        double *o = output + i * len;
        double acc = 0.0;
        for (int64_t j = 0; j < len; j++) {
            acc *= (double)g[j];
            acc += (double)v[j];
            o[j] = acc;
        }
    }
}

void oracle_bwd_f32_acc64(const float *gate, const float *output,
                          const float *out_grad, double *gate_grad,
                          double *value_grad, int64_t rows, int64_t len)
{
    for (int64_t i = 0; i < rows; i++) {
        const int64_t base = i * len;
        double d = 0.0;
        for (int64_t j = len - 1; j >= 0; j--) {
            double prev = 0.0;
            if (j > 0) {
                prev = (double)output[base + j - 1];
            }
            d += (double)out_grad[base + j];
            value_grad[base + j] = d;
            gate_grad[base + j] = d * prev;
            d *= (double)gate[base + j];
        }
    }
}

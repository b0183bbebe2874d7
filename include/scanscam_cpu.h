/*
 * scanscam_cpu.h -- C ABI of libscanscam_cpu.so: the gated linear scan
 * h[t] = a[t]*h[t-1] + b[t] and its backward pass for tensors that live in
 * host memory.
 *
 * The reference dispatches CPU tensors to its own native loop
 * (scanscam/op.py:33-34 -> scanscam/cpu.py:16-35 -> src/scanscam_cpu.hpp:30-52,
 * 80-113, bound with pybind11 in src/scanscam_cpu.cpp:3-8); these entry points
 * take the place of those two functions for a binding without torch types.
 * GPU tensors never come here: they are scanned by libscanscam_hip.so
 * (scanscam_hip.h) or not at all.
 *
 * Conventions (those of the reference's functions): dense row-major
 * [rows, T] arrays of one type, scanned along T; the caller allocates every
 * output; nothing is kept between calls; the call returns when the result is
 * written. Results are bit-identical to the reference's loop compiled without
 * floating-point contraction: per row the same operations in the same order,
 * multiply and add rounded separately. Several rows are advanced together so
 * that their loop-carried chains overlap; rows do not interact.
 *
 * Return value: 0 on success, 1 (null pointer with rows*T > 0, or a negative
 * size) otherwise. rows == 0 or T == 0 is a successful no-op.
 */
#ifndef SCANSCAM_CPU_H
#define SCANSCAM_CPU_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* simple_linear_scan_cpu(gate, value, output) -- src/scanscam_cpu.hpp:30-52 (float, double: :43) */
int scanscam_cpu_fwd_f32(const float *gate, const float *value, float *output, int64_t rows, int64_t T);
int scanscam_cpu_fwd_f64(const double *gate, const double *value, double *output, int64_t rows, int64_t T);

/* simple_linear_scan_backward_cpu(gate, output, outGrad, gateGradOut, valueGradOut) --
 * src/scanscam_cpu.hpp:80-113. gate_grad[r, 0] = value_grad[r, 0] * 0 is a multiplication, as there (:67-74). */
int scanscam_cpu_bwd_f32(const float *gate, const float *output, const float *out_grad, float *gate_grad,
                         float *value_grad, int64_t rows, int64_t T);
int scanscam_cpu_bwd_f64(const double *gate, const double *output, const double *out_grad, double *gate_grad,
                         double *value_grad, int64_t rows, int64_t T);

#ifdef __cplusplus
}
#endif

#endif /* SCANSCAM_CPU_H */

// libscanscam_cpu.so (declared in include/scanscam_cpu.h): the scan for tensors in host memory.
//
// Per row this is the reference's loop (src/scanscam_cpu.hpp:17-27 forward, :64-77 backward): one
// running value, multiplied by the gate and then added to, two roundings (build with
// -ffp-contract=off). That chain is latency-bound, one element per multiply + add latency, so kLanes
// rows are advanced side by side: their chains are independent and overlap in the pipeline, and each
// row still sees exactly the reference's operations in the reference's order.
#include "scanscam_cpu.h"

namespace {

constexpr int kLanes = 8;  // rows advanced together

// Row r runs kSkew elements behind row r - 1: rows whose length in bytes is a multiple of 4 KiB
// would otherwise touch, in the same iteration, addresses that differ by a multiple of 4 KiB in
// every stream -- one L1 set for all of them, and stores that look like hits to the loads after them.
constexpr int64_t kSkew = 16;

template <typename T, int R> void forward_rows(const T *gate, const T *value, T *output, int64_t len)
{
    T acc[R];
    for (int r = 0; r < R; r++) acc[r] = T(0);
    auto step = [&](int r, int64_t j) {
        const int64_t k = r * len + j;
        T x = acc[r] * gate[k];
        x = x + value[k];
        output[k] = x;
        acc[r] = x;
    };
    const int64_t lag = (R - 1) * kSkew;
    int64_t s = 0;
    for (; s < lag && s < len + lag; s++)  // rows enter one by one
        for (int r = 0; r < R; r++)
            if (s - r * kSkew >= 0 && s - r * kSkew < len) step(r, s - r * kSkew);
    for (; s < len; s++)  // all rows under way
        for (int r = 0; r < R; r++) step(r, s - r * kSkew);
    for (; s < len + lag; s++)  // rows leave one by one
        for (int r = 0; r < R; r++)
            if (s - r * kSkew >= 0 && s - r * kSkew < len) step(r, s - r * kSkew);
}

template <typename T, int R>
void backward_rows(const T *gate, const T *output, const T *out_grad, T *gate_grad, T *value_grad, int64_t len)
{
    T d[R];
    for (int r = 0; r < R; r++) d[r] = T(0);
    auto step = [&](int r, int64_t j) {
        const int64_t k = r * len + j;
        // h[-1] is the value 0 and enters as a factor: an infinite gradient at t = 0 gives NaN.
        const T prev = j > 0 ? output[k - 1] : T(0);
        const T g = d[r] + out_grad[k];
        value_grad[k] = g;
        gate_grad[k] = g * prev;
        d[r] = g * gate[k];
    };
    // s counts steps from the end of the rows: row r is at element len - 1 - (s - r * kSkew).
    const int64_t lag = (R - 1) * kSkew;
    int64_t s = 0;
    for (; s < lag && s < len + lag; s++)
        for (int r = 0; r < R; r++)
            if (s - r * kSkew >= 0 && s - r * kSkew < len) step(r, len - 1 - (s - r * kSkew));
    for (; s < len; s++)
        for (int r = 0; r < R; r++) step(r, len - 1 - (s - r * kSkew));
    for (; s < len + lag; s++)
        for (int r = 0; r < R; r++)
            if (s - r * kSkew >= 0 && s - r * kSkew < len) step(r, len - 1 - (s - r * kSkew));
}

template <typename T> int forward(const T *gate, const T *value, T *output, int64_t rows, int64_t len)
{
    if (rows < 0 || len < 0) return 1;
    if (rows == 0 || len == 0) return 0;
    if (!gate || !value || !output) return 1;
    int64_t i = 0;
    for (; i + kLanes <= rows; i += kLanes)
        forward_rows<T, kLanes>(gate + i * len, value + i * len, output + i * len, len);
    for (; i < rows; i++) forward_rows<T, 1>(gate + i * len, value + i * len, output + i * len, len);
    return 0;
}

template <typename T>
int backward(const T *gate, const T *output, const T *out_grad, T *gate_grad, T *value_grad, int64_t rows,
             int64_t len)
{
    if (rows < 0 || len < 0) return 1;
    if (rows == 0 || len == 0) return 0;
    if (!gate || !output || !out_grad || !gate_grad || !value_grad) return 1;
    int64_t i = 0;
    for (; i + kLanes <= rows; i += kLanes)
        backward_rows<T, kLanes>(gate + i * len, output + i * len, out_grad + i * len, gate_grad + i * len,
                                 value_grad + i * len, len);
    for (; i < rows; i++)
        backward_rows<T, 1>(gate + i * len, output + i * len, out_grad + i * len, gate_grad + i * len,
                            value_grad + i * len, len);
    return 0;
}

}  // namespace

extern "C" {

int scanscam_cpu_fwd_f32(const float *gate, const float *value, float *output, int64_t rows, int64_t T)
{
    return forward<float>(gate, value, output, rows, T);
}

int scanscam_cpu_fwd_f64(const double *gate, const double *value, double *output, int64_t rows, int64_t T)
{
    return forward<double>(gate, value, output, rows, T);
}

int scanscam_cpu_bwd_f32(const float *gate, const float *output, const float *out_grad, float *gate_grad,
                         float *value_grad, int64_t rows, int64_t T)
{
    return backward<float>(gate, output, out_grad, gate_grad, value_grad, rows, T);
}

int scanscam_cpu_bwd_f64(const double *gate, const double *output, const double *out_grad, double *gate_grad,
                         double *value_grad, int64_t rows, int64_t T)
{
    return backward<double>(gate, output, out_grad, gate_grad, value_grad, rows, T);
}

}  // extern "C"

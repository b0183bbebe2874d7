// Host-side launch plumbing shared by the per-dtype translation units.
#pragma once

#include "scan_kernels.hpp"

namespace scanscam {

enum Mode { kModeSmall = 1, kModeRow = 2, kModeLookback = 3 };

// A fully resolved launch: which kernel, with which shape.
struct Launch {
    int mode;
    int vec;     // elements per lane per load: 16 / sizeof(storage), or 1
    int unroll;  // chunks per wave per tile (U)
    int waves;   // waves per workgroup
    int wpr;     // ROW: waves per row
    int group;   // SMALL: lanes per row
    int64_t grid;
};

// Largest workgroup (threads) a kernel with U chunks per wave is compiled for.
constexpr int max_threads_for_unroll(int unroll) { return unroll <= 2 ? 1024 : unroll <= 4 ? 512 : 256; }

// One per storage type, defined in scan_f32.hip / scan_bf16.hip / scan_f16.hip.
// Returns hipErrorInvalidValue when (vec, unroll) is not an instantiated pair.
template <typename ST>
hipError_t launch_scan(const ScanArgs &args, const Launch &l, bool rev, hipStream_t stream);

#define SCANSCAM_LAUNCH_CASE(ST, VEC, U)                                                             \
    if (l.vec == (VEC) && l.unroll == (U)) {                                                         \
        constexpr int MAXT = max_threads_for_unroll(U);                                              \
        if (l.mode == kModeSmall) {                                                                  \
            if (rev) hipLaunchKernelGGL((scan_small_kernel<ST, VEC, U, true, MAXT>), grid, block, 0, stream, args);    \
            else     hipLaunchKernelGGL((scan_small_kernel<ST, VEC, U, false, MAXT>), grid, block, 0, stream, args);   \
        } else if (l.mode == kModeRow) {                                                             \
            if (rev) hipLaunchKernelGGL((scan_row_kernel<ST, VEC, U, true, MAXT>), grid, block, 0, stream, args);      \
            else     hipLaunchKernelGGL((scan_row_kernel<ST, VEC, U, false, MAXT>), grid, block, 0, stream, args);     \
        } else {                                                                                     \
            if (rev) hipLaunchKernelGGL((scan_lookback_kernel<ST, VEC, U, true, MAXT>), grid, block, 0, stream, args); \
            else     hipLaunchKernelGGL((scan_lookback_kernel<ST, VEC, U, false, MAXT>), grid, block, 0, stream, args);\
        }                                                                                            \
        return hipGetLastError();                                                                    \
    }

#define SCANSCAM_DEFINE_LAUNCH(ST)                                                                   \
    template <>                                                                                      \
    hipError_t launch_scan<ST>(const ScanArgs &args, const Launch &l, bool rev, hipStream_t stream)  \
    {                                                                                                \
        constexpr int FULL = 16 / (int)sizeof(ST);                                                   \
        const dim3 grid((unsigned)l.grid), block((unsigned)(l.waves * kWave));                       \
        SCANSCAM_LAUNCH_CASE(ST, FULL, 1)                                                            \
        SCANSCAM_LAUNCH_CASE(ST, FULL, 2)                                                            \
        SCANSCAM_LAUNCH_CASE(ST, FULL, 4)                                                            \
        SCANSCAM_LAUNCH_CASE(ST, FULL, 8)                                                            \
        SCANSCAM_LAUNCH_CASE(ST, 1, 1)                                                               \
        SCANSCAM_LAUNCH_CASE(ST, 1, 4)                                                               \
        return hipErrorInvalidValue;                                                                 \
    }

}  // namespace scanscam

// Host-side launch plumbing shared by the per-dtype translation units.
#pragma once

#include <hip/hip_ext.h>

#include "scan_cl_kernels.hpp"
#include "scan_flat_kernels.hpp"
#include "scan_kernels.hpp"

namespace scanscam {

enum Mode { kModeSmall = 1, kModeRow = 2, kModeLookback = 3, kModeFlat = 4 };

// A fully resolved launch: which kernel, with which shape.
struct Launch {
    int mode;
    int vec;     // elements per lane per load: 16 / sizeof(storage), or 1
    int unroll;  // chunks per wave per tile (U)
    int waves;   // waves per workgroup
    int wpr;     // ROW: waves per row
    int group;   // SMALL: lanes per row
    int64_t grid;
    bool ragged; // ROW / LOOKBACK with the full vector on rows that start at any element
    int grid_y;  // ROW / SMALL: groups of rows (blockIdx.y); 1 for LOOKBACK
};

// Largest workgroup (threads) a kernel with U chunks per wave is compiled for.
constexpr int max_threads_for_unroll(int unroll) { return unroll <= 4 ? 1024 : 512; }

// Launches `kernel(args)` and returns what the launch call itself returns (the runtime's sticky "last error" is
// neither read nor cleared, so an error the host application left there is not taken for this launch's, and
// stays there for the application to find). `start` / `stop` (may be null) receive the kernel's own time stamps.
template <typename Kernel, typename Args>
inline hipError_t launch_kernel(Kernel kernel, dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                                hipEvent_t start, hipEvent_t stop, const Args &args)
{
    Args copy = args;
    void *params[] = {&copy};
    return hipExtLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, params, lds_bytes, stream, start, stop, 0);
}

// One per storage type, defined in scan_f32.hip / scan_bf16.hip / scan_f16.hip.
// Returns hipErrorInvalidValue when (vec, unroll) is not an instantiated pair. `start` / `stop`
// (may be null) receive the kernel's own start and end time stamps.
template <typename ST>
hipError_t launch_scan(const ScanArgs &args, const Launch &l, bool rev, hipStream_t stream, hipEvent_t start,
                       hipEvent_t stop);

#define SCANSCAM_LAUNCH_CASE(ST, VEC, U)                                                             \
    if (l.vec == (VEC) && l.unroll == (U)) {                                                         \
        constexpr int MAXT = max_threads_for_unroll(U);                                              \
        hipError_t err = hipErrorInvalidValue;                                                       \
        if (l.mode == kModeSmall) {                                                                  \
            if (rev) err = launch_kernel(scan_small_kernel<ST, VEC, U, true, MAXT>, grid, block, 0, stream, start, stop, args);    \
            else     err = launch_kernel(scan_small_kernel<ST, VEC, U, false, MAXT>, grid, block, 0, stream, start, stop, args);   \
        } else if (l.mode == kModeRow) {                                                             \
            if (rev) err = launch_kernel(scan_row_kernel<ST, VEC, U, true, MAXT>, grid, block, 0, stream, start, stop, args);      \
            else     err = launch_kernel(scan_row_kernel<ST, VEC, U, false, MAXT>, grid, block, 0, stream, start, stop, args);     \
        } else {                                                                                     \
            if (rev) err = launch_kernel(scan_lookback_kernel<ST, VEC, U, true, MAXT>, grid, block, 0, stream, start, stop, args); \
            else     err = launch_kernel(scan_lookback_kernel<ST, VEC, U, false, MAXT>, grid, block, 0, stream, start, stop, args);\
        }                                                                                            \
        return err;                                                                    \
    }

// The same for rows that are only element-aligned (full vector, U = 2 or 4).
#define SCANSCAM_RAGGED_CASE(ST, VEC, U)                                                             \
    if (l.ragged && l.vec == (VEC) && l.unroll == (U)) {                                             \
        constexpr int MAXT = max_threads_for_unroll(U);                                              \
        hipError_t err = hipErrorInvalidValue;                                                       \
        if (l.mode == kModeRow) {                                                                    \
            if (rev) err = launch_kernel(scan_row_kernel<ST, VEC, U, true, MAXT, true>, grid, block, 0, stream, start, stop, args);      \
            else     err = launch_kernel(scan_row_kernel<ST, VEC, U, false, MAXT, true>, grid, block, 0, stream, start, stop, args);     \
        } else if (l.mode == kModeLookback) {                                                        \
            if (rev) err = launch_kernel(scan_lookback_kernel<ST, VEC, U, true, MAXT, true>, grid, block, 0, stream, start, stop, args); \
            else     err = launch_kernel(scan_lookback_kernel<ST, VEC, U, false, MAXT, true>, grid, block, 0, stream, start, stop, args);\
        } else {                                                                                     \
            if (rev) err = launch_kernel(scan_small_kernel<ST, VEC, U, true, MAXT, true>, grid, block, 0, stream, start, stop, args);    \
            else     err = launch_kernel(scan_small_kernel<ST, VEC, U, false, MAXT, true>, grid, block, 0, stream, start, stop, args);   \
        }                                                                                            \
        return err;                                                                    \
    }

#define SCANSCAM_DEFINE_LAUNCH(ST)                                                                   \
    template <>                                                                                      \
    hipError_t launch_scan<ST>(const ScanArgs &args, const Launch &l, bool rev, hipStream_t stream,  \
                               hipEvent_t start, hipEvent_t stop)                                    \
    {                                                                                                \
        constexpr int FULL = 16 / (int)sizeof(ST);                                                   \
        const dim3 grid((unsigned)l.grid, (unsigned)l.grid_y), block((unsigned)(l.waves * kWave));   \
        SCANSCAM_RAGGED_CASE(ST, FULL, 2)                                                            \
        SCANSCAM_RAGGED_CASE(ST, FULL, 3)                                                            \
        SCANSCAM_RAGGED_CASE(ST, FULL, 4)                                                            \
        if (l.ragged) return hipErrorInvalidValue;                                                   \
        SCANSCAM_LAUNCH_CASE(ST, FULL, 1)                                                            \
        SCANSCAM_LAUNCH_CASE(ST, FULL, 2)                                                            \
        SCANSCAM_LAUNCH_CASE(ST, FULL, 3)                                                            \
        SCANSCAM_LAUNCH_CASE(ST, FULL, 4)                                                            \
        SCANSCAM_LAUNCH_CASE(ST, FULL, 8)                                                            \
        SCANSCAM_LAUNCH_CASE(ST, 1, 1)                                                               \
        SCANSCAM_LAUNCH_CASE(ST, 1, 4)                                                               \
        return hipErrorInvalidValue;                                                                 \
    }

// The flat kernel (dense short rows scanned as one stream): `unroll` chunks per wave (2 or 4), `waves` waves
// per workgroup, full vector only. Returns hipErrorInvalidValue for an unroll that is not instantiated.
template <typename ST>
hipError_t launch_scan_flat(const FlatArgs &args, int unroll, int waves, bool rev, hipStream_t stream, hipEvent_t start,
                            hipEvent_t stop);

#define SCANSCAM_FLAT_CASE(ST, U)                                                                     \
    if (unroll == (U)) {                                                                              \
        hipError_t err = hipErrorInvalidValue;                                                        \
        if (rev) err = launch_kernel(scan_flat_kernel<ST, FULL, U, true, 1024>, grid, block, 0, stream, start, stop, args);  \
        else     err = launch_kernel(scan_flat_kernel<ST, FULL, U, false, 1024>, grid, block, 0, stream, start, stop, args); \
        return err;                                                                     \
    }

#define SCANSCAM_DEFINE_FLAT_LAUNCH(ST)                                                               \
    template <>                                                                                       \
    hipError_t launch_scan_flat<ST>(const FlatArgs &args, int unroll, int waves, bool rev, hipStream_t stream, \
                                    hipEvent_t start, hipEvent_t stop)                                \
    {                                                                                                 \
        constexpr int FULL = 16 / (int)sizeof(ST);                                                    \
        const int64_t per_wg = (int64_t)waves * unroll * kWave * FULL;                                \
        /* backwards the kernel shifts its positions by up to one chunk, to sit on line borders */   \
        const int64_t positions = args.N + (rev ? kWave * FULL - 1 : 0);                              \
        const dim3 grid((unsigned)((positions + per_wg - 1) / per_wg)), block((unsigned)(waves * kWave)); \
        SCANSCAM_FLAT_CASE(ST, 2)                                                                     \
        SCANSCAM_FLAT_CASE(ST, 4)                                                                     \
        return hipErrorInvalidValue;                                                                  \
    }

// Channels-last launches. `steps` = time steps per wave per tile (S).
struct ClLaunch {
    int vec;
    int steps;
    int waves;
    int kind;       // 0: a workgroup walks all of T; 2: tiles over workgroups with a look-back chain
    int group;      // kind 0: lanes per time step; below 64: the packed kernel for few channels
    int segments;   // kind 2: tiles per row-group
    bool ragged;    // kind 0, full lanes of a wave: lanes of vec channels on time steps that are only element-aligned,
                    // or whose C is no multiple of vec
    int64_t grid;
    size_t lds_bytes;
    size_t ws_bytes;
};

constexpr int cl_max_threads(int vec, int steps) { return (vec > 1 && steps >= 8) ? 512 : 1024; }

template <typename ST>
hipError_t launch_scan_cl(const ClArgs &args, const ClLaunch &l, bool rev, hipStream_t stream);

#define SCANSCAM_CL_CASE(ST, VEC, S)                                                                   \
    if (l.vec == (VEC) && l.steps == (S)) {                                                            \
        constexpr int MAXT = cl_max_threads(VEC, S);                                                   \
        hipError_t err = hipErrorInvalidValue;                                                         \
        if (l.kind == 2) {                                                                             \
            if (rev) err = launch_kernel(scan_cl_lookback_kernel<ST, VEC, S, true, MAXT>, grid, block, l.lds_bytes, stream, nullptr, nullptr, args);  \
            else     err = launch_kernel(scan_cl_lookback_kernel<ST, VEC, S, false, MAXT>, grid, block, l.lds_bytes, stream, nullptr, nullptr, args); \
        } else if (l.group < kWave) {                                                                  \
            if (rev) err = launch_kernel(scan_cl_packed_kernel<ST, VEC, S, true, MAXT>, grid, block, l.lds_bytes, stream, nullptr, nullptr, args);  \
            else     err = launch_kernel(scan_cl_packed_kernel<ST, VEC, S, false, MAXT>, grid, block, l.lds_bytes, stream, nullptr, nullptr, args); \
        } else if (l.ragged) {                                                                         \
            if constexpr ((VEC) > 1) {                                                                 \
                if (rev) err = launch_kernel(scan_cl_kernel<ST, VEC, S, true, MAXT, true>, grid, block, l.lds_bytes, stream, nullptr, nullptr, args);  \
                else     err = launch_kernel(scan_cl_kernel<ST, VEC, S, false, MAXT, true>, grid, block, l.lds_bytes, stream, nullptr, nullptr, args); \
            } else {                                                                                   \
                return hipErrorInvalidValue;                                                           \
            }                                                                                          \
        } else {                                                                                       \
            if (rev) err = launch_kernel(scan_cl_kernel<ST, VEC, S, true, MAXT>, grid, block, l.lds_bytes, stream, nullptr, nullptr, args);  \
            else     err = launch_kernel(scan_cl_kernel<ST, VEC, S, false, MAXT>, grid, block, l.lds_bytes, stream, nullptr, nullptr, args); \
        }                                                                                              \
        return err;                                                                      \
    }

#define SCANSCAM_DEFINE_CL_LAUNCH(ST)                                                                  \
    template <>                                                                                        \
    hipError_t launch_scan_cl<ST>(const ClArgs &args, const ClLaunch &l, bool rev, hipStream_t stream) \
    {                                                                                                  \
        constexpr int FULL = 16 / (int)sizeof(ST);                                                     \
        const dim3 grid((unsigned)l.grid), block((unsigned)(l.waves * kWave));                         \
        SCANSCAM_CL_CASE(ST, FULL, 2)                                                                  \
        SCANSCAM_CL_CASE(ST, FULL, 4)                                                                  \
        SCANSCAM_CL_CASE(ST, FULL, 8)                                                                  \
        SCANSCAM_CL_CASE(ST, 1, 4)                                                                     \
        SCANSCAM_CL_CASE(ST, 1, 8)                                                                     \
        SCANSCAM_CL_CASE(ST, 1, 16)                                                                    \
        if constexpr (sizeof(ST) == 2) { /* 16-bit storage: lanes of two channels (4 bytes) */         \
            SCANSCAM_CL_CASE(ST, 2, 4)                                                                 \
            SCANSCAM_CL_CASE(ST, 2, 8)                                                                 \
            SCANSCAM_CL_CASE(ST, 2, 16)                                                                \
        }                                                                                              \
        if constexpr (sizeof(ST) <= 4) { /* lanes of 8 bytes: two fp32 channels, four 16-bit ones */   \
            constexpr int HALF = FULL / 2;                                                             \
            SCANSCAM_CL_CASE(ST, HALF, 4)                                                              \
            SCANSCAM_CL_CASE(ST, HALF, 8)                                                              \
            SCANSCAM_CL_CASE(ST, HALF, 16)                                                             \
        }                                                                                              \
        return hipErrorInvalidValue;                                                                   \
    }

}  // namespace scanscam

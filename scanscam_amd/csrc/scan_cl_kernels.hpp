// Channels-last variant of the gated linear scan for gfx950: tensors are stored
// [B, T, C] (C fastest) and scanned along T, i.e. the logical [B, C, T] tensor
// is "transpose-contiguous". Same arithmetic as scan_kernels.hpp; replaces the
// reference's transposed_linear_scan / transposed_linear_scan_backward
// (src/scanscam_cuda.cu:471-723), which stage [time x channel] tiles through
// shared memory and scan them with a Hillis-Steele ladder.
//
// Here nothing is transposed. A lane owns VEC consecutive channels (one 16-byte
// vector, or one element), so the 64 lanes of a wave read one contiguous span
// of a time step per instruction, and the recurrence along T is sequential
// inside the lane: no lane ever needs another lane's data. Time is split over
// the waves of a workgroup instead: wave w takes S consecutive steps of each
// tile of W*S steps, folds them to one affine pair per channel, the pairs are
// exchanged through LDS (lane-contiguous, conflict-free), every wave forms its
// carry-in by folding the pairs of the waves before it, and replays its steps.
// Tile to tile the carry stays in registers. The backward pass walks time
// downwards; its shifted operands a[t+1] and h[t-1] are plain address offsets
// (one row of C elements), so it reads exactly 3 and writes 2 elements per
// element, like the row layout.
#pragma once

#include "scan_kernels.hpp"

namespace scanscam {

struct ClArgs {
    const void *a;  // gates                       [B, T, C]
    const void *x;  // forward: b      backward: gh
    const void *h;  // forward: unused backward: saved forward output
    void *y0;       // forward: h      backward: gb
    void *y1;       // forward: unused backward: ga
    int64_t batch;
    int32_t T;
    int32_t C;
};

// Dynamic LDS: two buffers (tiles alternate) of A and B, each [W][VEC][64] values.
template <typename ST, int VEC, int S, bool REV, int MAXT>
__global__ __launch_bounds__(MAXT) void scan_cl_kernel(const ClArgs p)
{
    using V = Vec<ST, VEC>;
    using raw_t = typename V::raw_t;
    using CT = typename ComputeOf<ST>::type;
    extern __shared__ double lds_raw[];  // 8-byte aligned for either arithmetic type
    CT *lds = reinterpret_cast<CT *>(lds_raw);

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int W = blockDim.x / kWave;
    const int T = p.T, C = p.C;

    const int groups = (C + kWave * VEC - 1) / (kWave * VEC);  // channel groups per batch element
    const int64_t c0 = ((int64_t)(blockIdx.x % groups) * kWave + lane) * VEC;  // first channel of this lane
    const bool c_ok = c0 < C;
    const int64_t base = (int64_t)(blockIdx.x / groups) * T * C + (c_ok ? c0 : 0);
    const ST *a = static_cast<const ST *>(p.a) + base;
    const ST *x = static_cast<const ST *>(p.x) + base;
    const ST *h = static_cast<const ST *>(p.h) + base;
    ST *y0 = static_cast<ST *>(p.y0) + base;
    ST *y1 = static_cast<ST *>(p.y1) + base;

    const int tile_steps = W * S;
    const int ntiles = (T + tile_steps - 1) / tile_steps;
    const int plane = W * VEC * kWave;  // floats per LDS array
    CT carry[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) carry[k] = CT(0);

    for (int it = 0; it < ntiles; it++) {
        CT *lds_A = lds + (it & 1) * 2 * plane;
        CT *lds_B = lds_A + plane;
        const int tau0 = it * tile_steps + wave * S;  // position in scan order

        raw_t ra[S], rx[S], rh[REV ? S : 1];
        bool ok[S];
#pragma unroll
        for (int s = 0; s < S; s++) {
            const int tau = tau0 + s;
            const int t = REV ? T - 1 - tau : tau;
            ok[s] = c_ok && tau < T;
            ra[s] = V::zero_raw();
            rx[s] = V::zero_raw();
            if (!REV) {
                if (ok[s]) {
                    ra[s] = V::load(a + (int64_t)t * C);
                    rx[s] = V::load(x + (int64_t)t * C);
                }
            } else {
                rh[s] = V::zero_raw();
                if (ok[s]) {
                    rx[s] = V::load(x + (int64_t)t * C);
                    if (t + 1 < T) ra[s] = V::load(a + (int64_t)(t + 1) * C);  // gate of the step after; 0 past the end
                    if (t > 0) rh[s] = V::load(h + (int64_t)(t - 1) * C);      // h[-1] = 0
                }
            }
        }

        CT g[S][VEC], v[S][VEC];
        CT A[VEC], B[VEC];
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            A[k] = CT(1);
            B[k] = CT(0);
        }
#pragma unroll
        for (int s = 0; s < S; s++) {
            CT fa[VEC], fx[VEC];
            V::unpack(ra[s], fa);
            V::unpack(rx[s], fx);
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                g[s][k] = ok[s] ? fa[k] : CT(1);
                v[s][k] = fx[k];  // zero where not ok
                B[k] = fma_(g[s][k], B[k], v[s][k]);
                A[k] = A[k] * g[s][k];
            }
        }

        CT mine[VEC];
        if (W > 1) {
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                lds_A[(wave * VEC + k) * kWave + lane] = A[k];
                lds_B[(wave * VEC + k) * kWave + lane] = B[k];
            }
            __syncthreads();
            CT c[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                c[k] = carry[k];
                mine[k] = carry[k];
            }
            for (int q = 0; q < W; q++) {
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    if (q == wave) mine[k] = c[k];
                    c[k] = fma_(lds_A[(q * VEC + k) * kWave + lane], c[k], lds_B[(q * VEC + k) * kWave + lane]);
                }
            }
#pragma unroll
            for (int k = 0; k < VEC; k++) carry[k] = c[k];
        } else {
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                mine[k] = carry[k];
                carry[k] = fma_(A[k], carry[k], B[k]);
            }
        }

#pragma unroll
        for (int s = 0; s < S; s++) {
            const int tau = tau0 + s;
            const int t = REV ? T - 1 - tau : tau;
            CT out[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                mine[k] = fma_(g[s][k], mine[k], v[s][k]);
                out[k] = mine[k];
            }
            if (!REV) {
                if (ok[s]) V::store(y0 + (int64_t)t * C, V::pack(out));
            } else {
                CT fh[VEC], ga[VEC];
                V::unpack(rh[s], fh);
#pragma unroll
                for (int k = 0; k < VEC; k++) ga[k] = out[k] * fh[k];
                if (ok[s]) {
                    V::store(y0 + (int64_t)t * C, V::pack(out));
                    V::store(y1 + (int64_t)t * C, V::pack(ga));
                }
            }
        }
    }
}

}  // namespace scanscam

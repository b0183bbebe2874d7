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
//
// A workgroup owns 64*VEC channels of one batch element. When that gives too
// few workgroups to fill the GPU, time is also cut into segments over
// workgroups (scan_cl_split_kernel): every workgroup first folds its segment
// to one pair per channel (its data stays in the memory-side cache), publishes
// it, collects the pairs of the segments before it, and only then replays its
// segment from the resulting carry.
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
    int32_t segments;   // split kernel: segments of time per (batch element, channel group)
    int32_t seg_steps;  // split kernel: time steps per segment (a multiple of the tile)
    uint64_t *ws;       // split kernel: ticket counters + segment aggregates
    int32_t spin_limit; // split kernel: polls before a wait gives up
};

// One workgroup's view of its channels: pointers already offset to (batch
// element, first channel of the lane).
template <typename ST> struct ClLane {
    const ST *a, *x, *h;
    ST *y0, *y1;
    bool c_ok;
};

// Processes the tile of W*S steps that starts at scan position tile0.
//   APPLY = true   `run` holds the scan value entering the tile per channel; the
//                  tile's outputs are stored and `run` advanced to its end.
//   APPLY = false  `runA`, `run` hold the affine pair of everything folded so
//                  far; the tile's pair is composed onto it; nothing is stored
//                  and loads are left cacheable (the data is read again later).
// lds_A / lds_B: [W][VEC][64] values each; the caller alternates two buffers.
template <typename ST, int VEC, int S, bool REV, bool APPLY, typename CT>
__device__ __forceinline__ void cl_tile(const ClLane<ST> &ln, int T, int C, int tile0, int limit, int wave, int W,
                                        int lane, CT *lds_A, CT *lds_B, CT (&runA)[VEC], CT (&run)[VEC])
{
    using V = Vec<ST, VEC>;
    using raw_t = typename V::raw_t;
    const int tau0 = tile0 + wave * S;  // position in scan order

    // Every load is issued unconditionally, masked lanes from offset 0 of their own column (always
    // valid), and masked by a select afterwards: no branch separates the loads, so all of a wave's
    // S x streams loads are in flight before the first one is waited for.
    raw_t ra[S], rx[S], rh[(REV && APPLY) ? S : 1];
    bool ok[S], a_ok[S], h_ok[S];
#pragma unroll
    for (int s = 0; s < S; s++) {
        const int tau = tau0 + s;
        const int t = REV ? T - 1 - tau : tau;
        ok[s] = ln.c_ok && tau < limit;
        // The gate of step t is a[t] forwards and a[t+1] backwards (0 past the end); h[-1] = 0.
        a_ok[s] = ok[s] && (!REV || t + 1 < T);
        h_ok[s] = ok[s] && t > 0;
        const int64_t off_x = ok[s] ? (int64_t)t * C : 0;
        const int64_t off_a = a_ok[s] ? (int64_t)(REV ? t + 1 : t) * C : 0;
        if (APPLY) {
            ra[s] = V::load(ln.a + off_a);
            rx[s] = V::load(ln.x + off_x);
            if (REV) rh[s] = V::load(ln.h + (h_ok[s] ? (int64_t)(t - 1) * C : 0));
        } else {
            ra[s] = V::load_cached(ln.a + off_a);
            rx[s] = V::load_cached(ln.x + off_x);
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
            g[s][k] = ok[s] ? (a_ok[s] ? fa[k] : CT(0)) : CT(1);
            v[s][k] = ok[s] ? fx[k] : CT(0);
            B[k] = fma_(g[s][k], B[k], v[s][k]);
            A[k] = A[k] * g[s][k];
        }
    }

    CT mine[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) mine[k] = run[k];
    if (W > 1) {
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            lds_A[(wave * VEC + k) * kWave + lane] = A[k];
            lds_B[(wave * VEC + k) * kWave + lane] = B[k];
        }
        __syncthreads();
        for (int q = 0; q < W; q++) {
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                const CT Aq = lds_A[(q * VEC + k) * kWave + lane], Bq = lds_B[(q * VEC + k) * kWave + lane];
                if (APPLY && q == wave) mine[k] = run[k];
                run[k] = fma_(Aq, run[k], Bq);
                if (!APPLY) runA[k] = Aq * runA[k];
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            run[k] = fma_(A[k], run[k], B[k]);
            if (!APPLY) runA[k] = A[k] * runA[k];
        }
    }
    if (!APPLY) return;

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
            if (ok[s]) V::store(ln.y0 + (int64_t)t * C, V::pack(out));
        } else {
            CT fh[VEC], ga[VEC];
            V::unpack(rh[s], fh);
#pragma unroll
            for (int k = 0; k < VEC; k++) ga[k] = out[k] * (h_ok[s] ? fh[k] : CT(0));
            if (ok[s]) {
                V::store(ln.y0 + (int64_t)t * C, V::pack(out));
                V::store(ln.y1 + (int64_t)t * C, V::pack(ga));
            }
        }
    }
}

template <typename ST, int VEC>
__device__ __forceinline__ ClLane<ST> cl_lane(const ClArgs &p, int64_t batch_index, int group, int lane)
{
    const int64_t c0 = ((int64_t)group * kWave + lane) * VEC;  // first channel of this lane
    ClLane<ST> ln;
    ln.c_ok = c0 < p.C;
    const int64_t base = batch_index * p.T * p.C + (ln.c_ok ? c0 : 0);
    ln.a = static_cast<const ST *>(p.a) + base;
    ln.x = static_cast<const ST *>(p.x) + base;
    ln.h = static_cast<const ST *>(p.h) + base;
    ln.y0 = static_cast<ST *>(p.y0) + base;
    ln.y1 = static_cast<ST *>(p.y1) + base;
    return ln;
}

// Dynamic LDS: two buffers (tiles alternate) of A and B, each [W][VEC][64] values.
template <typename ST, int VEC, int S, bool REV, int MAXT>
__global__ __launch_bounds__(MAXT) void scan_cl_kernel(const ClArgs p)
{
    using CT = typename ComputeOf<ST>::type;
    extern __shared__ double lds_raw[];  // 8-byte aligned for either arithmetic type
    CT *lds = reinterpret_cast<CT *>(lds_raw);

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int W = blockDim.x / kWave;
    const int groups = (p.C + kWave * VEC - 1) / (kWave * VEC);  // channel groups per batch element
    const ClLane<ST> ln = cl_lane<ST, VEC>(p, blockIdx.x / groups, blockIdx.x % groups, lane);

    const int tile_steps = W * S;
    const int ntiles = (p.T + tile_steps - 1) / tile_steps;
    const int plane = W * VEC * kWave;  // values per LDS array
    CT carry[VEC], unused[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) carry[k] = CT(0);

    for (int it = 0; it < ntiles; it++) {
        CT *lds_A = lds + (it & 1) * 2 * plane;
        cl_tile<ST, VEC, S, REV, true, CT>(ln, p.T, p.C, it * tile_steps, p.T, wave, W, lane, lds_A, lds_A + plane,
                                           unused, carry);
    }
}

// Time split over workgroups. Workspace, in 64-bit words: ticket counter of
// row-group r (= batch element x channel group) at word r * kCounterStride,
// word 1 raised on a timed-out wait; from word rowgroups * kCounterStride on,
// per (row-group, segment) the segment's pair per channel: A then B, each
// [VEC][64] published values (see Desc<CT>). Zeroed before each launch.
template <typename ST, int VEC, int S, bool REV, int MAXT>
__global__ __launch_bounds__(MAXT) void scan_cl_split_kernel(const ClArgs p)
{
    using CT = typename ComputeOf<ST>::type;
    using D = Desc<CT>;
    extern __shared__ double lds_raw[];
    CT *lds = reinterpret_cast<CT *>(lds_raw);
    __shared__ unsigned lds_ticket;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int W = blockDim.x / kWave;
    const int groups = (p.C + kWave * VEC - 1) / (kWave * VEC);
    const int64_t rowgroups = p.batch * groups;
    const int64_t rg = blockIdx.x % rowgroups;  // neighbouring workgroups hit different counters

    // The ticket is the segment: whoever holds segment s knows that segments 0..s-1 are running.
    if (threadIdx.x == 0)
        lds_ticket = __hip_atomic_fetch_add(reinterpret_cast<unsigned *>(p.ws + rg * kCounterStride), 1u,
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const int seg = (int)__builtin_amdgcn_readfirstlane(lds_ticket);
    const ClLane<ST> ln = cl_lane<ST, VEC>(p, rg / groups, (int)(rg % groups), lane);

    const int tile_steps = W * S;
    const int seg0 = seg * p.seg_steps;
    const int seg_end = (seg0 + p.seg_steps < p.T) ? seg0 + p.seg_steps : p.T;
    const int ntiles = (seg_end - seg0 + tile_steps - 1) / tile_steps;  // <= 0 for an empty trailing segment
    const int plane = W * VEC * kWave;
    constexpr int kSegWords = 2 * VEC * kWave * D::W;
    uint64_t *segs = p.ws + rowgroups * kCounterStride + rg * (int64_t)p.segments * kSegWords;

    // Pass 1: the segment's pair per channel.
    CT aggA[VEC], aggB[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        aggA[k] = CT(1);
        aggB[k] = CT(0);
    }
    for (int it = 0; it < ntiles; it++) {
        CT *lds_A = lds + (it & 1) * 2 * plane;
        cl_tile<ST, VEC, S, REV, false, CT>(ln, p.T, p.C, seg0 + it * tile_steps, seg_end, wave, W, lane, lds_A,
                                            lds_A + plane, aggA, aggB);
    }
    if (wave == 0 && seg + 1 < p.segments) {
        uint64_t *mine = segs + (int64_t)seg * kSegWords;
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            D::store(mine + (k * kWave + lane) * D::W, aggA[k]);
            D::store(mine + ((VEC + k) * kWave + lane) * D::W, aggB[k]);
        }
    }

    // Carry into the segment: the pairs of segments 0..seg-1 applied to 0 in order. Wave w
    // fetches segment w, w + W, ... into LDS; then every lane folds them for its channels.
    CT carry[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) carry[k] = CT(0);
    __syncthreads();  // pass 1 is done with both LDS buffers
    for (int first = 0; first < seg; first += W) {
        const int q = first + wave;
        if (q < seg) {
            const uint64_t *theirs = segs + (int64_t)q * kSegWords;
            CT pa[VEC], pb[VEC];
            bool got = false;
            for (int spin = 0; spin < p.spin_limit && !got; spin++) {
                bool ready = true;
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    ready = D::load(theirs + (k * kWave + lane) * D::W, pa[k]) && ready;
                    ready = D::load(theirs + ((VEC + k) * kWave + lane) * D::W, pb[k]) && ready;
                }
                got = __ballot(ready) == ~0ull;
                if (!got) __builtin_amdgcn_s_sleep(1);
            }
            if (!got) {
                if (lane == 0)
                    __hip_atomic_store(p.ws + kTimeoutWord, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int k = 0; k < VEC; k++) pb[k] = CT(__builtin_nanf(""));
            }
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                lds[(wave * VEC + k) * kWave + lane] = pa[k];
                lds[plane + (wave * VEC + k) * kWave + lane] = pb[k];
            }
        }
        __syncthreads();
        const int count = (seg - first < W) ? seg - first : W;
        for (int w = 0; w < count; w++) {
#pragma unroll
            for (int k = 0; k < VEC; k++)
                carry[k] = fma_(lds[(w * VEC + k) * kWave + lane], carry[k], lds[plane + (w * VEC + k) * kWave + lane]);
        }
        __syncthreads();
    }

    // Pass 2: replay the segment from its carry (its data is still in the memory-side cache).
    CT unused[VEC];
    for (int it = 0; it < ntiles; it++) {
        CT *lds_A = lds + (it & 1) * 2 * plane;
        cl_tile<ST, VEC, S, REV, true, CT>(ln, p.T, p.C, seg0 + it * tile_steps, seg_end, wave, W, lane, lds_A,
                                           lds_A + plane, unused, carry);
    }
}

}  // namespace scanscam

// Short rows of any length, dense tensors: the FLAT kernel.
//
// Rows of up to one chunk (64 lanes x 16 bytes) whose vector count is not a power of two leave lanes of the
// SMALL kernel idle (33 vectors take a group of 64 lanes), and rows whose length is no multiple of the vector
// width make its accesses element-aligned. A dense [rows, T] tensor, though, is one contiguous array of
// rows * T elements: this kernel scans that array as ONE stream, every lane a 16-byte aligned vector of it,
// every load and store instruction a whole 1 KiB span, no lane idle -- and resets the recurrence where a row
// starts. A vector may straddle a row border (at most one: T >= VEC).
//
// The reset is a third component of the scanned pairs, not a gate of zero: an element's map is
//     x -> fma(g, R ? 0 : x, v)          R = "the scan enters a new row here"
// and a run of elements composes to (A, B, F): x -> F ? B : fma(A, x, B), with
//     (A2, B2, F2) o (A1, B1, F1) = (A2*A1, F2 ? B2 : fma(A2, B1, B2), F1 | F2),
// so nothing of one row (an infinity, a NaN) can reach the next through 0 * inf. At a row's first element
// the forward pass still multiplies its gate by the initial 0, and the backward pass starts from a plain 0,
// as the reference's loops do (src/scanscam_cpu.hpp:17-27, 64-77).
//
// Everything is written in scan order: position sigma = e forwards, N-1-e backwards (e = index into the
// flat array, N = rows * T, a multiple of VEC by the host's choice of rows). In both directions a row starts,
// in scan order, at sigma % T == 0. A workgroup owns W*U consecutive chunks of scan positions; wave to wave
// the (A, B, F) totals go through LDS; the scan value entering the workgroup's span -- the part of a row that
// lies before it, at most T-1 elements -- is recomputed by wave 0 from one extra, partly loaded chunk (the
// "halo"), so workgroups do not depend on each other.
#pragma once

#include "scan_kernels.hpp"

namespace scanscam {

struct FlatArgs {
    const void *a;  // gates                       [rows, T] dense
    const void *x;  // forward: b      backward: gh
    const void *h;  // forward: unused backward: saved forward output
    void *y0;       // forward: h      backward: gb
    void *y1;       // forward: unused backward: ga
    int64_t N;      // rows * T, a multiple of VEC
    int32_t T;      // VEC <= T <= 64 * VEC
};

// Inclusive scan of (A, B, F) over the lanes of a wave (ascending lane = later in scan order).
template <typename CT>
__device__ __forceinline__ void wave_scan_reset(CT &A, CT &B, int &F)
{
#define SCANSCAM_STEP3(CTRL, ROW_MASK)                                                   \
    {                                                                                    \
        const CT A1 = dpp_move<CTRL, ROW_MASK>(CT(1), A);                                \
        const CT B1 = dpp_move<CTRL, ROW_MASK>(CT(0), B);                                \
        const int F1 = __builtin_amdgcn_update_dpp(0, F, CTRL, ROW_MASK, 0xf, false);    \
        B = F ? B : fma_(A, B1, B);                                                      \
        A = A * A1;                                                                      \
        F = F | F1;                                                                      \
    }
    SCANSCAM_STEP3(0x111, 0xf)  // row_shr:1
    SCANSCAM_STEP3(0x112, 0xf)  // row_shr:2
    SCANSCAM_STEP3(0x114, 0xf)  // row_shr:4
    SCANSCAM_STEP3(0x118, 0xf)  // row_shr:8
    SCANSCAM_STEP3(0x142, 0xa)  // row_bcast:15 into rows 1 and 3
    SCANSCAM_STEP3(0x143, 0xc)  // row_bcast:31 into rows 2 and 3
#undef SCANSCAM_STEP3
}

// One wave's U consecutive chunks of the flat stream.
template <typename ST, int VEC, int U, bool REV>
struct FlatTile {
    using V = Vec<ST, VEC>;
    using raw_t = typename V::raw_t;
    using CT = typename ComputeOf<ST>::type;

    int64_t elem[U];    // index of the vector's first element in the flat array (0 for a lane without a vector)
    bool valid[U];
    uint32_t reset[U];  // bit k: scan position k of the vector enters a new row
    uint32_t tzero[REV ? U : 1];  // backward: bit k: scan position k is time step 0 of its row (h[t-1] = 0)
    raw_t ra[U], rx[U], rh[REV ? U : 1];
    CT edge_a[REV ? 1 : 1], edge_h[REV ? 1 : 1];  // backward: a[] just above / h[] just below the wave's span in memory
    CT g[U][VEC], v[U][VEC];
    CT PA[U], PB[U];
    int PF[U];

    // sigma0: scan position of the vector's first component (in scan order); r = sigma0 % T.
    __device__ __forceinline__ void place(int u, int64_t sigma0, int r, bool wanted, int64_t N, int T)
    {
        valid[u] = wanted && sigma0 >= 0 && sigma0 < N;
        const int64_t e = REV ? N - VEC - sigma0 : sigma0;
        elem[u] = valid[u] ? e : 0;
        const int k0 = r == 0 ? 0 : T - r;  // the one scan position of the vector (if below VEC) where a row starts
        reset[u] = (valid[u] && k0 < VEC) ? (1u << k0) : 0u;
        if (REV) {
            const int k1 = T - 1 - r;       // ... where a row's time step 0 sits
            tzero[u] = (valid[u] && k1 < VEC) ? (1u << k1) : 0u;
        }
    }

    // Issues every load of the wave's chunks (lanes without a vector read element 0 and are masked later).
    __device__ __forceinline__ void load(const FlatArgs &p, int lane)
    {
        const ST *a = static_cast<const ST *>(p.a);
        const ST *x = static_cast<const ST *>(p.x);
        const ST *h = static_cast<const ST *>(p.h);
#pragma unroll
        for (int u = 0; u < U; u++) {
            ra[u] = V::load(a + elem[u]);
            rx[u] = V::load(x + elem[u]);
            if (REV) rh[u] = V::load(h + elem[u]);
        }
        if (REV) {
            // Neighbours in memory that no lane of this wave holds: a[] right above the vector of lane 0 of
            // chunk 0, h[] right below the vector of lane 63 of the last chunk.
            edge_a[0] = CT(0);
            edge_h[0] = CT(0);
            if (valid[0] && lane == 0 && elem[0] + VEC < p.N) edge_a[0] = (CT)a[elem[0] + VEC];
            if (valid[U - 1] && lane == kWave - 1 && elem[U - 1] > 0) edge_h[0] = (CT)h[elem[U - 1] - 1];
        }
    }

    // (gate, value) per element of chunk u in scan order, reset bits, and backward h[t-1].
    __device__ __forceinline__ void build(int u, int lane, const CT (&first_a)[REV ? U : 1], const CT (&last_h)[REV ? U : 1],
                                          CT (&G)[VEC], CT (&X)[VEC], CT (&HP)[VEC]) const
    {
        CT fa[VEC], fx[VEC];
        V::unpack(ra[u], fa);
        V::unpack(rx[u], fx);
#pragma unroll
        for (int k = 0; k < VEC; k++) {  // lanes without a vector hold a = 0, x = 0
            fa[k] = valid[u] ? fa[k] : CT(0);
            fx[k] = valid[u] ? fx[k] : CT(0);
        }
        if (!REV) {
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                G[k] = valid[u] ? fa[k] : CT(1);
                X[k] = fx[k];
            }
        } else {
            CT fh[VEC];
            V::unpack(rh[u], fh);
#pragma unroll
            for (int k = 0; k < VEC; k++) fh[k] = valid[u] ? fh[k] : CT(0);
            // Scan position k <-> element VEC-1-k of the vector; gate = a[e+1], hp = h[e-1], taken from the
            // neighbouring lane (lane-1 holds the vector above in memory, lane+1 the one below), the
            // neighbouring chunk, or the edge loads.
            CT a_next = lane_prev(fa[0], CT(0));
            CT h_prev = lane_next(fh[VEC - 1], CT(0));
            CT border_a = edge_a[0], border_h = edge_h[0];
            if (u > 0) border_a = read_lane(first_a[u - 1], kWave - 1);
            if (u + 1 < U) border_h = read_lane(last_h[u + 1], 0);
            a_next = (lane == 0) ? border_a : a_next;
            h_prev = (lane == kWave - 1) ? border_h : h_prev;
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                const CT gk = (k == 0) ? a_next : fa[(VEC - k) % VEC];
                const bool starts = (reset[u] >> k) & 1u;  // time step T-1 of a row: nothing is carried into it
                G[k] = valid[u] ? (starts ? CT(0) : gk) : CT(1);
                X[k] = fx[VEC - 1 - k];
                const CT hk = (k == VEC - 1) ? h_prev : fh[(VEC - 2 - k) < 0 ? 0 : (VEC - 2 - k)];
                HP[k] = ((tzero[u] >> k) & 1u) ? CT(0) : hk;
            }
        }
    }

    __device__ __forceinline__ void reduce(int lane, CT (&hp)[REV ? U : 1][VEC])
    {
        CT first_a[REV ? U : 1], last_h[REV ? U : 1];
        if (REV) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                CT t[VEC];
                V::unpack(ra[u], t);
                first_a[u] = valid[u] ? t[0] : CT(0);
                V::unpack(rh[u], t);
                last_h[u] = valid[u] ? t[VEC - 1] : CT(0);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            CT G[VEC], X[VEC], HP[VEC];
            build(u, lane, first_a, last_h, G, X, HP);
            CT A = CT(1), B = CT(0);
            int F = 0;
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                g[u][k] = G[k];
                v[u][k] = X[k];
                if (REV) hp[u][k] = HP[k];
                const bool starts = (reset[u] >> k) & 1u;
                B = fma_(G[k], starts ? CT(0) : B, X[k]);
                A = starts ? CT(0) : A * G[k];
                F |= starts ? 1 : 0;
            }
            wave_scan_reset<CT>(A, B, F);
            PA[u] = A;
            PB[u] = B;
            PF[u] = F;
        }
    }

    // Map of the wave's U chunks in scan order.
    __device__ __forceinline__ void total(CT &WA, CT &WB, int &WF) const
    {
        WA = read_lane(PA[0], 63);
        WB = read_lane(PB[0], 63);
        WF = __builtin_amdgcn_readlane(PF[0], 63);
#pragma unroll
        for (int u = 1; u < U; u++) {
            const CT TA = read_lane(PA[u], 63), TB = read_lane(PB[u], 63);
            const int TF = __builtin_amdgcn_readlane(PF[u], 63);
            WB = TF ? TB : fma_(TA, WB, TB);
            WA = TA * WA;
            WF |= TF;
        }
    }

    __device__ __forceinline__ void apply(const FlatArgs &p, CT carry, const CT (&hp)[REV ? U : 1][VEC])
    {
        ST *y0 = static_cast<ST *>(p.y0);
        ST *y1 = static_cast<ST *>(p.y1);
#pragma unroll
        for (int u = 0; u < U; u++) {
            // Map of everything before this lane inside the chunk, applied to the value entering the chunk.
            const CT EA = lane_prev(PA[u], CT(1)), EB = lane_prev(PB[u], CT(0));
            const int EF = __builtin_amdgcn_update_dpp(0, PF[u], 0x138, 0xf, 0xf, false);  // wave_shr:1
            CT acc = EF ? EB : fma_(EA, carry, EB);
            CT out[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                const bool starts = (reset[u] >> k) & 1u;
                acc = fma_(g[u][k], starts ? CT(0) : acc, v[u][k]);
                out[k] = acc;
            }
            if (u + 1 < U) {
                const int TF = __builtin_amdgcn_readlane(PF[u], 63);
                const CT TA = read_lane(PA[u], 63), TB = read_lane(PB[u], 63);
                carry = TF ? TB : fma_(TA, carry, TB);
            }
            if (!REV) {
                if (valid[u]) V::store(y0 + elem[u], V::pack(out));
            } else {
                CT gb[VEC], ga[VEC];
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    gb[VEC - 1 - k] = out[k];
                    ga[VEC - 1 - k] = out[k] * hp[u][k];
                }
                if (valid[u]) {
                    V::store(y0 + elem[u], V::pack(gb));
                    V::store(y1 + elem[u], V::pack(ga));
                }
            }
        }
    }
};

template <typename ST, int VEC, int U, bool REV, int MAXT>
__global__ __launch_bounds__(MAXT) void scan_flat_kernel(const FlatArgs p)
{
    using CT = typename ComputeOf<ST>::type;
    __shared__ CT lds_A[kMaxWaves];
    __shared__ CT lds_B[kMaxWaves];
    __shared__ int lds_F[kMaxWaves];
    __shared__ CT lds_in;  // the scan value entering the workgroup's span

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int W = blockDim.x / kWave;
    const int T = p.T;
    constexpr int kChunk = kWave * VEC;  // elements per chunk

    // Backwards, scan position sigma is element N-1-sigma, so chunks counted from sigma = 0 would sit on
    // 1 KiB borders of memory only if N were a multiple of a chunk. The scan positions are therefore shifted
    // by `pad` (the first `pad` positions of the first chunk do not exist): every load and store instruction
    // of a wave then covers whole 128-byte lines in both directions (fp32 T = 65: 234 us -> 211 us backward).
    const int pad = REV ? (int)((kChunk - p.N % kChunk) % kChunk) : 0;
    const int64_t span0 = (int64_t)blockIdx.x * W * U * kChunk - pad;  // first scan position of the workgroup (may be < 0)
    // How far into a row the span starts; 64 rows' worth (at least a chunk) keeps the dividend positive.
    const int r_span = (int)((span0 + (int64_t)kWave * T) % T);
    // Offsets inside the workgroup's span fit 32 bits; so does their sum with r_span.
    FlatTile<ST, VEC, U, REV> w;
#pragma unroll
    for (int u = 0; u < U; u++) {
        const unsigned in_span = (unsigned)(((wave * U + u) * kWave + lane) * VEC);
        w.place(u, span0 + in_span, (int)(((unsigned)r_span + in_span) % (unsigned)T), true, p.N, T);
    }
    w.load(p, lane);

    // The halo: the chunk of scan positions right before the span, of which the last r_span elements belong to
    // the row the span starts in. Lanes whose vector holds none of them stay out; the row's start (a reset)
    // lies inside, so whatever precedes it does not matter.
    FlatTile<ST, VEC, 1, REV> halo;
    CT halo_hp[REV ? 1 : 1][VEC];
    const bool with_halo = wave == 0 && r_span != 0;
    if (with_halo) {
        const int back = (kWave - lane) * VEC;             // the lane's vector starts this far before the span
        const bool wanted = back - VEC < r_span;           // it reaches into the row
        // (r_span - back) mod T, kept non-negative: T >= VEC, so 64 rows' worth covers a chunk.
        const int r = (int)(((unsigned)r_span + (unsigned)kWave * (unsigned)T - (unsigned)back) % (unsigned)T);
        halo.place(0, span0 - back, r, wanted, p.N, T);
        halo.load(p, lane);
    }

    CT hp[REV ? U : 1][VEC];
    w.reduce(lane, hp);
    CT WA, WB;
    int WF;
    w.total(WA, WB, WF);
    if (lane == 0) {
        lds_A[wave] = WA;
        lds_B[wave] = WB;
        lds_F[wave] = WF;
    }
    if (wave == 0) {
        CT cin = CT(0);
        if (with_halo) {
            halo.reduce(lane, halo_hp);
            CT HA, HB;
            int HF;
            halo.total(HA, HB, HF);
            cin = HB;  // HF is set: the halo holds the row's start
        }
        if (lane == 0) lds_in = cin;
    }
    __syncthreads();

    CT carry = lds_in;
    for (int q = 0; q < wave; q++) carry = lds_F[q] ? lds_B[q] : fma_(lds_A[q], carry, lds_B[q]);
    w.apply(p, carry, hp);
}

}  // namespace scanscam

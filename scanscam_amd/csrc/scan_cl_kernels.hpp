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
// few workgroups to fill the GPU, time is also cut into tiles over workgroups
// (scan_cl_lookback_kernel), with a decoupled look-back chain that carries one
// affine pair per channel from tile to tile. When C is so small that a time
// step does not fill half a wave, a wave holds several consecutive time steps
// instead (scan_cl_packed_kernel) and scans across them with lane moves.
#pragma once

#include "scan_kernels.hpp"

namespace scanscam {

struct ClArgs {
    const void *a;  // gates                       [B, T, C]
    const void *x;  // forward: b      backward: gh
    const void *h;  // forward: unused backward: saved forward output
    void *y0;       // forward: h      backward: gb
    void *y1;       // forward: unused backward: ga
    int64_t sB[5];  // element stride from batch element to batch element, per tensor in the order above
    int32_t sT[5];  // element stride from time step to time step (C when dense)
    int64_t batch;
    int32_t T;
    int32_t C;
    int32_t segments;   // look-back kernel: tiles per (batch element, channel group)
    int32_t group;      // packed kernel: lanes per time step (power of two below 64)
    int32_t xcd_order;  // scan_cl_kernel, scan_cl_lookback_kernel: consecutive (batch element, channel group) pairs share an XCD
    int32_t cached_stores;  // outputs through the caches' normal policy instead of non-temporal (the host decides, see run_cl)
    uint64_t *ws;       // look-back kernel: ticket counters + published pairs
    int32_t spin_limit; // look-back kernel: polls before a wait gives up
};

// One workgroup's view of its channels: pointers offset to the batch element
// (the same in every lane, so they live in scalar registers, and so does every
// time-step offset added to them) and the lane's first channel `c`, the only
// per-lane part of an address: loads and stores then take the scalar-base form
// with one shared 32-bit lane offset instead of a 64-bit address pair in vector
// registers per access.
template <typename ST> struct ClLane {
    const ST *a, *x, *h;
    ST *y0, *y1;
    int pa, px, ph, py0, py1;  // elements from one time step to the next, per tensor
    unsigned c;                // byte offset of the lane's first channel (0 for a lane without channels)
    bool c_ok;
    bool cached;               // ClArgs::cached_stores (the same in every wave of the launch)
    // Element-aligned lanes (RAGGED): C need not be a multiple of the lane's VEC channels, so the last lane of
    // a time step may own fewer. It loads the window of VEC channels that ends with the time step instead
    // (`c` points there) and moves its components down by `shift` places; its stores go out per channel.
    int shift;

    // base + elems elements + the lane's channel offset. The lane part enters as a zero-extended 32-bit
    // byte count, the form the scalar-base addressing mode takes.
    static __device__ __forceinline__ const ST *at(const ST *base, int64_t elems, unsigned c)
    {
        return reinterpret_cast<const ST *>(reinterpret_cast<const char *>(base + elems) + c);
    }
    static __device__ __forceinline__ ST *at(ST *base, int64_t elems, unsigned c)
    {
        return reinterpret_cast<ST *>(reinterpret_cast<char *>(base + elems) + c);
    }
};

// Addressing for the kernels in which a wave's lanes are the channels of one time step: an access is
// (base, lane offset, step offset), where the base is a 64-bit address that is the same for the whole wave
// (batch element and first time step of the wave's span: scalar registers), the lane offset is the lane's
// channel in bytes (one vector register, shared by every access of the kernel) and the step offset is the
// time step's distance from the base in bytes (a scalar). Offsets are 32-bit: the host keeps
// (S + 2) * time stride * element size below 4 GiB for these kernels.
// Two forms. BUF: buffer instructions, which take exactly these three operands, so no 64-bit address is
// formed per lane and access. Otherwise global instructions on base + offsets. Measured on the same
// kernels in one run (cl_buffered() below holds the outcome): the forward passes run the same either way
// (within 2 %; bf16 [64, 2048, 1001], lanes of one 16-bit channel, 265 us against 310); the backward
// passes (five tensors, i.e. five resources of four scalar registers) are 2-10 % faster on global
// instructions when a workgroup walks all of T (bf16 [256, 4096, 64] 142 us against 157, [16, 4096, 1024]
// 147 against 160, fp32 [64, 2048, 1024] 453 against 463) except with one 16-bit channel per lane and 8
// steps per wave ([64, 2048, 1001] bf16: 463 us against 541); with time split over workgroups fp32 is 3-6 %
// faster on global instructions ([4, 16384, 1024] 261 us against 277) and 16-bit storage 30 % faster on
// buffer instructions ([8, 4096, 512] bf16 48 us against 69).
template <typename ST, int VEC, bool BUF> struct ClAccess;

template <typename ST, int VEC, int S, bool REV, bool SPLIT /* time split over workgroups */>
constexpr bool cl_buffered()
{
    if (!REV) return true;
    if (SPLIT) return sizeof(ST) == 2;
    return sizeof(ST) * VEC == 2 && S <= 8;
}

template <typename ST, int VEC> struct ClAccess<ST, VEC, true> {
    using raw_t = typename Vec<ST, VEC>::raw_t;
    static constexpr int kBytes = (int)sizeof(raw_t);
    using Base = __amdgpu_buffer_rsrc_t;
    static __device__ __forceinline__ Base base(const ST *p)
    {
        // No bounds: the offsets handed in are always inside the tensor.
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<ST *>(p), 0, -1, 0x00020000);
    }
    // aux 2 = non-temporal (streamed data), 0 = the caches' normal policy.
    template <int AUX> static __device__ __forceinline__ raw_t load(Base r, unsigned lane_off, unsigned step_off)
    {
        if constexpr (kBytes == 16) return __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, step_off, AUX);
        else if constexpr (kBytes == 8) return __builtin_amdgcn_raw_buffer_load_b64(r, lane_off, step_off, AUX);
        else if constexpr (kBytes == 4) return __builtin_amdgcn_raw_buffer_load_b32(r, lane_off, step_off, AUX);
        else return __builtin_amdgcn_raw_buffer_load_b16(r, lane_off, step_off, AUX);
    }
    static __device__ __forceinline__ void store_cached(raw_t v, Base r, unsigned lane_off, unsigned step_off)
    {
        if constexpr (kBytes == 16) __builtin_amdgcn_raw_buffer_store_b128(v, r, lane_off, step_off, 0);
        else if constexpr (kBytes == 8) __builtin_amdgcn_raw_buffer_store_b64(v, r, lane_off, step_off, 0);
        else if constexpr (kBytes == 4) __builtin_amdgcn_raw_buffer_store_b32(v, r, lane_off, step_off, 0);
        else __builtin_amdgcn_raw_buffer_store_b16(v, r, lane_off, step_off, 0);
    }
    static __device__ __forceinline__ void store(raw_t v, Base r, unsigned lane_off, unsigned step_off)
    {
        if constexpr (kBytes == 16) __builtin_amdgcn_raw_buffer_store_b128(v, r, lane_off, step_off, 2);
        else if constexpr (kBytes == 8) __builtin_amdgcn_raw_buffer_store_b64(v, r, lane_off, step_off, 2);
        else if constexpr (kBytes == 4) __builtin_amdgcn_raw_buffer_store_b32(v, r, lane_off, step_off, 2);
        else __builtin_amdgcn_raw_buffer_store_b16(v, r, lane_off, step_off, 2);
    }
};

template <typename ST, int VEC> struct ClAccess<ST, VEC, false> {
    using raw_t = typename Vec<ST, VEC>::raw_t;
    typedef raw_t raw_elem_aligned_t __attribute__((aligned(sizeof(ST))));
    using Base = char *;
    static __device__ __forceinline__ Base base(const ST *p) { return reinterpret_cast<char *>(const_cast<ST *>(p)); }
    template <int AUX> static __device__ __forceinline__ raw_t load(Base r, unsigned lane_off, unsigned step_off)
    {
        const raw_elem_aligned_t *q = reinterpret_cast<const raw_elem_aligned_t *>(r + step_off + lane_off);
        if (AUX == 2) return __builtin_nontemporal_load(q);
        return *q;
    }
    static __device__ __forceinline__ void store(raw_t v, Base r, unsigned lane_off, unsigned step_off)
    {
        __builtin_nontemporal_store(v, reinterpret_cast<raw_elem_aligned_t *>(r + step_off + lane_off));
    }
    // Through the caches' normal policy. Lanes on their natural alignment take the buffer form: were both forms
    // plain stores to one address under a run-time choice, the compiler would fold them into one and drop the hint.
    static __device__ __forceinline__ void store_cached(raw_t v, Base r, unsigned lane_off, unsigned step_off)
    {
        ClAccess<ST, VEC, true>::store_cached(v, ClAccess<ST, VEC, true>::base(reinterpret_cast<const ST *>(r)), lane_off, step_off);
    }
    static __device__ __forceinline__ void store_cached_elem_aligned(raw_t v, Base r, unsigned lane_off, unsigned step_off)
    {
        *reinterpret_cast<raw_elem_aligned_t *>(r + step_off + lane_off) = v;
    }
};

// One wave's S consecutive time steps of a tile, for the 64*VEC channels of the workgroup.
//   load_fold   issues all loads and folds the steps to one affine pair per channel
//   apply       replays the steps from the scan value entering them and stores the results
// With APPLY = false only load_fold is used, and its loads are left cacheable (the data is
// read again later).
// Components of a vector moved down by s places (those moved in from above are zero).
template <typename ST, int VEC>
__device__ __forceinline__ typename Vec<ST, VEC>::raw_t cl_shift_down(typename Vec<ST, VEC>::raw_t r, int s)
{
    if constexpr (sizeof(r) == 16) {
        return Vec<ST, VEC>::shift_components(r, -s);
    } else if constexpr (sizeof(r) == 8) {
        const uint64_t v = ((uint64_t)r.x | ((uint64_t)r.y << 32)) >> (s * (int)sizeof(ST) * 8);
        decltype(r) out;
        out.x = (uint32_t)v;
        out.y = (uint32_t)(v >> 32);
        return out;
    } else if constexpr (sizeof(r) == 4) {
        return r >> (s * (int)sizeof(ST) * 8);
    } else {
        return r;  // lanes of one element have nothing to move
    }
}

template <typename ST, int VEC, int S, bool REV, bool APPLY, typename CT, bool SPLIT = false, bool RAGGED = false>
struct ClSteps {
    using V = Vec<ST, VEC>;
    using raw_t = typename V::raw_t;
    // Element-aligned lanes take global instructions (buffer instructions want 4-byte alignment).
    using BV = ClAccess<ST, VEC, !RAGGED && cl_buffered<ST, VEC, S, REV, SPLIT>()>;
    using Base = typename BV::Base;

    CT g[S][VEC], v[S][VEC];
    raw_t rh[(REV && APPLY) ? S : 1];
    int tau0;   // scan position of the first step
    int limit;  // scan positions from here on do not exist
    int tb;     // time step the resources' bases point at: no access of this wave lies before it
    // issue() may run for the next span of steps while the folded one still awaits apply(): what it sets is kept
    // apart (n_*) until fold() takes it over. The raw gates and values need no second copy, fold() has used them up.
    raw_t n_rh[(REV && APPLY) ? S : 1];
    int n_tau0, n_limit, n_tb;

    // Byte distance of time step t from the base, for a tensor with `stride` elements per step.
    __device__ __forceinline__ unsigned step_off(int t, int stride) const
    {
        return (unsigned)(t - tb) * (unsigned)stride * (unsigned)sizeof(ST);
    }

    // Whether a step exists, and whether its shifted operands do, is the same for every lane of the
    // wave (tau0 and limit are wave-uniform): scalar conditions, scalar offsets. A lane without
    // channels (C no multiple of the workgroup's channels) computes on channel 0's data like any
    // other lane and only its stores are masked, so no per-lane mask is kept per step.
    raw_t ra[S], rx[S];  // what issue() brought; dead once fold() has run

    // Issues every load of the wave's S steps; nothing waits for them here.
    __device__ __forceinline__ void issue(const ClLane<ST> &ln, int T, int first_step, int limit_)
    {
        n_tau0 = first_step;
        n_limit = limit_;
        // Forwards the wave touches times tau0 ... tau0+S-1; backwards T-1-tau for the same tau, plus
        // a[t+1] and h[t-1]: nothing before T-1-(tau0+S-1)-1. Clamped into the tensor.
        const int lowest = REV ? T - 1 - (n_tau0 + S - 1) - 1 : n_tau0;
        n_tb = lowest < 0 ? 0 : (lowest > T - 1 ? T - 1 : lowest);
        const int tb = n_tb, tau0 = n_tau0, limit = n_limit;  // this function's own view (step_off below takes tb from here)
        auto step_off = [tb](int t, int stride) { return (unsigned)(t - tb) * (unsigned)stride * (unsigned)sizeof(ST); };
        const Base res_a = BV::base(ln.a + (int64_t)tb * ln.pa), res_x = BV::base(ln.x + (int64_t)tb * ln.px);
        const Base res_h = BV::base(ln.h + (int64_t)tb * ln.ph);
        // Every load is issued unconditionally (a step that does not exist reads the base): no
        // branch separates the loads, so all of a wave's S x streams loads are in flight before the
        // first one is waited for.
#pragma unroll
        for (int s = 0; s < S; s++) {
            const int tau = tau0 + s;
            const int t = REV ? T - 1 - tau : tau;
            const bool in = tau < limit;
            // The gate of step t is a[t] forwards and a[t+1] backwards (0 past the end); h[-1] = 0.
            const bool a_in = in && (!REV || t + 1 < T), h_in = in && t > 0;
            const unsigned off_x = in ? step_off(t, ln.px) : 0u;
            const unsigned off_a = a_in ? step_off(REV ? t + 1 : t, ln.pa) : 0u;
            if (APPLY) {
                ra[s] = BV::template load<2>(res_a, ln.c, off_a);
                rx[s] = BV::template load<2>(res_x, ln.c, off_x);
                if (REV) n_rh[s] = BV::template load<2>(res_h, ln.c, h_in ? step_off(t - 1, ln.ph) : 0u);
            } else {
                ra[s] = BV::template load<0>(res_a, ln.c, off_a);
                rx[s] = BV::template load<0>(res_x, ln.c, off_x);
            }
        }
    }

    // Folds the issued steps to one affine pair per channel (and keeps gate and value per step for apply()).
    __device__ __forceinline__ void fold(int T, CT (&A)[VEC], CT (&B)[VEC], int shift = 0)
    {
        tau0 = n_tau0;
        limit = n_limit;
        tb = n_tb;
        if (REV && APPLY) {
#pragma unroll
            for (int s = 0; s < S; s++) rh[s] = n_rh[s];
        }
        if (RAGGED && shift != 0) {  // the last lane of a time step: its window's components into place
#pragma unroll
            for (int s = 0; s < S; s++) {
                ra[s] = cl_shift_down<ST, VEC>(ra[s], shift);
                rx[s] = cl_shift_down<ST, VEC>(rx[s], shift);
                if (REV && APPLY) rh[s] = cl_shift_down<ST, VEC>(rh[s], shift);
            }
        }
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            A[k] = CT(1);
            B[k] = CT(0);
        }
#pragma unroll
        for (int s = 0; s < S; s++) {
            const int tau = tau0 + s;
            const int t = REV ? T - 1 - tau : tau;
            const bool in = tau < limit, a_in = in && (!REV || t + 1 < T);
            CT fa[VEC], fx[VEC];
            V::unpack(ra[s], fa);
            V::unpack(rx[s], fx);
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                g[s][k] = in ? (a_in ? fa[k] : CT(0)) : CT(1);
                v[s][k] = in ? fx[k] : CT(0);
                B[k] = fma_(g[s][k], B[k], v[s][k]);
                A[k] = A[k] * g[s][k];
            }
        }
    }

    __device__ __forceinline__ void load_fold(const ClLane<ST> &ln, int T, int first_step, int limit_,
                                              CT (&A)[VEC], CT (&B)[VEC])
    {
        issue(ln, T, first_step, limit_);
        fold(T, A, B, ln.shift);
    }

    // A lane's vector to its channels of one time step; the last lane of an element-aligned time step stores
    // the channels it owns one by one (its window started `shift` channels early).
    // CACHED: through the caches' normal policy instead of non-temporal. Lanes of 8 bytes or less only:
    // element-aligned ones always (their time steps are never whole lines), the others where the host asks for it.
    template <bool CACHED>
    static __device__ __forceinline__ void put(raw_t r, Base res, const ClLane<ST> &ln, unsigned off)
    {
        if (!RAGGED || ln.shift == 0) {
            if constexpr (RAGGED && sizeof(raw_t) <= 8) BV::store_cached_elem_aligned(r, res, ln.c, off);
            else if constexpr (CACHED) BV::store_cached(r, res, ln.c, off);
            else BV::store(r, res, ln.c, off);
        } else if constexpr (RAGGED) {
            using One = ClAccess<ST, 1, false>;
            const Elems<ST, VEC> e = __builtin_bit_cast(Elems<ST, VEC>, r);
#pragma unroll
            for (int k = 0; k < VEC; k++)
                if (k < VEC - ln.shift) {
                    if constexpr (sizeof(raw_t) <= 8)
                        One::store_cached_elem_aligned(__builtin_bit_cast(typename One::raw_t, e.e[k]), res, ln.c + (unsigned)((ln.shift + k) * sizeof(ST)), off);
                    else
                        One::store(__builtin_bit_cast(typename One::raw_t, e.e[k]), res, ln.c + (unsigned)((ln.shift + k) * sizeof(ST)), off);
                }
        }
    }

    // One copy of the store loop per policy, chosen once per call (the choice is the same for the whole launch).
    __device__ __forceinline__ void apply(const ClLane<ST> &ln, int T, CT (&mine)[VEC])
    {
        if constexpr (!RAGGED && sizeof(raw_t) <= 8) {
            if (ln.cached) {
                apply_as<true>(ln, T, mine);
                return;
            }
        }
        apply_as<false>(ln, T, mine);
    }

    template <bool CACHED> __device__ __forceinline__ void apply_as(const ClLane<ST> &ln, int T, CT (&mine)[VEC])
    {
        const Base res_y0 = BV::base(ln.y0 + (int64_t)tb * ln.py0), res_y1 = BV::base(ln.y1 + (int64_t)tb * ln.py1);
#pragma unroll
        for (int s = 0; s < S; s++) {
            const int tau = tau0 + s;
            const int t = REV ? T - 1 - tau : tau;
            const bool in = tau < limit, h_in = in && t > 0;
            CT out[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                mine[k] = fma_(g[s][k], mine[k], v[s][k]);
                out[k] = mine[k];
            }
            if (!REV) {
                if (in && ln.c_ok) put<CACHED>(V::pack(out), res_y0, ln, step_off(t, ln.py0));
            } else {
                CT fh[VEC], ga[VEC];
                V::unpack(rh[s], fh);
#pragma unroll
                for (int k = 0; k < VEC; k++) ga[k] = out[k] * (h_in ? fh[k] : CT(0));
                if (in && ln.c_ok) {
                    put<CACHED>(V::pack(out), res_y0, ln, step_off(t, ln.py0));
                    put<CACHED>(V::pack(ga), res_y1, ln, step_off(t, ln.py1));
                }
            }
        }
    }
};

// Index r of n, dealt round-robin to the 8 XCDs (r % 8), mapped so that every XCD holds one contiguous run
// of the n indices: a permutation of 0 ... n-1.
__device__ __forceinline__ int xcd_contiguous(int r, int n)
{
    const int per = (n + 7) / 8, rem = n % 8 == 0 ? 8 : n % 8;
    const int xcd = r % 8, slot = r / 8;
    return xcd < rem ? xcd * per + slot : rem * per + (xcd - rem) * (per - 1) + slot;
}

template <typename ST, int VEC, bool RAGGED = false>
__device__ __forceinline__ ClLane<ST> cl_lane(const ClArgs &p, int64_t batch_index, int group, int lane)
{
    const int64_t c0 = ((int64_t)group * kWave + lane) * VEC;  // first channel of this lane
    ClLane<ST> ln;
    ln.cached = p.cached_stores != 0;
    ln.c_ok = c0 < p.C;
    ln.shift = (RAGGED && ln.c_ok && c0 + VEC > p.C) ? (int)(c0 + VEC - p.C) : 0;  // C >= VEC: the host checks it
    ln.c = ln.c_ok ? (unsigned)((c0 - ln.shift) * sizeof(ST)) : 0u;
    ln.a = static_cast<const ST *>(p.a) + batch_index * p.sB[0];
    ln.x = static_cast<const ST *>(p.x) + batch_index * p.sB[1];
    ln.h = static_cast<const ST *>(p.h) + batch_index * p.sB[2];
    ln.y0 = static_cast<ST *>(p.y0) + batch_index * p.sB[3];
    ln.y1 = static_cast<ST *>(p.y1) + batch_index * p.sB[4];
    ln.pa = p.sT[0];
    ln.px = p.sT[1];
    ln.ph = p.sT[2];
    ln.py0 = p.sT[3];
    ln.py1 = p.sT[4];
    return ln;
}

// Dynamic LDS: two buffers (tiles alternate) of A and B, each [W][VEC][64] values.
template <typename ST, int VEC, int S, bool REV, int MAXT, bool RAGGED = false>
__global__ __launch_bounds__(MAXT) void scan_cl_kernel(const ClArgs p)
{
    using CT = typename ComputeOf<ST>::type;
    extern __shared__ double lds_raw[];  // 8-byte aligned for either arithmetic type
    CT *lds = reinterpret_cast<CT *>(lds_raw);

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // wave-uniform: kept in a scalar register
    const int W = blockDim.x / kWave;
    const int groups = (p.C + kWave * VEC - 1) / (kWave * VEC);  // channel groups per batch element
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2. When a time step of C
    // channels is not a whole number of 128-byte lines, neighbouring channel groups share a line at
    // every time step; handled by different XCDs that line is fetched twice and written in two parts.
    // xcd_order gives each XCD a contiguous run of (batch element, channel group) pairs instead, so that
    // neighbours meet in one L2.
    const int bid = p.xcd_order ? xcd_contiguous((int)blockIdx.x, (int)gridDim.x) : (int)blockIdx.x;
    const ClLane<ST> ln = cl_lane<ST, VEC, RAGGED>(p, bid / groups, bid % groups, lane);

    const int tile_steps = W * S;
    const int ntiles = (p.T + tile_steps - 1) / tile_steps;
    const int plane = W * VEC * kWave;  // values per LDS array
    CT carry[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) carry[k] = CT(0);

    // AHEAD: the loads of tile it + 1 are issued as soon as tile it is folded, so that they are in flight while the
    // waves exchange their pairs, wait at the barrier, and compute and store tile it. Both tiles' registers are live
    // then (the next one's packed gates and values beside this one's unpacked ones): taken for 16-bit storage in
    // lanes of up to 8 bytes, where the packed half is small and the kernels wait most -- bf16 [64, 2048, 1024]
    // 151 / 228 -> 129 / 220 us, [32, 2048, 2048] 148 / 231 -> 131 / 222 us, [256, 1024, 1024] backward 447 -> 424 us,
    // [8, 4096, 2048] forward 93 -> 90 us. fp32 pays 30 to 120 registers for it and is level on average (+28 % to -10 %),
    // 16-byte lanes of 16-bit storage spill.
    constexpr bool AHEAD = sizeof(ST) == 2 && VEC <= 4 && VEC * S <= 32;
    ClSteps<ST, VEC, S, REV, true, CT, false, RAGGED> steps;
    if (AHEAD) steps.issue(ln, p.T, wave * S, p.T);
    for (int it = 0; it < ntiles; it++) {
        CT *lds_A = lds + (it & 1) * 2 * plane, *lds_B = lds_A + plane;
        CT A[VEC], B[VEC], mine[VEC];
        if (!AHEAD) steps.issue(ln, p.T, it * tile_steps + wave * S, p.T);
        steps.fold(p.T, A, B, ln.shift);
        if (AHEAD && it + 1 < ntiles) steps.issue(ln, p.T, (it + 1) * tile_steps + wave * S, p.T);
#pragma unroll
        for (int k = 0; k < VEC; k++) mine[k] = carry[k];
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
                    if (q == wave) mine[k] = carry[k];
                    carry[k] = fma_(Aq, carry[k], Bq);
                }
            }
        } else {
#pragma unroll
            for (int k = 0; k < VEC; k++) carry[k] = fma_(A[k], carry[k], B[k]);
        }
        steps.apply(ln, p.T, mine);
    }
}

// ---------------------------------------------------------------------------
// Few channels (C <= 32*VEC): a time step fills only G = pow2 >= C/VEC lanes, so
// a wave holds 64/G consecutive time steps per instruction: lane = (step in the
// instruction, channel vector), and every load and store instruction still
// covers one contiguous span (64/G steps of C channels). The recurrence along
// time is then a scan ACROSS lanes at stride G (a lane never folds in time by
// itself: its S instructions are 64/G steps apart). Per instruction: an
// inclusive scan of the affine pairs over the lanes of one channel vector (DPP
// moves inside each row of 16 lanes, two shuffles across rows); instruction to
// instruction the
// total (held by the last step's lanes) is composed onto a running pair; wave
// to wave through LDS, tile to tile in registers, as in scan_cl_kernel. Every
// element's output is then one FMA: inclusive pair applied to the value entering
// the wave. A workgroup owns one batch element.
// LDS: two buffers (tiles alternate) of A and B, each [W][VEC][G] values.
// ---------------------------------------------------------------------------
// Inclusive scan of affine pairs over the lanes that hold one channel vector: lanes cl, cl + G, cl + 2G, ... of a
// wave (G a power of two below 64; ascending lane = later in scan order). DPP moves inside each row of 16 lanes
// at distances G ... 8 (lanes without a source in their row receive the identity), then two shuffles across
// rows: rows 1 and 3 take the total of the row before (held by its last lanes of the same channel vector), then
// rows 2 and 3 the total of rows 0-1.
template <typename CT>
__device__ __forceinline__ void packed_lane_scan(CT &A, CT &B, int G, int cl, int lane)
{
#define SCANSCAM_ROW_STEP(OFF)                                  \
    if (G <= (OFF)) {                                           \
        const CT A1 = dpp_move<0x110 + (OFF), 0xf>(CT(1), A);   \
        const CT B1 = dpp_move<0x110 + (OFF), 0xf>(CT(0), B);   \
        B = fma_(A, B1, B);                                     \
        A = A * A1;                                             \
    }
    SCANSCAM_ROW_STEP(1)
    SCANSCAM_ROW_STEP(2)
    SCANSCAM_ROW_STEP(4)
    SCANSCAM_ROW_STEP(8)
#undef SCANSCAM_ROW_STEP
    if (G <= 16) {
        const int src = ((lane & ~15) - G + cl) & (kWave - 1);  // rows 0 and 2 discard what they read
        const CT A1 = __shfl(A, src, kWave), B1 = __shfl(B, src, kWave);
        if (lane & 16) {
            B = fma_(A, B1, B);
            A = A * A1;
        }
    }
    {
        const int src = 32 - G + cl;
        const CT A1 = __shfl(A, src, kWave), B1 = __shfl(B, src, kWave);
        if (lane & 32) {
            B = fma_(A, B1, B);
            A = A * A1;
        }
    }
}

template <typename ST, int VEC, int S, bool REV, int MAXT>
__global__ __launch_bounds__(MAXT) void scan_cl_packed_kernel(const ClArgs p)
{
    using CT = typename ComputeOf<ST>::type;
    using V = Vec<ST, VEC>;
    using raw_t = typename V::raw_t;
    extern __shared__ double lds_raw[];
    CT *lds = reinterpret_cast<CT *>(lds_raw);

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int W = blockDim.x / kWave;
    const int G = p.group;
    const int subs = kWave / G;       // time steps per instruction
    const int cl = lane & (G - 1);    // channel vector of this lane
    const int sub = lane / G;         // its step inside the instruction
    const ClLane<ST> ln = cl_lane<ST, VEC>(p, blockIdx.x, 0, cl);

    const int wave_steps = S * subs;
    const int tile_steps = W * wave_steps;
    const int ntiles = (p.T + tile_steps - 1) / tile_steps;
    const int plane = W * VEC * G;
    CT carry[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) carry[k] = CT(0);

    for (int it = 0; it < ntiles; it++) {
        CT *lds_A = lds + (it & 1) * 2 * plane, *lds_B = lds_A + plane;
        // All loads first, unconditionally (masked lanes read offset 0 of their own column).
        raw_t ra[S], rx[S], rh[REV ? S : 1];
        bool ok[S], a_ok[S], h_ok[S];
        int tt[S];
#pragma unroll
        for (int s = 0; s < S; s++) {
            const int tau = it * tile_steps + (wave * S + s) * subs + sub;  // scan position
            const int t = REV ? p.T - 1 - tau : tau;
            tt[s] = t;
            ok[s] = ln.c_ok && tau < p.T;
            a_ok[s] = ok[s] && (!REV || t + 1 < p.T);  // backward gate a[t+1], 0 past the end
            h_ok[s] = ok[s] && t > 0;                   // h[-1] = 0
            ra[s] = V::load(ln.at(ln.a, a_ok[s] ? (int64_t)(REV ? t + 1 : t) * ln.pa : 0, ln.c));
            rx[s] = V::load(ln.at(ln.x, ok[s] ? (int64_t)t * ln.px : 0, ln.c));
            if (REV) rh[s] = V::load(ln.at(ln.h, h_ok[s] ? (int64_t)(t - 1) * ln.ph : 0, ln.c));
        }
        // PA/PB: the pair of everything in this wave's span up to and including the lane's step of
        // instruction s; (RA, RB): instructions 0..s-1 composed (the same in every lane of a channel).
        CT PA[S][VEC], PB[S][VEC], RA[VEC], RB[VEC];
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            RA[k] = CT(1);
            RB[k] = CT(0);
        }
#pragma unroll
        for (int s = 0; s < S; s++) {
            CT fa[VEC], fx[VEC];
            V::unpack(ra[s], fa);
            V::unpack(rx[s], fx);
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                CT A = ok[s] ? (a_ok[s] ? fa[k] : CT(0)) : CT(1);
                CT B = ok[s] ? fx[k] : CT(0);
                // Two ways to the same inclusive scan over the steps of one instruction. Measured, the backward
                // pass with one channel per lane is 15 % faster on plain shuffles at distances G, 2G, ... 32;
                // everything else 8-20 % faster with the ladder below.
                if (REV && VEC == 1) {
                    for (int off = G; off < kWave; off <<= 1) {
                        const CT A1 = __shfl_up(A, off, kWave), B1 = __shfl_up(B, off, kWave);
                        if (lane >= off) {
                            B = fma_(A, B1, B);
                            A = A * A1;
                        }
                    }
                } else {
                    packed_lane_scan<CT>(A, B, G, cl, lane);
                }
                const CT TA = __shfl(A, kWave - G + cl, kWave), TB = __shfl(B, kWave - G + cl, kWave);
                PB[s][k] = fma_(A, RB[k], B);
                PA[s][k] = A * RA[k];
                RB[k] = fma_(TA, RB[k], TB);
                RA[k] = TA * RA[k];
            }
        }
        CT mine[VEC];
#pragma unroll
        for (int k = 0; k < VEC; k++) mine[k] = carry[k];
        if (W > 1) {
            if (sub == 0) {
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    lds_A[(wave * VEC + k) * G + cl] = RA[k];
                    lds_B[(wave * VEC + k) * G + cl] = RB[k];
                }
            }
            __syncthreads();
            for (int q = 0; q < W; q++) {
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    const CT Aq = lds_A[(q * VEC + k) * G + cl], Bq = lds_B[(q * VEC + k) * G + cl];
                    if (q == wave) mine[k] = carry[k];
                    carry[k] = fma_(Aq, carry[k], Bq);
                }
            }
        } else {
#pragma unroll
            for (int k = 0; k < VEC; k++) carry[k] = fma_(RA[k], carry[k], RB[k]);
        }
#pragma unroll
        for (int s = 0; s < S; s++) {
            CT out[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) out[k] = fma_(PA[s][k], mine[k], PB[s][k]);
            if (!REV) {
                if (ok[s]) V::store(ln.at(ln.y0, (int64_t)tt[s] * ln.py0, ln.c), V::pack(out));
            } else {
                CT fh[VEC], ga[VEC];
                V::unpack(rh[s], fh);
#pragma unroll
                for (int k = 0; k < VEC; k++) ga[k] = out[k] * (h_ok[s] ? fh[k] : CT(0));
                if (ok[s]) {
                    V::store(ln.at(ln.y0, (int64_t)tt[s] * ln.py0, ln.c), V::pack(out));
                    V::store(ln.at(ln.y1, (int64_t)tt[s] * ln.py1, ln.c), V::pack(ga));
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Time split over workgroups in ONE pass: decoupled look-back with one affine
// pair per channel. A tile is W*S time steps of the workgroup's 64*VEC channels;
// tiles of a row-group (batch element x channel group) are taken by ticket. W
// consecutive tiles form a super-tile. The protocol is the two-level one of
// scan_lookback_kernel with the roles of lanes and waves exchanged, because here
// a lane is a channel: WAVE w of the workgroup fetches tile w of the current
// super-tile (w < j) and super-tile m-1-w into LDS, polling until all 64 lanes
// see them; then every lane folds, for its own channels and in a fixed order,
//   S_m     from the nearest super-tile with a published end value SI and the
//           aggregates (SA, SB) of the super-tiles after it,
//   carry   from S_m through the aggregates of tiles 0..j-1.
// The last tile of a super-tile publishes (SA, SB) as soon as it holds all W
// tile aggregates, and SI = fma(SA, S_m, SB) once S_m is known.
//
// Workspace, in 64-bit words: ticket counter of row-group r at word
// r * kCounterStride, word 1 raised on a timed-out wait; then per (row-group,
// tile) its [VEC][64] published pairs; then per (row-group, super-tile) its
// [VEC][64] pairs (SA, SB) and its [VEC][64] end values SI (encodings: Desc).
// LDS: [W][7][VEC][64] values (per wave slot: wave pairs A, B; tile aggregates A, B;
// super-tile SI, SA, SB).
// ---------------------------------------------------------------------------
template <typename CT, int VEC>
__device__ __forceinline__ bool cl_fetch(const uint64_t *src, int lane, CT (&out)[VEC])
{
    using D = Desc<CT>;
    bool ready = true;
#pragma unroll
    for (int k = 0; k < VEC; k++) ready = D::load(src + (k * kWave + lane) * D::W, out[k]) && ready;
    return __ballot(ready) == ~0ull;  // all 64 lanes: the decision is the same for the whole wave
}

template <typename CT, int VEC>
__device__ __forceinline__ void cl_publish(uint64_t *dst, int lane, const CT (&val)[VEC])
{
    using D = Desc<CT>;
#pragma unroll
    for (int k = 0; k < VEC; k++) D::store(dst + (k * kWave + lane) * D::W, val[k]);
}

// The same for an affine pair per channel: [VEC][64] pairs (fp32: one word per pair, one load per poll).
template <typename CT, int VEC>
__device__ __forceinline__ bool cl_fetch_pair(const uint64_t *src, int lane, CT (&a)[VEC], CT (&b)[VEC])
{
    using D = Desc<CT>;
    bool ready = true;
#pragma unroll
    for (int k = 0; k < VEC; k++) ready = D::load_pair(src + (k * kWave + lane) * D::PAIR, a[k], b[k]) && ready;
    return __ballot(ready) == ~0ull;
}

template <typename CT, int VEC>
__device__ __forceinline__ void cl_publish_pair(uint64_t *dst, int lane, const CT (&a)[VEC], const CT (&b)[VEC])
{
    using D = Desc<CT>;
#pragma unroll
    for (int k = 0; k < VEC; k++) D::store_pair(dst + (k * kWave + lane) * D::PAIR, a[k], b[k]);
}

template <typename ST, int VEC, int S, bool REV, int MAXT>
__global__ __launch_bounds__(MAXT) void scan_cl_lookback_kernel(const ClArgs p)
{
    using CT = typename ComputeOf<ST>::type;
    using D = Desc<CT>;
    extern __shared__ double lds_raw[];
    CT *lds = reinterpret_cast<CT *>(lds_raw);
    __shared__ unsigned lds_ticket;
    __shared__ int lds_flags[2][kMaxWaves];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // wave-uniform: kept in a scalar register
    const int W = blockDim.x / kWave;
    const int groups = (p.C + kWave * VEC - 1) / (kWave * VEC);
    const int64_t rowgroups = p.batch * groups;
    const int tpr = p.segments;              // tiles per row-group
    const int spr = (tpr + W - 1) / W;       // super-tiles per row-group
    // LDS: per wave slot w, seven [VEC][64] arrays one after the other, so that an access is the slot's
    // base plus the lane (one register) and a constant.
    enum { exA, exB,   // pairs of this tile's waves
           tA, tB,     // aggregates of tiles 0..j-1 of the super-tile
           sI, sA, sB  // super-tiles m-1, m-2, ...
    };
    constexpr int kVals = VEC * kWave * D::W;      // words of one [VEC][64] array of published values
    constexpr int kPairs = VEC * kWave * D::PAIR;  // ... of published pairs
    constexpr int kSup = kPairs + kVals;           // a super-tile: its pair (SA, SB), then its end value SI
#define AT(arr, w, k) lds[((w) * 7 + (arr)) * (VEC * kWave) + (k) * kWave + lane]

    // Row-groups of a workgroup's XCD: with p.xcd_order (time steps that are not whole 128-byte lines) a
    // contiguous run of them, so that channel groups that share a line meet in one L2 (as in scan_cl_kernel;
    // exact when the number of row-groups is a multiple of 8, where a row-group keeps its XCD over all tiles).
    // (xcd_order 2, any number of row-groups: XCD x = blockIdx % 8 owns the x-th run of them, of n / 8 rounded up or
    // down, and its workgroups go round that run; the host pads the grid to 8 shares of the longer run's size, so the
    // last workgroups of a shorter run's XCD have nothing to do.)
    int64_t rg;
    if (p.xcd_order == 2) {
        const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
        const int per = (int)((rowgroups + 7) / 8), rem = rowgroups % 8 == 0 ? 8 : (int)(rowgroups % 8);
        const int mine = xcd < rem ? per : per - 1;
        if (slot >= mine * tpr) return;
        rg = (xcd < rem ? xcd * per : rem * per + (xcd - rem) * (per - 1)) + slot % mine;
    } else {
        const int64_t rg0 = blockIdx.x % rowgroups;
        rg = (p.xcd_order && rowgroups % 8 == 0) ? xcd_contiguous((int)rg0, (int)rowgroups) : rg0;
    }
    if (threadIdx.x == 0)
        lds_ticket = __hip_atomic_fetch_add(reinterpret_cast<unsigned *>(p.ws + rg * kCounterStride), 1u,
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const int tile = (int)__builtin_amdgcn_readfirstlane((int)lds_ticket);
    const ClLane<ST> ln = cl_lane<ST, VEC>(p, rg / groups, (int)(rg % groups), lane);
    uint64_t *tiles = p.ws + rowgroups * kCounterStride + rg * (int64_t)tpr * kPairs;
    uint64_t *supers = p.ws + rowgroups * kCounterStride + rowgroups * (int64_t)tpr * kPairs +
                       rg * (int64_t)spr * kSup;
    const int j = tile % W, m = tile / W;

    ClSteps<ST, VEC, S, REV, true, CT, true> cur;
    CT A[VEC], B[VEC];
    cur.load_fold(ln, p.T, tile * W * S + wave * S, p.T, A, B);
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        AT(exA, wave, k) = A[k];
        AT(exB, wave, k) = B[k];
    }
    __syncthreads();

    // The tile's own aggregate (every wave computes it for its lanes).
    CT TA[VEC], TB[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        TA[k] = CT(1);
        TB[k] = CT(0);
    }
    for (int q = 0; q < W; q++) {
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            TB[k] = fma_(AT(exA, q, k), TB[k], AT(exB, q, k));
            TA[k] = AT(exA, q, k) * TA[k];
        }
    }
    CT carry[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) carry[k] = CT(0);

    if (tpr > 1) {
        const bool closes = (j == W - 1) && (m + 1 < spr);
        if (wave == 0 && j < W - 1 && tile + 1 < tpr) cl_publish_pair<CT, VEC>(tiles + (int64_t)tile * kPairs, lane, TA, TB);
        // Wave w is responsible for tile w of this super-tile (if w < j) and for super-tile m-1-w.
        bool have_t = wave >= j;
        const int sidx = m - 1 - wave;
        bool have_si = sidx < 0, have_sa = sidx < 0;
        if (sidx < 0) {  // before the row-group starts: value 0, identity aggregate
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                AT(sI, wave, k) = CT(0);
                AT(sA, wave, k) = CT(1);
                AT(sB, wave, k) = CT(0);
            }
        }
        bool tiles_done = false, supers_done = false, super_published = false;
        int first = 0;
        for (int spin = 0; spin < p.spin_limit; spin++) {
            CT val[VEC], val2[VEC];
            if (!have_t) {
                if (cl_fetch_pair<CT, VEC>(tiles + (int64_t)(m * W + wave) * kPairs, lane, val, val2)) {
                    have_t = true;
#pragma unroll
                    for (int k = 0; k < VEC; k++) {
                        AT(tA, wave, k) = val[k];
                        AT(tB, wave, k) = val2[k];
                    }
                }
            }
            if (!have_si) {
                if (cl_fetch<CT, VEC>(supers + (int64_t)sidx * kSup + kPairs, lane, val)) {
                    have_si = true;
#pragma unroll
                    for (int k = 0; k < VEC; k++) AT(sI, wave, k) = val[k];
                }
            }
            if (!have_sa) {
                if (cl_fetch_pair<CT, VEC>(supers + (int64_t)sidx * kSup, lane, val, val2)) {
                    have_sa = true;
#pragma unroll
                    for (int k = 0; k < VEC; k++) {
                        AT(sA, wave, k) = val[k];
                        AT(sB, wave, k) = val2[k];
                    }
                }
            }
            if (lane == 0) lds_flags[spin & 1][wave] = (have_t ? 1 : 0) | (have_si ? 2 : 0) | (have_sa ? 4 : 0);
            __syncthreads();
            // The same decision in every thread of the workgroup.
            tiles_done = true;
            supers_done = false;
            bool chain_ok = true;
            for (int w = 0; w < W; w++) {
                const int f = lds_flags[spin & 1][w];
                tiles_done = tiles_done && (f & 1);
                if (!supers_done && chain_ok) {
                    if (f & 2) {
                        supers_done = true;
                        first = w;
                    } else if (!(f & 4)) {
                        chain_ok = false;
                    }
                }
            }
            if (tiles_done && closes && !super_published) {
                // (SA, SB): the W tile aggregates composed in order, this tile's last.
                super_published = true;
                if (wave == 0) {
                    CT SA[VEC], SB[VEC];
#pragma unroll
                    for (int k = 0; k < VEC; k++) {
                        SA[k] = CT(1);
                        SB[k] = CT(0);
                    }
                    for (int w = 0; w < W - 1; w++) {
#pragma unroll
                        for (int k = 0; k < VEC; k++) {
                            SB[k] = fma_(AT(tA, w, k), SB[k], AT(tB, w, k));
                            SA[k] = AT(tA, w, k) * SA[k];
                        }
                    }
#pragma unroll
                    for (int k = 0; k < VEC; k++) {
                        SB[k] = fma_(TA[k], SB[k], TB[k]);
                        SA[k] = TA[k] * SA[k];
                    }
                    cl_publish_pair<CT, VEC>(supers + (int64_t)m * kSup, lane, SA, SB);
                }
            }
            if (tiles_done && supers_done) break;
            __builtin_amdgcn_s_sleep(1);
        }
        // S_m, then the carry into this tile, for this lane's channels.
#pragma unroll
        for (int k = 0; k < VEC; k++) carry[k] = AT(sI, first, k);
        for (int q = first - 1; q >= 0; q--) {
#pragma unroll
            for (int k = 0; k < VEC; k++) carry[k] = fma_(AT(sA, q, k), carry[k], AT(sB, q, k));
        }
        if (!(tiles_done && supers_done)) {
            if (threadIdx.x == 0)
                __hip_atomic_store(p.ws + kTimeoutWord, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int k = 0; k < VEC; k++) carry[k] = CT(__builtin_nanf(""));
        }
        CT S_m[VEC];
#pragma unroll
        for (int k = 0; k < VEC; k++) S_m[k] = carry[k];
        for (int w = 0; w < j; w++) {
#pragma unroll
            for (int k = 0; k < VEC; k++) carry[k] = fma_(AT(tA, w, k), carry[k], AT(tB, w, k));
        }
        if (closes && wave == 0) {
            // SI = fma(SA, S_m, SB) with (SA, SB) recomposed exactly as published above.
            CT SA[VEC], SB[VEC], SI[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                SA[k] = CT(1);
                SB[k] = CT(0);
            }
            for (int w = 0; w < W - 1; w++) {
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    SB[k] = fma_(AT(tA, w, k), SB[k], AT(tB, w, k));
                    SA[k] = AT(tA, w, k) * SA[k];
                }
            }
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                SB[k] = fma_(TA[k], SB[k], TB[k]);
                SA[k] = TA[k] * SA[k];
                SI[k] = fma_(SA[k], S_m[k], SB[k]);
            }
            cl_publish<CT, VEC>(supers + (int64_t)m * kSup + kPairs, lane, SI);
        }
    }

    // Carry into this wave's steps: through the pairs of the waves before it.
    for (int q = 0; q < wave; q++) {
#pragma unroll
        for (int k = 0; k < VEC; k++) carry[k] = fma_(AT(exA, q, k), carry[k], AT(exB, q, k));
    }
    cur.apply(ln, p.T, carry);
#undef AT
}

}  // namespace scanscam

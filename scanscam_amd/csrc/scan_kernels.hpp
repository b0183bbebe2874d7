// First-order gated linear scan for gfx950 (MI355X): device code.
//
//   forward   h[t]  = a[t] * h[t-1] + b[t],            h[-1] = 0
//   backward  gb[t] = gh[t] + a[t+1] * gb[t+1],        gb[T] = 0
//             ga[t] = gb[t] * h[t-1],                  h[-1] = 0
//
// (the arithmetic of the reference's CPU loops, src/scanscam_cpu.hpp:17-27 and
// :64-77, which its CUDA kernels src/scanscam_cuda.cu:144-258, 366-425 also
// compute). Both directions are the same scan over affine maps h -> A*h + B,
// composed as (A2, B2) o (A1, B1) = (A2*A1, A2*B1 + B2); the backward pass is
// that scan run over reversed time with gate a[t+1] and value gh[t].
//
// Data layout: every tensor is a dense row-major [rows, T] array, scanned along
// T. A lane owns one 16-byte vector (VEC elements) of a 64-lane "chunk"
// (64*VEC consecutive elements of one row), so every load and store
// instruction of a wave covers one contiguous 1 KiB span. For the backward
// pass lane l owns vector 63-l of the chunk and reads its components in
// descending order: the span per instruction is unchanged, and the scan
// runs "forwards" over lanes in both directions.
//
// Per chunk a lane (1) folds its VEC elements into one affine pair, (2) takes
// part in a wave64 inclusive scan of the pairs on DPP lane moves (row_shr 1, 2,
// 4, 8, row_bcast 15, row_bcast 31), (3) once the carry into the chunk is
// known, replays its VEC elements from its own carry-in and stores them.
// Chunk-to-chunk carries are single FMAs; wave-to-wave carries go through LDS;
// tile-to-tile carries go through registers (ROW kernel, one workgroup walks a
// row) or through a decoupled look-back chain in global memory (LOOKBACK
// kernel, the tiles of a row are spread over workgroups).
//
// The op is HBM-bound (12 B/element forward, 20 B/element backward in fp32) and
// has no contraction in it, so no MFMA is used anywhere.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#ifndef SCANSCAM_NT_LOAD
#define SCANSCAM_NT_LOAD 1
#endif
#ifndef SCANSCAM_NT_STORE
#define SCANSCAM_NT_STORE 1
#endif


namespace scanscam {

constexpr int kWave = 64;
constexpr int kMaxWaves = 16;

// ---------------------------------------------------------------------------
// Kernel arguments (plain pointers; the host fills them per launch).
// ---------------------------------------------------------------------------
//
// Rows form a two-level grid of n0 groups of n1 rows. Row r1 of group r0 of tensor k starts at
// element r0 * s0[k] + r1 * s1[k]; time is unit-stride. A contiguous [rows, T] tensor is one group
// with s1 = T. The ROW and SMALL kernels take the group from blockIdx.y and `rows` = n1; the
// LOOKBACK kernel takes `rows` = n0 * n1 and divides.
struct ScanArgs {
    const void *a;   // gates                       [rows, T]
    const void *x;   // forward: b      backward: gh
    const void *h;   // forward: unused backward: saved forward output
    void *y0;        // forward: h      backward: gb (value grad)
    void *y1;        // forward: unused backward: ga (gate grad)
    int64_t s0[5];   // element stride from group to group, per tensor in the order above
    int64_t s1[5];   // element stride from row to row
    int64_t rows;
    int64_t n1;      // LOOKBACK: rows per group
    int32_t T;
    int32_t nch;            // chunks per row = ceil(T / (64*VEC))
    int32_t wpr;            // ROW: waves cooperating on one row
    int32_t group;          // SMALL: lanes per row (power of two, <= 64)
    int32_t tiles_per_row;  // LOOKBACK: tiles per row
    int32_t counters;       // LOOKBACK: number of ticket counters (row r uses counter r % counters)
    int32_t row_major;      // LOOKBACK: a counter's tickets walk its rows one after the other
    int32_t line_shift;     // ROW, LOOKBACK: chunks are laid out from the 128-byte line border before each row's start
    int32_t desc_base;      // LOOKBACK: first tile-descriptor word of the workspace
    int64_t super_base;     // LOOKBACK: first super-tile-descriptor word of the workspace
    int32_t spin_limit;     // LOOKBACK: polls before a wait gives up
    uint64_t *ws;           // LOOKBACK: ticket counters + tile descriptors
};

// Look-back workspace layout, in 64-bit words. Ticket counter c is word
// c * kCounterStride (one counter per 128-byte line, so that counters do not
// serialise on one another); word 1 is raised if a look-back wait ever expired
// (results are then NaN). Then come the descriptor words: per tile its aggregate
// pair, per super-tile of 64 tiles its aggregate pair and its end value (see
// Desc below for their encoding). Before each launch the counters are zeroed
// and the descriptor words set to all ones ("not yet").
constexpr int kCounterStride = 16;
constexpr int kMaxCounters = 256;

// ---------------------------------------------------------------------------
// Storage types: float, __bf16, _Float16 (arithmetic in fp32) and double (fp64).
// ---------------------------------------------------------------------------
template <int BYTES> struct RawT;
template <> struct RawT<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <> struct RawT<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct RawT<4> { typedef uint32_t type; };
template <> struct RawT<2> { typedef uint16_t type; };

template <typename ST, int VEC> struct Elems { ST e[VEC]; };

// Arithmetic type of a storage type: fp32 for float and the 16-bit types, fp64 for double.
template <typename ST> struct ComputeOf { using type = float; };
template <> struct ComputeOf<double> { using type = double; };

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_(double a, double b, double c) { return __builtin_fma(a, b, c); }

template <typename ST, int VEC> struct Vec {
    using raw_t = typename RawT<sizeof(ST) * VEC>::type;

    static __device__ __forceinline__ raw_t zero_raw()
    {
        Elems<ST, VEC> z;
#pragma unroll
        for (int k = 0; k < VEC; k++) z.e[k] = (ST)0.0f;
        return __builtin_bit_cast(raw_t, z);
    }
    static __device__ __forceinline__ raw_t load(const ST *p)
    {
        const raw_t *q = reinterpret_cast<const raw_t *>(p);
#if SCANSCAM_NT_LOAD
        return __builtin_nontemporal_load(q);
#else
        return *q;
#endif
    }
    // The same accesses for a vector that is only element-aligned (rows of a length that is not a
    // multiple of VEC start anywhere): still one 16-byte instruction, the memory pipeline splits it.
    typedef raw_t raw_unaligned_t __attribute__((aligned(sizeof(ST))));
    static __device__ __forceinline__ raw_t load_unaligned(const ST *p)
    {
        return __builtin_nontemporal_load(reinterpret_cast<const raw_unaligned_t *>(p));
    }
    static __device__ __forceinline__ void store_unaligned(ST *p, raw_t r)
    {
        __builtin_nontemporal_store(r, reinterpret_cast<raw_unaligned_t *>(p));
    }
    // The partial vector at the start or the end of a row (bit k of `inside` set = component k lies
    // inside the row; the others are neither read nor written) is loaded with one element-aligned
    // 16-byte load like every other vector's: the window of VEC elements that ends with the row
    // (partial vector at its end) or starts with it (at its start), whose components are then moved
    // into place inside the registers (shift_components; those outside the row become zero). No
    // branch and no instruction per element, so all loads of a wave are still issued before the first
    // is waited for. Needs rows of at least VEC elements. window_shift: how many components the window
    // starts after (> 0) or before (< 0) the vector; 0 for a whole vector and for a lane without one.
    static __device__ __forceinline__ int window_shift(uint32_t inside)
    {
        const int lo = inside ? __builtin_ctz(inside) : 0, hi = inside ? 32 - __builtin_clz(inside) : VEC;
        return hi < VEC ? hi - VEC : lo;  // < 0: the window starts before component 0; > 0: after it
    }
    // Components moved up by s places (s > 0) or down by -s (s < 0) inside a 16-byte vector.
    static __device__ __forceinline__ raw_t shift_components(raw_t r, int s)
    {
        if constexpr (sizeof(raw_t) != 16) {
            return r;
        } else {
            const uint64_t lo = (uint64_t)r.x | ((uint64_t)r.y << 32), hi = (uint64_t)r.z | ((uint64_t)r.w << 32);
            const int bits = (s < 0 ? -s : s) * (int)sizeof(ST) * 8;  // 0 ... 112
            const int b = bits & 63;
            const bool far = bits >= 64;
            uint64_t out_lo, out_hi;
            if (s < 0) {
                out_lo = far ? (hi >> b) : ((lo >> b) | ((hi << 1) << (63 - b)));
                out_hi = far ? 0 : (hi >> b);
            } else {
                out_hi = far ? (lo << b) : ((hi << b) | ((lo >> 1) >> (63 - b)));
                out_lo = far ? 0 : (lo << b);
            }
            raw_t out;
            out.x = (uint32_t)out_lo;
            out.y = (uint32_t)(out_lo >> 32);
            out.z = (uint32_t)out_hi;
            out.w = (uint32_t)(out_hi >> 32);
            return out;
        }
    }
    // The components whose bit is set in `inside` only: one store per component under a lane mask.
    static __device__ __forceinline__ void store_part(ST *p, raw_t r, uint32_t inside)
    {
        const Elems<ST, VEC> e = __builtin_bit_cast(Elems<ST, VEC>, r);
#pragma unroll
        for (int k = 0; k < VEC; k++)
            if ((inside >> k) & 1u) p[k] = e.e[k];
    }
    // For data that is read a second time soon: left to the caches' normal policy.
    static __device__ __forceinline__ raw_t load_cached(const ST *p) { return *reinterpret_cast<const raw_t *>(p); }
    static __device__ __forceinline__ void store(ST *p, raw_t r)
    {
        raw_t *q = reinterpret_cast<raw_t *>(p);
#if SCANSCAM_NT_STORE
        __builtin_nontemporal_store(r, q);
#else
        *q = r;
#endif
    }
    template <typename CT> static __device__ __forceinline__ void unpack(raw_t r, CT (&f)[VEC])
    {
        Elems<ST, VEC> e = __builtin_bit_cast(Elems<ST, VEC>, r);
#pragma unroll
        for (int k = 0; k < VEC; k++) f[k] = (CT)e.e[k];
    }
    template <typename CT> static __device__ __forceinline__ raw_t pack(const CT (&f)[VEC])
    {
        Elems<ST, VEC> e;
#pragma unroll
        for (int k = 0; k < VEC; k++) e.e[k] = (ST)f[k];
        return __builtin_bit_cast(raw_t, e);
    }
};

// ---------------------------------------------------------------------------
// Lane moves.
// ---------------------------------------------------------------------------
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float old, float src)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, src),
                                           CTRL, ROW_MASK, 0xf, false));
}

struct Halves { int lo, hi; };

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_move(double old, double src)
{
    const Halves o = __builtin_bit_cast(Halves, old), s = __builtin_bit_cast(Halves, src);
    Halves r;
    r.lo = __builtin_amdgcn_update_dpp(o.lo, s.lo, CTRL, ROW_MASK, 0xf, false);
    r.hi = __builtin_amdgcn_update_dpp(o.hi, s.hi, CTRL, ROW_MASK, 0xf, false);
    return __builtin_bit_cast(double, r);
}

// Value of the previous / next lane of the wave; `fill` where there is none.
template <typename CT> __device__ __forceinline__ CT lane_prev(CT src, CT fill) { return dpp_move<0x138, 0xf>(fill, src); }
template <typename CT> __device__ __forceinline__ CT lane_next(CT src, CT fill) { return dpp_move<0x130, 0xf>(fill, src); }

__device__ __forceinline__ float read_lane(float v, int lane)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ double read_lane(double v, int lane)
{
    const Halves s = __builtin_bit_cast(Halves, v);
    Halves r;
    r.lo = __builtin_amdgcn_readlane(s.lo, lane);
    r.hi = __builtin_amdgcn_readlane(s.hi, lane);
    return __builtin_bit_cast(double, r);
}

// Inclusive scan of affine pairs over the lanes of a wave (ascending lane =
// later in scan order). With GROUPED the wave is cut into independent groups of
// `group` lanes (j = lane index inside its group). Lanes that have no source
// in a step receive the identity map (1, 0). All 64 lanes must be active.
template <bool GROUPED, typename CT>
__device__ __forceinline__ void wave_scan(CT &A, CT &B, int j)
{
#define SCANSCAM_STEP(CTRL, ROW_MASK, OFF)                      \
    {                                                           \
        CT A1 = dpp_move<CTRL, ROW_MASK>(CT(1), A);            \
        CT B1 = dpp_move<CTRL, ROW_MASK>(CT(0), B);            \
        if (GROUPED) {                                          \
            const bool use = j >= (OFF);                        \
            A1 = use ? A1 : CT(1);                              \
            B1 = use ? B1 : CT(0);                              \
        }                                                       \
        B = fma_(A, B1, B);                                     \
        A = A * A1;                                             \
    }
    SCANSCAM_STEP(0x111, 0xf, 1)   // row_shr:1
    SCANSCAM_STEP(0x112, 0xf, 2)   // row_shr:2
    SCANSCAM_STEP(0x114, 0xf, 4)   // row_shr:4
    SCANSCAM_STEP(0x118, 0xf, 8)   // row_shr:8
    SCANSCAM_STEP(0x142, 0xa, 16)  // row_bcast:15 into rows 1 and 3
    SCANSCAM_STEP(0x143, 0xc, 32)  // row_bcast:31 into rows 2 and 3
#undef SCANSCAM_STEP
}

// ---------------------------------------------------------------------------
// One wave's share of a tile: U chunks.
//
// Phase "load":   issue every global load of the U chunks.
// Phase "reduce": per-lane fold + wave scan per chunk -> PA/PB, chunk totals.
// Phase "apply":  given the carry into chunk 0, replay and store.
// With CHAIN the U chunks are consecutive in scan order (carry flows from one
// into the next); without it they are unrelated rows (SMALL kernel).
// ---------------------------------------------------------------------------
// With RAGGED, rows may start at any element (their length need not be a
// multiple of VEC, bases need not be 16-byte aligned): vectors are loaded and
// stored element-aligned, and the first and the last vector of a row may hold
// fewer than VEC of its elements (bit mask `inside`), the rest being masked to
// the identity.
template <typename ST, int VEC, int U, bool REV, bool GROUPED, bool CHAIN, bool RAGGED = false, bool LEAN = false>
struct WaveTile {
    using V = Vec<ST, VEC>;
    using raw_t = typename V::raw_t;
    using CT = typename ComputeOf<ST>::type;
    static constexpr uint32_t kAll = (1u << VEC) - 1u;  // all components of a vector

    // Where this lane's vector of chunk u lives. Lanes without a vector point at element 0 of an
    // existing row (col = 0), which is always readable.
    int32_t col[U];  // first element of the vector inside its row (m*VEC)
    bool valid[U];   // inside the row (and the row exists)
    uint32_t inside[RAGGED ? U : 1];  // RAGGED: bit k set = component k of the vector lies inside the row
    // Start of the row in tensor k = 0..4 (a, x, h, y0, y1), in elements. The ROW and LOOKBACK kernels
    // have one row per wave (wave-uniform); in the SMALL kernel `base` is the start of the group and
    // the row of chunk u, which differs from lane to lane, is added per access.
    int64_t base[5];
    int64_t rowi[GROUPED ? U : 1];

    __device__ __forceinline__ void set_row(const ScanArgs &p, int64_t group, int64_t row)
    {
#pragma unroll
        for (int k = 0; k < 5; k++) base[k] = group * p.s0[k] + row * p.s1[k];
    }
    // Rows that start inside a 128-byte line (a row length that is no multiple of it): laying the
    // chunks out from the line border before the row's start keeps every load and store instruction of
    // a wave on whole lines. Returns how many vectors lie between that border and the row's start (in
    // tensor a; the other tensors of a dense call share it). Vector m of the row is then slot
    // m + shift of the chunks; slots before the row and past its end are masked like any other.
    // With RAGGED (rows start at any element) the shift is counted in elements: the vectors then start
    // on 16-byte borders of tensor a, and the first vector of a row may lie partly before its start.
    __device__ __forceinline__ int line_shift(const ScanArgs &p) const
    {
        if (GROUPED || !p.line_shift) return 0;
        const uint64_t byte = (uint64_t)reinterpret_cast<uintptr_t>(p.a) + (uint64_t)base[0] * sizeof(ST);
        return (int)((byte & 127u) / ((RAGGED ? 1 : VEC) * sizeof(ST)));
    }

    // Places slot q of the chunks (a vector index counted from the row's line border) in the row.
    __device__ __forceinline__ void place(int u, int q, int shift, bool row_ok, int T)
    {
        if (!RAGGED) {
            const int m = q - shift;
            valid[u] = row_ok && m >= 0 && (int64_t)m * VEC < T;
            col[u] = valid[u] ? m * VEC : 0;
        } else {
            const int64_t x0 = (int64_t)q * VEC - shift;  // element of the row at component 0
            const int64_t l = x0 < 0 ? -x0 : 0, h = T - x0;
            const int lo = (int)(l < VEC ? l : VEC), hi = (int)(h < 0 ? 0 : (h < VEC ? h : VEC));
            valid[u] = row_ok && q >= 0 && lo < hi;
            inside[u] = valid[u] ? ((kAll >> (VEC - hi)) & (kAll << lo) & kAll) : 0u;
            col[u] = valid[u] ? (int32_t)x0 : 0;
        }
    }
    template <int K> __device__ __forceinline__ int64_t at(const ScanArgs &p, int u) const
    {
        int64_t o = base[K] + col[u];
        if (GROUPED) o += rowi[u] * p.s1[K];
        return o;
    }

    __device__ __forceinline__ void put(ST *p, raw_t r, int u) const
    {
        if (!RAGGED) {
            V::store(p, r);
        } else if (inside[u] == kAll) {
            V::store_unaligned(p, r);
        } else {
            V::store_part(p, r, inside[u]);
        }
    }

    raw_t ra[U], rx[U], rh[REV ? U : 1];
    CT edge_a[REV ? U : 1];  // a[(m+1)*VEC] for the first lane of a group
    CT edge_h[REV ? U : 1];  // h[m*VEC - 1] for the last lane of a group

    // LEAN, for 16-bit storage with 8 elements per vector: the (gate, value) pairs are not kept from
    // reduce() to apply() (64 fp32 registers per lane at U = 4, 96 with h[t-1] in the backward pass)
    // but built a second time from the packed vectors, which take half the registers. It pays where
    // waves wait between the two (the look-back kernel: more waves per SIMD cover the wait) and
    // costs 1-2 % where they do not (the row kernel).
    static constexpr bool REBUILD = LEAN && sizeof(ST) == 2 && VEC == 8;
    CT g[REBUILD ? 1 : U][VEC], v[REBUILD ? 1 : U][VEC];
    CT PA[U], PB[U];

    __device__ __forceinline__ void load(const ScanArgs &p, int j, int jlast)
    {
        const ST *a = static_cast<const ST *>(p.a);
        const ST *x = static_cast<const ST *>(p.x);
        const ST *h = static_cast<const ST *>(p.h);
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (!RAGGED) {
                // Unconditional: lanes outside the row read element 0 of a row instead and are
                // masked in reduce(). No branch separates the loads, so all of the wave's U x streams
                // loads are in flight before the first one is waited for.
                ra[u] = V::load(a + at<0>(p, u));
                rx[u] = V::load(x + at<1>(p, u));
                if (REV) rh[u] = V::load(h + at<2>(p, u));
            } else {
                // Just as unconditional: a partial vector is loaded as the window of VEC elements that
                // starts or ends with the row (settle() moves its components into place once all loads
                // are under way), lanes outside the row read the row's first vector.
                const int s = V::window_shift(inside[u]);
                ra[u] = V::load_unaligned(a + at<0>(p, u) + s);
                rx[u] = V::load_unaligned(x + at<1>(p, u) + s);
                if (REV) rh[u] = V::load_unaligned(h + at<2>(p, u) + s);
            }
            if (REV) {
                edge_a[u] = CT(0);
                edge_h[u] = CT(0);
                // Neighbours that no lane of this group holds. With CHAIN the chunks of a
                // wave are adjacent, so only the wave's outer borders need memory: the
                // inner ones are taken from the neighbouring chunk's registers in reduce().
                const bool need_a = !CHAIN || u == 0;
                const bool need_h = !CHAIN || u == U - 1;
                if (need_a && valid[u] && j == 0 && col[u] + VEC < p.T) edge_a[u] = (CT)a[at<0>(p, u) + VEC];
                if (need_h && valid[u] && j == jlast && col[u] > 0) edge_h[u] = (CT)h[at<2>(p, u) - 1];
            }
        }
    }

    // RAGGED: the partial vectors, loaded as windows, get their components moved into place (those
    // outside the row become zero). Only VALU work: no wait separates the loads issued by load().
    __device__ __forceinline__ void settle()
    {
        if (RAGGED) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int s = V::window_shift(inside[u]);
                if (s != 0) {
                    ra[u] = V::shift_components(ra[u], s);
                    rx[u] = V::shift_components(rx[u], s);
                    if (REV) rh[u] = V::shift_components(rh[u], s);
                }
            }
        }
    }

    // Backward with CHAIN: a[first element] and h[last element] of every chunk's vectors, for the
    // lanes at the borders between the chunks of this wave.
    __device__ __forceinline__ void borders(CT (&first_a)[REV ? U : 1], CT (&last_h)[REV ? U : 1]) const
    {
        if (REV && CHAIN) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                CT t[VEC];
                V::unpack(ra[u], t);
                first_a[u] = valid[u] ? t[0] : CT(0);
                V::unpack(rh[u], t);
                last_h[u] = valid[u] ? t[VEC - 1] : CT(0);
            }
        }
    }

    // (gate, value) per element of chunk u in scan order, and for the backward pass h[t-1].
    __device__ __forceinline__ void build(int u, int j, int jlast, const CT (&first_a)[REV ? U : 1],
                                          const CT (&last_h)[REV ? U : 1], CT (&G)[VEC], CT (&X)[VEC],
                                          CT (&HP)[VEC]) const
    {
        CT fa[VEC], fx[VEC];
        V::unpack(ra[u], fa);
        V::unpack(rx[u], fx);
#pragma unroll
        for (int k = 0; k < VEC; k++) {  // lanes outside the row hold a = 0, x = 0
            fa[k] = valid[u] ? fa[k] : CT(0);
            fx[k] = valid[u] ? fx[k] : CT(0);
        }
        if (!REV) {
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                const bool in_row = RAGGED ? ((inside[u] >> k) & 1u) != 0 : valid[u];
                G[k] = in_row ? fa[k] : CT(1);
                X[k] = fx[k];  // zero-filled where invalid
            }
        } else {
            CT fh[VEC];
            V::unpack(rh[u], fh);
#pragma unroll
            for (int k = 0; k < VEC; k++) fh[k] = valid[u] ? fh[k] : CT(0);
            // Scan order k <-> time t0 + VEC-1-k. gate = a[t+1], value = gh[t],
            // hp = h[t-1]. Invalid lanes hold a = 0, so a neighbour past the
            // end of the row reads as gate 0, which is what t = T-1 needs.
            CT a_next = lane_prev(fa[0], CT(0));        // lane-1 holds vector m+1
            CT h_prev = lane_next(fh[VEC - 1], CT(0));  // lane+1 holds vector m-1
            CT border_a = edge_a[u], border_h = edge_h[u];
            if (CHAIN && u > 0) border_a = read_lane(first_a[u - 1], kWave - 1);
            if (CHAIN && u + 1 < U) border_h = read_lane(last_h[u + 1], 0);
            a_next = (j == 0) ? border_a : a_next;
            h_prev = (j == jlast) ? border_h : h_prev;
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                const CT gk = (k == 0) ? a_next : fa[(VEC - k) % VEC];
                // Scan position k is element VEC-1-k of the vector; past the row's end it is the identity
                // (its a and gh read as 0, so the element below it sees gate 0, as t = T-1 must).
                const bool in_row = RAGGED ? ((inside[u] >> (VEC - 1 - k)) & 1u) != 0 : valid[u];
                G[k] = in_row ? gk : CT(1);
                X[k] = fx[VEC - 1 - k];
                HP[k] = (k == VEC - 1) ? h_prev : fh[(VEC - 2 - k) < 0 ? 0 : (VEC - 2 - k)];
            }
        }
    }

    // Builds (gate, value) per element in scan order and reduces them.
    __device__ __forceinline__ void reduce(int j, int jlast, CT (&hp)[REV ? U : 1][VEC])
    {
        CT first_a[REV ? U : 1], last_h[REV ? U : 1];
        settle();
        borders(first_a, last_h);
#pragma unroll
        for (int u = 0; u < U; u++) {
            CT G[VEC], X[VEC], HP[VEC];
            build(u, j, jlast, first_a, last_h, G, X, HP);
            if (!REBUILD) {
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    g[u][k] = G[k];
                    v[u][k] = X[k];
                    if (REV) hp[u][k] = HP[k];
                }
            }
            CT A = G[0], B = X[0];
#pragma unroll
            for (int k = 1; k < VEC; k++) {
                B = fma_(G[k], B, X[k]);
                A = A * G[k];
            }
            wave_scan<GROUPED, CT>(A, B, j);
            PA[u] = A;
            PB[u] = B;
        }
        if (REBUILD) {
            // The packed vectors pass through an empty asm statement, so that the compiler
            // cannot carry their unpacked form over to apply() instead of unpacking again.
#pragma unroll
            for (int u = 0; u < U; u++) {
                asm volatile("" : "+v"(ra[u]), "+v"(rx[u]));
                if (REV) asm volatile("" : "+v"(rh[u]));
            }
        }
    }

    // Aggregate of the wave's U chunks (CHAIN only): composition in scan order.
    __device__ __forceinline__ void total(CT &WA, CT &WB) const
    {
        WA = read_lane(PA[0], 63);
        WB = read_lane(PB[0], 63);
#pragma unroll
        for (int u = 1; u < U; u++) {
            const CT TA = read_lane(PA[u], 63), TB = read_lane(PB[u], 63);
            WB = fma_(TA, WB, TB);
            WA = TA * WA;
        }
    }

    __device__ __forceinline__ void apply(const ScanArgs &p, CT carry, int j, int jlast,
                                          const CT (&hp)[REV ? U : 1][VEC])
    {
        ST *y0 = static_cast<ST *>(p.y0);
        ST *y1 = static_cast<ST *>(p.y1);
        CT first_a[REV ? U : 1], last_h[REV ? U : 1];
        if (REBUILD) borders(first_a, last_h);
#pragma unroll
        for (int u = 0; u < U; u++) {
            CT G[VEC], X[VEC], HP[VEC];
            if (REBUILD) {
                build(u, j, jlast, first_a, last_h, G, X, HP);
            } else {
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    G[k] = g[u][k];
                    X[k] = v[u][k];
                    if (REV) HP[k] = hp[u][k];
                }
            }
            // Map of everything before this lane inside the chunk.
            CT EA = lane_prev(PA[u], CT(1));
            CT EB = lane_prev(PB[u], CT(0));
            if (GROUPED) {
                EA = (j == 0) ? CT(1) : EA;
                EB = (j == 0) ? CT(0) : EB;
            }
            const CT c = CHAIN ? carry : CT(0);
            CT acc = fma_(EA, c, EB);
            CT out[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                acc = fma_(G[k], acc, X[k]);
                out[k] = acc;
            }
            if (CHAIN && u + 1 < U)
                carry = fma_(read_lane(PA[u], 63), carry, read_lane(PB[u], 63));
            if (!REV) {
                if (valid[u]) put(y0 + at<3>(p, u), V::pack(out), u);
            } else {
                CT gb[VEC], ga[VEC];
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    gb[VEC - 1 - k] = out[k];
                    ga[VEC - 1 - k] = out[k] * HP[k];
                }
                if (valid[u]) {
                    put(y0 + at<3>(p, u), V::pack(gb), u);
                    put(y1 + at<4>(p, u), V::pack(ga), u);
                }
            }
        }
    }
};

// ---------------------------------------------------------------------------
// ROW kernel: `wpr` waves walk one row tile by tile; a workgroup of W waves
// holds W / wpr rows. Tile = wpr * U chunks. Carries: FMA chunk to chunk, LDS
// wave to wave, a register tile to tile.
// ---------------------------------------------------------------------------
template <typename ST, int VEC, int U, bool REV, int MAXT, bool RAGGED = false>
__global__ __launch_bounds__(MAXT) void scan_row_kernel(const ScanArgs p)
{
    using CT = typename ComputeOf<ST>::type;
    __shared__ CT lds_A[2][kMaxWaves];
    __shared__ CT lds_B[2][kMaxWaves];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // wave-uniform, kept in a scalar register
    const int nwaves = blockDim.x / kWave;
    const int wpr = p.wpr;
    const int rows_per_wg = nwaves / wpr;
    const int wr = wave % wpr;          // this wave's place among the row's waves
    const int wbase = wave - wr;        // first wave of the row's group
    // Consecutive workgroups (which the hardware deals round-robin to the 8 XCDs) take consecutive
    // rows; giving each XCD one contiguous eighth of the rows instead measured 5 % slower.
    const int64_t row = (int64_t)blockIdx.x * rows_per_wg + wave / wpr;
    const bool row_ok = row < p.rows;
    const int nvp = p.nch * kWave;      // vectors per row, padded to whole chunks
    const int tile_chunks = wpr * U;
    const int ntiles = (p.nch + tile_chunks - 1) / tile_chunks;

    WaveTile<ST, VEC, U, REV, false, true, RAGGED> w;
    w.set_row(p, blockIdx.y, row_ok ? row : 0);
    CT hp[REV ? U : 1][VEC];
    CT row_carry = CT(0);
    const int shift = w.line_shift(p);

    for (int it = 0; it < ntiles; it++) {
        const int chunk0 = (it * wpr + wr) * U;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int s = (chunk0 + u) * kWave + lane;  // slot in scan order
            w.place(u, REV ? nvp - 1 - s : s, shift, row_ok, p.T);
        }
        w.load(p, lane, kWave - 1);
        w.reduce(lane, kWave - 1, hp);

        CT carry = row_carry;
        if (wpr > 1) {
            CT WA, WB;
            w.total(WA, WB);
            if (lane == 0) {
                lds_A[it & 1][wave] = WA;
                lds_B[it & 1][wave] = WB;
            }
            __syncthreads();
            CT c = row_carry;
            for (int q = 0; q < wpr; q++) {
                if (q == wr) carry = c;
                c = fma_(lds_A[it & 1][wbase + q], c, lds_B[it & 1][wbase + q]);
            }
            row_carry = c;
        } else if (ntiles > 1) {
            CT WA, WB;
            w.total(WA, WB);
            row_carry = fma_(WA, row_carry, WB);
        }
        w.apply(p, carry, lane, kWave - 1, hp);
    }
}

// ---------------------------------------------------------------------------
// SMALL kernel: rows no longer than one chunk. `group` lanes hold one row, a
// wave holds U * 64 / group rows, and nothing is carried anywhere. With RAGGED
// the rows start at any element: a lane's vector is loaded element-aligned and
// the last vector of a row is partial.
// ---------------------------------------------------------------------------
template <typename ST, int VEC, int U, bool REV, int MAXT, bool RAGGED = false>
__global__ __launch_bounds__(MAXT) void scan_small_kernel(const ScanArgs p)
{
    using CT = typename ComputeOf<ST>::type;
    const int lane = threadIdx.x & (kWave - 1);
    const int G = p.group;
    const int j = lane & (G - 1);
    const int rows_per_chunk = kWave / G;
    const int64_t wave_id = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    const int64_t row0 = wave_id * (U * rows_per_chunk) + lane / G;

    WaveTile<ST, VEC, U, REV, true, false, RAGGED> w;
    w.set_row(p, blockIdx.y, 0);
    CT hp[REV ? U : 1][VEC];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int64_t row = row0 + (int64_t)u * rows_per_chunk;
        w.place(u, REV ? G - 1 - j : j, 0, row < p.rows, p.T);
        w.rowi[u] = w.valid[u] ? row : 0;
    }
    w.load(p, j, G - 1);
    w.reduce(j, G - 1, hp);
    w.apply(p, CT(0), j, G - 1, hp);
}

// ---------------------------------------------------------------------------
// LOOKBACK kernel: the tiles of a row are spread over workgroups. Tiles are
// handed out by atomic tickets, so every tile a workgroup may wait for was
// taken by a workgroup that is already running. A single counter would
// serialise the whole grid on one address, so there are up to kMaxCounters of
// them, each serving the rows r with r % counters == c. In tile-major order
// ticket k of a counter works on its (k % rows_here)-th row, tile k / rows_here,
// which keeps the tiles in flight at any moment spread over all rows: few
// neighbours wait for each other. In row-major order (p.row_major, chosen by the
// host for many rows of a few tiles each, with few counters) ticket k works on
// tile k % tiles_per_row of the counter's (k / tiles_per_row)-th row, so the
// tiles in flight cover consecutive rows: one sweep through memory in address
// order, which the memory system serves faster than many separate spans.
// Either way a tile only ever waits for tiles of its own row with smaller
// tickets of the same counter.
//
// Carry protocol, two levels, run by wave 0 of the workgroup. 64 consecutive
// tiles of a row form a super-tile. Let (A_q, B_q) be the aggregate of tile q
// of super-tile m, (SA_m, SB_m) the composition of all 64 of them and S_m the
// scan value entering the super-tile (S_0 = 0).
//   tile level   tile j publishes (A_j, B_j), collects those of tiles 0..j-1 of
//                its own super-tile (one per lane), and scans them with the
//                wave ladder: its carry-in is P_{j-1}(S_m). Tile 63 thereby
//                also has (SA_m, SB_m), and publishes it at once.
//   super level  64 lanes inspect the 64 preceding super-tiles; the nearest
//                one with a published end value SI_s = fma(SA_s, S_s, SB_s)
//                starts a chain of FMAs through the aggregates of the
//                super-tiles after it, oldest first, which ends in S_m. Tile 63
//                then publishes SI_m.
// Nothing waits for a value that itself waited for a predecessor's carry
// except along the SI chain, which advances 64 tiles per step and can skip
// over up to 64 super-tiles whose aggregates are known. Every value has one
// defining expression (S_{m+1} = fma(SA_m, S_m, SB_m), fixed ladder inside a
// super-tile), so results do not depend on timing.
// ---------------------------------------------------------------------------
constexpr int kSuper = 64;  // tiles per super-tile (one per lane)

// Published values. The workspace's descriptor words are set to all ones before each launch, and every
// word that is written is distinguishable from that pattern on its own, so a word is self-validating and
// no fence is needed around it (each is written with one relaxed agent-scope 64-bit store).
//   fp32 pair (A, B) of an affine map: ONE word {bits(A), bits(B) << 32}. "Not yet" is the low half
//     0xffffffff, a NaN pattern that no published A has: a NaN A is published as the canonical quiet
//     NaN 0x7fc00000. A tile owns one such word; one poll of it is one 8-byte load.
//   fp32 single value (a super-tile's end value): {bits(v), 1 << 32}.
//   fp64: every 32-bit half of a value in the low half of its own word under the flag 1 (a pair is 4
//     words, a single value 2).
// A tile owns kTileWords<CT> words, a super-tile kSuperWords<CT>: its pair (SA, SB), then its end value SI.
template <typename CT> struct Desc;
template <> struct Desc<float> {
    static constexpr int W = 1;        // words per single value
    static constexpr int PAIR = 1;     // words per pair
    static constexpr uint32_t kNotYet = 0xffffffffu;
    static __device__ __forceinline__ void store(uint64_t *p, float v)
    {
        const uint64_t w = (1ull << 32) | (uint64_t)__builtin_bit_cast(uint32_t, v);
        __hip_atomic_store(p, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    static __device__ __forceinline__ bool load(const uint64_t *p, float &v)
    {
        const uint64_t w = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v = __builtin_bit_cast(float, (uint32_t)w);
        return (w >> 32) == 1;
    }
    static __device__ __forceinline__ uint64_t pack_pair(float a, float b)
    {
        uint32_t ua = __builtin_bit_cast(uint32_t, a);
        ua = (a != a) ? 0x7fc00000u : ua;
        return (uint64_t)ua | ((uint64_t)__builtin_bit_cast(uint32_t, b) << 32);
    }
    static __device__ __forceinline__ void store_pair(uint64_t *p, float a, float b)
    {
        __hip_atomic_store(p, pack_pair(a, b), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // A raw word (fetched now, looked at later) and its interpretation as a pair or as a single value.
    static __device__ __forceinline__ uint64_t fetch_raw(const uint64_t *p)
    {
        return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    static __device__ __forceinline__ bool unpack(uint64_t w, float &v)
    {
        v = __builtin_bit_cast(float, (uint32_t)w);
        return (w >> 32) == 1;
    }
    static __device__ __forceinline__ bool unpack_pair(uint64_t w, float &a, float &b)
    {
        a = __builtin_bit_cast(float, (uint32_t)w);
        b = __builtin_bit_cast(float, (uint32_t)(w >> 32));
        return (uint32_t)w != kNotYet;
    }
    static __device__ __forceinline__ bool load_pair(const uint64_t *p, float &a, float &b)
    {
        return unpack_pair(fetch_raw(p), a, b);
    }
};
template <> struct Desc<double> {
    static constexpr int W = 2;
    static constexpr int PAIR = 4;
    static __device__ __forceinline__ void store(uint64_t *p, double v)
    {
        const uint64_t b = __builtin_bit_cast(uint64_t, v);
        __hip_atomic_store(p + 0, (1ull << 32) | (b & 0xffffffffull), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(p + 1, (1ull << 32) | (b >> 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    static __device__ __forceinline__ bool load(const uint64_t *p, double &v)
    {
        const uint64_t lo = __hip_atomic_load(p + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint64_t hi = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v = __builtin_bit_cast(double, (hi << 32) | (lo & 0xffffffffull));
        return (lo >> 32) == 1 && (hi >> 32) == 1;
    }
    static __device__ __forceinline__ void store_pair(uint64_t *p, double a, double b)
    {
        store(p, a);
        store(p + W, b);
    }
    static __device__ __forceinline__ bool load_pair(const uint64_t *p, double &a, double &b)
    {
        const bool ra = load(p, a), rb = load(p + W, b);
        return ra && rb;
    }
    // (No raw form: a pair is four words. The look-back polls fp64 descriptors where it needs them.)
    static __device__ __forceinline__ uint64_t fetch_raw(const uint64_t *) { return ~0ull; }
    static __device__ __forceinline__ bool unpack(uint64_t, double &) { return false; }
    static __device__ __forceinline__ bool unpack_pair(uint64_t, double &, double &) { return false; }
};
template <typename CT> constexpr int kTileWords = Desc<CT>::PAIR;
template <typename CT> constexpr int kSuperWords = Desc<CT>::PAIR + Desc<CT>::W;

// Default number of polls before a waiting wave gives up. Tickets make every
// awaited tile belong to a workgroup that is already running, so the limit is
// never reached in a correct launch (a poll is a memory round trip; the limit
// is about a second). It exists so that no wave can spin for ever: on expiry
// the wave raises word kTimeoutWord of the workspace and carries NaN onwards.
constexpr int kSpinLimit = 1 << 20;
constexpr int kTimeoutWord = 1;

// The look-back of one tile, run by all 64 lanes of one wave (`tile` is wave-uniform). Lane q < j
// collects tile q of this tile's super-tile, lane j holds the tile itself, the rest the identity; lane k
// also watches super-tile m-1-k (before the row starts the value is 0).
//   begin()   where everything lies, what is already known;
//   issue()   the loads of one poll of what is still missing (fp32: raw words kept in registers, not
//             looked at -- so a poll can be in flight while the wave does other work);
//   absorb()  looks at them;
//   finish()  publishes the tile's own aggregate, then polls until the carry is known and returns the
//             scan value entering the tile.
// With EARLY the kernel issues one poll as soon as the wave's data has arrived and reduces the data
// while it is in flight: a predecessor's aggregate that became visible in the meantime is then in hand
// when the tile's own aggregate is, one memory round trip earlier than a poll issued after the reduce.
template <typename CT>
struct Lookback {
    using D = Desc<CT>;
    static constexpr int TW = kTileWords<CT>, SW = kSuperWords<CT>;
    static constexpr bool RAW = sizeof(CT) == 4;  // polls may be issued ahead (one word per pair)

    uint64_t *trow, *srow;
    int j, m, sidx, spr, tpr;
    bool have_t, have_si, have_sa, pending;
    CT A, B, SI, SA, SB;
    uint64_t raw_t, raw_sa, raw_si;

    __device__ __forceinline__ void begin(const ScanArgs &p, int64_t row, int tile, int lane)
    {
        tpr = p.tiles_per_row;
        spr = (tpr + kSuper - 1) / kSuper;
        j = tile % kSuper;
        m = tile / kSuper;
        trow = p.ws + p.desc_base + row * (int64_t)tpr * TW;
        srow = p.ws + p.super_base + row * (int64_t)spr * SW;
        have_t = lane >= j;
        A = CT(1);
        B = CT(0);
        sidx = m - 1 - lane;
        have_si = have_sa = sidx < 0;
        SI = CT(0);
        SA = CT(1);
        SB = CT(0);
        pending = false;
        raw_t = raw_sa = raw_si = ~0ull;
    }

    __device__ __forceinline__ void issue(int lane)
    {
        if (RAW) {
            // Lanes with nothing to fetch keep "not yet" words, which absorb() skips.
            if (!have_t) raw_t = D::fetch_raw(trow + (int64_t)(m * kSuper + lane) * TW);
            if (!have_sa) raw_sa = D::fetch_raw(srow + (int64_t)sidx * SW);
            if (!have_si) raw_si = D::fetch_raw(srow + (int64_t)sidx * SW + D::PAIR);
            pending = true;
        }
    }

    __device__ __forceinline__ void absorb(int lane)
    {
        if (RAW) {
            if (!pending) issue(lane);
            pending = false;
            CT va, vb;
            if (!have_t && D::unpack_pair(raw_t, va, vb)) {
                have_t = true;
                A = va;
                B = vb;
            }
            if (!have_sa && D::unpack_pair(raw_sa, va, vb)) {
                have_sa = true;
                SA = va;
                SB = vb;
            }
            if (!have_si && D::unpack(raw_si, va)) {
                have_si = true;
                SI = va;
            }
        } else {
            CT va, vb;
            if (!have_t && D::load_pair(trow + (int64_t)(m * kSuper + lane) * TW, va, vb)) {
                have_t = true;
                A = va;
                B = vb;
            }
            if (!have_sa && D::load_pair(srow + (int64_t)sidx * SW, va, vb)) {
                have_sa = true;
                SA = va;
                SB = vb;
            }
            if (!have_si && D::load(srow + (int64_t)sidx * SW + D::PAIR, va)) {
                have_si = true;
                SI = va;
            }
        }
    }

    __device__ __forceinline__ CT finish(const ScanArgs &p, int tile, CT TA, CT TB, int lane)
    {
        const bool closes = (j == kSuper - 1) && (m + 1 < spr);  // a later super-tile needs (SA, SB, SI)
        if (lane == 0 && j < kSuper - 1 && tile + 1 < tpr) D::store_pair(trow + (int64_t)tile * TW, TA, TB);
        if (lane == j) {
            A = TA;
            B = TB;
        }
        bool tiles_done = false, super_done = false;
        CT PA = CT(1), PB = CT(0), S = CT(0);
        for (int spin = 0; spin < p.spin_limit; spin++) {
            absorb(lane);
            if (!tiles_done && __ballot(have_t) == ~0ull) {
                tiles_done = true;
                PA = A;
                PB = B;
                wave_scan<false, CT>(PA, PB, lane);
                if (closes) {
                    const CT sa = read_lane(PA, kSuper - 1), sb = read_lane(PB, kSuper - 1);
                    if (lane == 0) D::store_pair(srow + (int64_t)m * SW, sa, sb);
                }
            }
            if (!super_done) {
                const uint64_t mi = __ballot(have_si);
                const uint64_t ma = __ballot(have_sa);
                if (mi != 0) {
                    const int first = __builtin_ctzll(mi);  // nearest super-tile with a published end value
                    const uint64_t need = (first == 0) ? 0ull : ((~0ull) >> (64 - first));
                    if ((ma & need) == need) {
                        S = read_lane(SI, first);
                        for (int q = first - 1; q >= 0; q--) S = fma_(read_lane(SA, q), S, read_lane(SB, q));
                        super_done = true;
                    }
                }
            }
            if (tiles_done && super_done) break;
            if (spin > 0) __builtin_amdgcn_s_sleep(1);
        }
        if (!(tiles_done && super_done)) {
            if (lane == 0) __hip_atomic_store(p.ws + kTimeoutWord, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            S = CT(__builtin_nanf(""));
        }
        const CT end_a = read_lane(PA, kSuper - 1), end_b = read_lane(PB, kSuper - 1);
        if (closes && lane == 0) D::store(srow + (int64_t)m * SW + D::PAIR, fma_(end_a, S, end_b));
        return j > 0 ? fma_(read_lane(PA, j - 1), S, read_lane(PB, j - 1)) : S;
    }
};

#ifndef SCANSCAM_EARLY_POLL
#define SCANSCAM_EARLY_POLL 0
#endif

template <typename ST, int VEC, int U, bool REV, int MAXT, bool RAGGED = false>
__global__ __launch_bounds__(MAXT) void scan_lookback_kernel(const ScanArgs p)
{
    using CT = typename ComputeOf<ST>::type;
    __shared__ CT lds_A[kMaxWaves];
    __shared__ CT lds_B[kMaxWaves];
    __shared__ CT lds_carry;
    __shared__ unsigned lds_ticket;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int nwaves = blockDim.x / kWave;

    // Counter c serves the rows r with r % counters == c; its tickets walk those
    // rows round-robin, tile by tile, or one row after the other.
    const int nctr = p.counters;
    const int ctr = blockIdx.x % nctr;
    if (threadIdx.x == 0)
        lds_ticket = __hip_atomic_fetch_add(reinterpret_cast<unsigned *>(p.ws + (int64_t)ctr * kCounterStride), 1u,
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const unsigned ticket = __builtin_amdgcn_readfirstlane(lds_ticket);
    const int64_t rows_here = (p.rows - ctr + nctr - 1) / nctr;
    if ((int64_t)ticket >= rows_here * p.tiles_per_row) return;  // surplus workgroup of an uneven split
    int64_t row;
    int tile;
    if (p.row_major) {
        row = ctr + (int64_t)nctr * (int64_t)(ticket / (unsigned)p.tiles_per_row);
        tile = (int)(ticket % (unsigned)p.tiles_per_row);
    } else {
        row = ctr + (int64_t)nctr * (int64_t)(ticket % (uint64_t)rows_here);
        tile = (int)(ticket / (uint64_t)rows_here);
    }
    const int nvp = p.nch * kWave;
    const int chunk0 = (tile * nwaves + wave) * U;

    WaveTile<ST, VEC, U, REV, false, true, RAGGED, true> w;
    const int64_t group = row / p.n1;
    w.set_row(p, group, row - group * p.n1);
    CT hp[REV ? U : 1][VEC];
    const int shift = w.line_shift(p);
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int s = (chunk0 + u) * kWave + lane;
        w.place(u, REV ? nvp - 1 - s : s, shift, true, p.T);
    }
    w.load(p, lane, kWave - 1);
    Lookback<CT> lb;
    const bool chained = p.tiles_per_row > 1;
    if (wave == 0 && chained) {
        lb.begin(p, row, tile, lane);
        if (SCANSCAM_EARLY_POLL && Lookback<CT>::RAW) {
            // Once this wave's data is in, one poll goes out and is in flight during the reduce.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            lb.issue(lane);
        }
    }
    w.reduce(lane, kWave - 1, hp);

    CT WA, WB;
    w.total(WA, WB);
    if (lane == 0) {
        lds_A[wave] = WA;
        lds_B[wave] = WB;
    }
    __syncthreads();

    if (wave == 0) {
        // Aggregate of the whole tile, waves in scan order.
        CT TA = lds_A[0], TB = lds_B[0];
        for (int q = 1; q < nwaves; q++) {
            TB = fma_(lds_A[q], TB, lds_B[q]);
            TA = lds_A[q] * TA;
        }
        CT cin = CT(0);
        if (chained) cin = lb.finish(p, tile, TA, TB, lane);
        if (lane == 0) lds_carry = cin;
    }
    __syncthreads();

    CT carry = lds_carry;
    for (int q = 0; q < wave; q++) carry = fma_(lds_A[q], carry, lds_B[q]);
    w.apply(p, carry, lane, kWave - 1, hp);
}

}  // namespace scanscam

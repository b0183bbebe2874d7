// C ABI of libscanscam_hip.so (declared in include/scanscam_hip.h): argument
// checks, the choice of kernel family and launch shape, and the launches.
#include "scanscam_hip.h"

#include "scan_launch.hpp"
#include "scan_cl_plan.hpp"

#include <mutex>

// Look-back scratch of scanscam_scan_fwd_noalloc: a fixed array in every GPU's memory that the library
// runs on, held until the process ends. Host code never uses this name as an address -- it is a
// host-side stand-in for the symbol; noalloc_scratch() asks the runtime where the current device keeps
// its copy and hands that pointer to the kernels.
static __device__ __align__(256) unsigned char scratch[SCANSCAM_NOALLOC_SCRATCH_BYTES];

namespace {

using scanscam::kCounterStride;
using scanscam::kMaxCounters;
using scanscam::kSuper;
using scanscam::kModeFlat;
using scanscam::kModeLookback;
using scanscam::kModeRow;
using scanscam::kModeSmall;
using scanscam::kWave;
using scanscam::Launch;
using scanscam::ScanArgs;

// Prepares the look-back workspace (a kernel, not a memset, so that a caller may capture the launch
// sequence in a HIP graph): the ticket counters and the time-out flag (the first `zero_words` words) are
// zeroed, every descriptor word after them is set to all ones, the kernels' "not yet".
__global__ __launch_bounds__(256) void scan_ws_clear_kernel(uint64_t *ws, int64_t words, int64_t zero_words)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < words) ws[i] = i < zero_words ? 0ull : ~0ull;
}

hipError_t clear_workspace(uint64_t *ws, int64_t words, int64_t zero_words, hipStream_t stream)
{
    void *params[] = {&ws, &words, &zero_words};
    return hipLaunchKernel(reinterpret_cast<const void *>(scan_ws_clear_kernel), dim3((unsigned)((words + 255) / 256)),
                           dim3(256), params, 0, stream);
}

constexpr int64_t kMaxT = (int64_t(1) << 31) - (int64_t(1) << 20);

int elem_size(int dtype)
{
    switch (dtype) {
    case SCANSCAM_F32: return 4;
    case SCANSCAM_BF16:
    case SCANSCAM_F16: return 2;
    case SCANSCAM_F64: return 8;
    default: return 0;
    }
}

// 64-bit words per value published in the look-back workspace (one per 32-bit half), and per tile (its
// aggregate pair) and super-tile (its pair and its end value) of the row layout's look-back kernel, whose
// fp32 pairs are one word (scanscam::kTileWords, kSuperWords).
int value_words(int dtype) { return dtype == SCANSCAM_F64 ? 2 : 1; }
int tile_words(int dtype) { return dtype == SCANSCAM_F64 ? scanscam::kTileWords<double> : scanscam::kTileWords<float>; }
int super_words(int dtype) { return dtype == SCANSCAM_F64 ? scanscam::kSuperWords<double> : scanscam::kSuperWords<float>; }

// Bytes of the arithmetic type behind a storage type.
int compute_size(int dtype) { return dtype == SCANSCAM_F64 ? 8 : 4; }


int pow2_ceil(int64_t v)
{
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

bool unroll_ok(int vec, int full, int unroll)
{
    if (vec == full) return unroll == 1 || unroll == 2 || unroll == 3 || unroll == 4 || unroll == 8;
    return unroll == 1 || unroll == 4;
}

struct Resolved {
    Launch l;
    int nch;
    int tiles_per_row;
    int counters;
    int row_major;       // a counter's tickets walk its rows one after the other (see resolve)
    int line_shift;      // chunks laid out from the 128-byte line border before each row's start (see resolve)
    int64_t super_base;  // word offset of the super-tile descriptors
    size_t ws_bytes;
};

// Look-back tiles in chunks (8 waves x 4 chunks per wave) and the ticket order of the look-back kernel.
// Tile-major: a counter's tickets visit tile 0 of each of its rows, then tile 1 of each, ...; few tiles of a
// row are in flight together, so carries arrive with little waiting, at the price of as many separate spans of
// memory being streamed at once as there are rows. Row-major: a counter's tickets finish one row before the
// next, so the tiles in flight sweep memory in address order, which the memory system serves 5-8 points
// faster (measured with scan-free streaming kernels in both orders), while all tiles of a row are in flight together and wait for each other:
// worth it when a row is only a few tiles long.
constexpr int kTileChunks = 32;
constexpr int kRowMajorCounters = 4;

bool row_major_order(int64_t rows, int tiles_per_row) { return rows >= 256 && tiles_per_row <= 16; }

// Many rows of moderate length: from two tiles per row on, the look-back kernel in row-major order beats one
// workgroup walking each row, which streams as many separate spans as there are rows in flight, leaves CUs
// idle in its last round of workgroups, and whose 16-wave steps seldom divide a row. Measured at 16 M to 128 M
// elements, fp32 and bf16, with tiles fitted to the row (resolve): 2 to 15 tiles per row gain +2 to +20 % forward
// and +9 to +30 % backward, also where the row kernel's workgroups come out in full rounds of 256; rows of 8
// tiles (4 exact steps of the row kernel) tie forward. At 16 tiles the forward pass of the row kernel (8 exact
// steps) is 5-8 % faster and keeps the shape unless its rounds do not come out; the backward pass still gains
// 4-6 %. A problem of fewer than 2048 tiles is too small to hide the extra launch that clears the workspace.
// Rows of more than 16 tiles go to the look-back kernel (in tile-major order) only where the row kernel's
// rounds do not come out.
constexpr int kComputeUnits = 256;  // MI355X

bool prefer_lookback_for_many_rows(int64_t rows, int nch, bool rev, int esize)
{
    const int tpr = (nch + kTileChunks - 1) / kTileChunks;
    if (rows < 256 || tpr < 2 || rows * tpr < 2048) return false;
    // Two tiles of up to 24 chunks, 4- and 8-byte elements, forward: one workgroup of up to 12 waves per row is
    // faster (fp32, 34-48 chunks: 72 against 63 % of peak at 16 M elements, 78-80 against 76 % at 64 M; from 52
    // chunks on, and backward, the look-back kernel; 16-bit storage: the look-back kernel, 70 against 60-64 %).
    if (!rev && esize >= 4 && tpr == 2 && nch <= 48) return false;
    const int64_t rounds = (rows + kComputeUnits - 1) / kComputeUnits;
    const bool ragged_rounds = rows * 100 < rounds * kComputeUnits * 93;  // the row kernel's CUs idle > 7 % of the time
    if (rev && tpr <= 16) return true;
    if (tpr <= 15) return true;
    return ragged_rounds;
}

// Turns (shape, alignment, direction, optional user plan) into a launch. `aligned128` says whether every
// row of every tensor starts on a 128-byte line border; `aligned16` says
// whether every tensor base is 16-byte aligned.
int gcd_int(int a, int b) { return b == 0 ? a : gcd_int(b, a % b); }

// Rows the flat kernel can take of `rows` rows of length T: the largest count whose elements are a whole
// number of 16-byte vectors (the few rows left over go to the other kernels).
int64_t flat_rows(int64_t rows, int64_t T, int full) { return rows - rows % (full / gcd_int((int)(T % full), full)); }

// Short rows that start at any element, or whose vectors do not fill the SMALL kernel's power-of-two group of
// lanes: the flat kernel, where the tensors allow it (dense, 16-byte aligned bases). Measured at 32 M and 64 M
// elements, forward / backward, % of peak: fp32 flat 80-83 / 76-79 at every T from 4 to 256, SMALL the same
// where T / 4 is a power of two and 64-77 / 63-77 elsewhere (T = 70: 64 / 64, 132: 70 / 67, 36: 74 / 72); float64
// alike. 16-bit storage: flat 72-73 / 66-68 at every T (the three-component scan costs its instruction-bound
// backward pass 8-10 points), SMALL 70-77 / 68-78 on vector-aligned rows that fill at least 0.6 of their group,
// 57-68 / 55-67 otherwise (T = 100, 136, 264, 500).
bool prefer_flat(int64_t T, int full, int esize)
{
    if (T % full != 0) return true;
    const int nv = (int)(T / full), group = pow2_ceil(nv);
    if (esize == 2) return nv * 10 < group * 6;
    return nv != group;
}

// `flat_ok`: the tensors are dense [rows, T] arrays on 16-byte aligned bases (what the flat kernel needs).
int resolve(const scanscam_plan *user, int64_t rows, int64_t T, int dtype, bool aligned16, bool aligned128, bool rev,
            Resolved *out, bool flat_ok = false)
{
    const int esize = elem_size(dtype);
    if (esize == 0) return SCANSCAM_EDTYPE;
    if (rows < 0 || T < 0 || T >= kMaxT) return SCANSCAM_EINVAL;
    const int full = 16 / esize;
    scanscam_plan u = {0, 0, 0, 0, 0, 0};
    if (user) u = *user;

    Launch &l = out->l;
    l = Launch{0, 0, 0, 0, 1, 64, 0, false, 1};
    const bool flat_possible = flat_ok && T >= full && T <= (int64_t)kWave * full && flat_rows(rows, T, full) > 0;
    // Up to 32 MiB per tensor the flat kernel's larger workgroups (16 chunks each, a halo chunk and an LDS exchange
    // per workgroup) cost more than the few lanes it still fills gain: rows of four vectors or more stay with the small kernel's
    // element-aligned vectors there (fp32 [16513, 127] forward 9.2 -> 7.4 us, bf16 [33554, 250] 15.6 -> 12.7 us over 200
    // launches; [8224, 255], 64 vectors per row, 6.7 against 7.0 us; at 100 MB, [200000, 127], the flat kernel is
    // ahead, 49 against 58 us).
    // (Only where the rows fill nine tenths of their lane group: at bf16 [119837, 70], 9 vectors in 16 lanes, the flat
    // kernel is 15 / 38 % ahead at 16 MB too.)
    const int64_t row_vectors = (T + full - 1) / full;
    const bool small_problem = rows * T * esize <= (int64_t(1) << 25) && T >= 4 * full &&
                               row_vectors * 10 >= (int64_t)pow2_ceil((int)row_vectors) * 9;
    if (u.mode == kModeFlat ||
        (u.mode == SCANSCAM_MODE_AUTO && flat_possible && !u.vec && (u.unroll == 0 || u.unroll == 2 || u.unroll == 4) &&
         !small_problem && prefer_flat(T, full, esize))) {
        if (!flat_possible) return SCANSCAM_EPLAN;
        if (u.vec && u.vec != full) return SCANSCAM_EPLAN;
        l.mode = kModeFlat;
        l.vec = full;
        // 4 waves x 4 chunks; 16-bit storage (twice the registers per chunk) 8 waves x 2 chunks -- from 16 MiB per
        // tensor on: below, 4 x 4 there too (bf16 [119837, 70] forward 16.0 -> 14.3 us, [27962, 300] 12.7 -> 11.2 us).
        const bool halves = esize == 2 && rows * T * esize > (int64_t(1) << 24);
        l.unroll = u.unroll ? u.unroll : (halves ? 2 : 4);
        l.waves = u.waves ? u.waves : (halves ? 8 : 4);
        if ((l.unroll != 2 && l.unroll != 4) || l.waves < 1 || l.waves > scanscam::kMaxWaves) return SCANSCAM_EPLAN;
        out->nch = 1;
        out->tiles_per_row = 0;
        out->counters = 1;
        out->row_major = 0;
        out->line_shift = 0;
        out->super_base = 0;
        out->ws_bytes = 0;
        return SCANSCAM_OK;
    }
    // The full 16-byte vector needs rows that start on 16-byte borders -- or the element-aligned ("ragged")
    // variants of the kernels: ROW and LOOKBACK for rows of at least nine tenths of a chunk (on shorter rows
    // most of their lanes would idle), SMALL for rows of 4 vectors to one chunk (shorter ones lose nothing
    // with one element per lane).
    const bool vec_aligned = aligned16 && (T % full == 0);
    const bool small_rows = u.mode == kModeSmall || (u.mode == SCANSCAM_MODE_AUTO && T <= (int64_t)kWave * full);
    const bool ragged_possible = full > 1 && (small_rows ? (T >= 4 * full && T <= (int64_t)kWave * full)
                                                         : T * 10 >= (int64_t)kWave * full * 9);
    l.vec = u.vec ? u.vec : ((vec_aligned || ragged_possible) ? full : 1);
    if (l.vec != 1 && l.vec != full) return SCANSCAM_EPLAN;
    l.ragged = l.vec == full && full != 1 && !vec_aligned;
    if (l.ragged && !ragged_possible) return SCANSCAM_EPLAN;

    const int64_t chunk = (int64_t)kWave * l.vec;
    // Rows that start inside a 128-byte line, longer than one chunk: the ROW and LOOKBACK kernels lay their
    // chunks out from the line border before each row's start, so that a wave's loads and stores cover
    // whole lines (fp32 [23140, 2900], rows 16-byte aligned only: 129 / 220 us, 136 / 250 us without). A row
    // then takes up to one line's worth of vector slots more, which is not worth a fifth chunk for rows of
    // up to four (one wave per row: [67108, 1000] 128 us forward without, 150 with).
    // (Element-aligned rows: the border is counted in elements, and the vectors then sit on 16-byte borders.)
    const int64_t lead = l.ragged ? 128 / esize - 1 : 128 / ((int64_t)l.vec * esize) - 1;
    const int64_t nvec = l.ragged ? (T + lead + l.vec - 1) / l.vec : (T + l.vec - 1) / l.vec + lead;
    const int64_t nch_plain = (T + chunk - 1) / chunk, nch_lines = (nvec + kWave - 1) / kWave;
    // Rows of up to 4 chunks take one wave with 1, 2 or 4 chunks (2 or 4 when element-aligned): no shift
    // either where it would double that count and leave half the wave's slots empty (bf16 [33520, 1001], two
    // chunks: 38 / 57 us without the shift, 51 / 87 us with it in a wave of 4).
    // (Element-aligned 16-bit rows of three chunks take a wave of exactly three, below.)
    auto chunks_of_one_wave = [&](int64_t n) { return (l.ragged && esize == 2 && n == 3) ? 3 : pow2_ceil(l.ragged && n < 2 ? 2 : n); };
    const bool same_wave_shape =
        nch_plain > 4 || (nch_lines <= 4 && chunks_of_one_wave(nch_lines) == chunks_of_one_wave(nch_plain));
    out->line_shift = (!aligned128 && !small_rows && (T > chunk || l.ragged) && same_wave_shape) ? 1 : 0;
    const int64_t nch64 = out->line_shift ? nch_lines : nch_plain;
    const int nch = (int)nch64;
    out->nch = nch;
    out->tiles_per_row = 0;
    out->counters = 1;
    out->row_major = 0;
    out->super_base = 0;
    out->ws_bytes = 0;
    if (rows == 0 || T == 0) return SCANSCAM_OK;

    l.mode = u.mode;
    if (l.mode == SCANSCAM_MODE_AUTO) {
        if (T <= chunk) l.mode = kModeSmall;  // (line_shift is 0 here)
        // From 256 rows on, one 16-wave workgroup per row fills the chip as well as tiles over
        // workgroups do and needs no carry hand-off between workgroups.
        else if (nch >= 64 && rows < 256) l.mode = kModeLookback;
        else if (prefer_lookback_for_many_rows(rows, nch, rev, esize)) l.mode = kModeLookback;
        else l.mode = kModeRow;
    }

    if (l.mode == kModeSmall) {
        if (T > chunk) return SCANSCAM_EPLAN;
        l.group = pow2_ceil((T + l.vec - 1) / l.vec);
        l.unroll = u.unroll ? u.unroll : 4;
        l.waves = u.waves ? u.waves : 4;
        const int64_t rows_per_wg = (int64_t)l.waves * l.unroll * (kWave / l.group);
        l.grid = (rows + rows_per_wg - 1) / rows_per_wg;
    } else if (l.mode == kModeRow) {
        l.unroll = u.unroll;
        l.waves = u.waves;
        l.wpr = u.waves_per_row;
        if (!l.unroll && !l.waves && !l.wpr) {
            // Element-aligned rows of 16-bit storage that take 3 or 9 chunks: waves of exactly 3 chunks instead of 4
            // with a quarter of their slots empty. These kernels issue the most instructions per byte, and the
            // empty slots cost them their share: bf16 [65000, 1025] 58 / 67 -> 72 / 74 % of peak, [16380, 4097]
            // (9 chunks, 3 waves) 59-65 / 62-68 -> 73 / 73 %. fp32 and rows of whole vectors gain nothing from it
            // (fp32 [87000, 769] 79 / 75 -> 76 / 72 %, bf16 [43000, 1536] 79 / 78 either way).
            const bool threes = l.ragged && esize == 2 && l.vec == full;
            if (threes && nch == 3) {
                l.unroll = 3;
                l.wpr = 1;
                l.waves = 4;
            } else if (threes && nch == 9) {
                l.unroll = 3;
                l.wpr = l.waves = 3;
            } else if (nch <= 4) {
                l.unroll = (l.vec == full) ? pow2_ceil(nch) : (nch == 1 ? 1 : 4);
                l.wpr = 1;
                l.waves = 4;
            } else if (nch <= 16) {
                // 4 waves per workgroup. 5-6 chunks: 2 chunks per wave; 7-8: 4 chunks per wave and two
                // rows per workgroup (fp32 [32768, 2048] 122 / 211 us against 124 / 215 with 2 chunks per
                // wave and one row, bf16 [16384, 4096] 63.2 / 109.5 against 65.0 / 111.3); 9-16: one row.
                l.unroll = (l.vec == full && nch <= 6) ? 2 : 4;
                l.wpr = (l.vec == full && (nch == 7 || nch == 8)) ? 2 : 4;
                l.waves = 4;
                // Element-aligned rows of 9-12 chunks: 3 waves (bf16 [16380, 4097]: 76 / 123 us, 96 / 149 with 4);
                // of 5-6 chunks: 3 waves x 2 chunks (bf16 [16376, 2049]: 45 / 66 us, 55 / 82 with 4 waves;
                // fp32 [32736, 1025]: 69 / 110 against 76 / 110).
                if (l.ragged && nch > 8 && nch <= 12) l.wpr = l.waves = 3;
                if (l.ragged && nch >= 5 && nch <= 6) l.wpr = l.waves = 3;
            } else {
                // Longer rows: a workgroup tile (waves x 4 chunks) that covers the row in one step, or
                // in as few as 16 waves allow -- each further step waits for the carry of the last --
                // with just the waves those steps need: a row of 36 chunks takes 9 waves, not 8 waves
                // twice or 16 waves of which 7 idle (fp32 [7456, 9000]: 138 / 250 us against 145 / 258).
                // Few rows as well: fewer steps count for more than more waves per row ([300, 16640]:
                // 15.5 / 23.9 us with 9 waves x 4 chunks x 2 steps, 18.8 / 27.1 with 16 waves x 4 x 2).
                l.unroll = 4;
                const int steps = (nch + 63) / 64;
                l.wpr = l.waves = (nch + steps * 4 - 1) / (steps * 4);
                // 16-bit storage, 17-24 chunks (to 28 when element-aligned): two steps of half as many waves with
                // 2 chunks each. These kernels are as much bound by their instructions as by memory (unpacking,
                // 8 elements per lane and chunk), and with 2 chunks per wave they need half the registers, so
                // twice the waves cover each other: bf16 [3883, 8640] 41.5 / 63.6 us -> 35.1 / 59.4 us, element-
                // aligned [3297, 10175] 46.1 / 69.3 -> 35.9 / 60.8 us. From 32 chunks on the single step wins back.
                if (esize == 2 && l.vec == full && nch <= (l.ragged ? 28 : 24)) {
                    l.unroll = 2;
                    l.wpr = l.waves = (nch + 3) / 4;
                }
            }
        } else {
            if (!l.unroll) l.unroll = 4;
            if (!l.waves) l.waves = l.wpr ? l.wpr : 4;
            if (!l.wpr) l.wpr = l.waves;
        }
        if (l.wpr < 1 || l.wpr > l.waves || l.waves % l.wpr != 0) return SCANSCAM_EPLAN;
        const int rows_per_wg = l.waves / l.wpr;
        l.grid = (rows + rows_per_wg - 1) / rows_per_wg;
    } else if (l.mode == kModeLookback) {
        // Tiles of 32 chunks (8192 fp32 elements): fewer, larger tiles keep the wait for the
        // carry short relative to the time a tile spends on its data. With very few rows the
        // tiles in flight are neighbours in one row, which publish almost together and so wait
        // longest for each other: 64 chunks there (up to 8 rows: forward +1 to +4 points of peak at
        // 2^26 fp32 elements; from 12 rows on the 32-chunk tile is 4 to 6 points faster).
        l.unroll = u.unroll ? u.unroll : 4;
        l.waves = u.waves ? u.waves : (rows <= 8 && l.unroll <= 4 ? 16 : 8);
        // Forward fp32 with up to 16 rows: the 64-chunk tile as 8 waves of 8 chunks (two workgroups per CU
        // instead of one of 16 waves): [1, 2^26] 61 -> 64 % of peak, [16, 2^22] 64 -> 66 %, [8, 2^21] 53 -> 57 %;
        // the backward pass gains nothing from it, 16-bit storage with 2 to 8 rows (bf16 [8, 2^22] 50 -> 43 us,
        // [4, 2^23] 48 -> 46 us, [2, 2^24] 49 -> 46 us; [1, 2^26] level, [16, 2^21] 47 -> 51 us).
        // (fp32 with 17 to 64 rows likewise while the whole problem is 8 M elements or less, i.e. up to 512 such tiles:
        // [32, 262144] forward 26.1 -> 20.0 us, [64, 131072] 25.4 -> 21.4 us; at 32 M elements the 32-chunk tile is level.)
        const bool few_tiles = esize == 4 && rows > 16 && rows <= 64 && rows * (int64_t)nch <= 32768;
        if (!u.waves && !u.unroll && !rev && l.vec == full && !l.ragged &&
            (esize == 4 ? (rows <= 16 || few_tiles) : (esize == 2 && rows >= 2 && rows <= 8))) {
            l.unroll = 8;
            l.waves = 8;
        }
        if (!u.waves && !u.unroll && rows > 8 && !(few_tiles && l.unroll == 8)) {
            // As many tiles as 8-wave tiles would take, but with only the waves they need: 75 chunks are 3
            // tiles of 7 waves (84 chunk slots), not of 8 (96).
            int tiles = (nch + kTileChunks - 1) / kTileChunks;
            // Element-aligned rows of 16-bit storage up to 96 chunks: tiles of up to 16 chunks (3-4 waves). Their
            // waves do more arithmetic per byte (components of partial vectors moved into place, masks per
            // element), and the smaller workgroups cover each other better: bf16 [2013, 33333] 55 / 58 -> 62 / 66 %
            // of peak, [3947, 17001] 59 / 63 -> 65 / 68 %, [1973, 34001] 61 / 62 -> 63 / 67 %; from 190 chunks on
            // the larger tile is 3-4 points faster, and rows of whole vectors keep it throughout.
            if (l.ragged && esize == 2 && nch <= 96) tiles = (nch + kTileChunks / 2 - 1) / (kTileChunks / 2);
            l.waves = (nch + tiles * l.unroll - 1) / (tiles * l.unroll);
        }
        const int tile_chunks = l.waves * l.unroll;
        out->tiles_per_row = (nch + tile_chunks - 1) / tile_chunks;
        // One ticket counter per row up to kMaxCounters; when rows do not divide
        // evenly every counter gets the grid share of the fullest one.
        out->counters = (int)(rows < kMaxCounters ? rows : kMaxCounters);
        // Row-major order: a few counters, so that their rows stay neighbours in memory.
        out->row_major = row_major_order(rows, out->tiles_per_row) ? 1 : 0;
        if (out->row_major) out->counters = kRowMajorCounters;
        const int64_t rows_per_counter = (rows + out->counters - 1) / out->counters;
        const int64_t tiles = rows * (int64_t)out->tiles_per_row;
        l.grid = (int64_t)out->counters * rows_per_counter * out->tiles_per_row;
        if (l.grid >= (int64_t(1) << 31)) return SCANSCAM_EINVAL;
        const int64_t supers = rows * (int64_t)((out->tiles_per_row + kSuper - 1) / kSuper);
        out->super_base = (int64_t)out->counters * kCounterStride + tiles * tile_words(dtype);
        out->ws_bytes = (size_t)(out->super_base + supers * super_words(dtype)) * sizeof(uint64_t);
    } else {
        return SCANSCAM_EPLAN;
    }

    if (l.ragged) {
        if (!u.unroll && l.unroll < 2) l.unroll = 2;  // instantiated for 2, 3 and 4 chunks per wave
        if (l.unroll != 2 && l.unroll != 3 && l.unroll != 4) return SCANSCAM_EPLAN;
    }
    if (!unroll_ok(l.vec, full, l.unroll)) return SCANSCAM_EPLAN;
    if (l.waves < 1 || l.waves > scanscam::kMaxWaves ||
        l.waves * kWave > scanscam::max_threads_for_unroll(l.unroll))
        return SCANSCAM_EPLAN;
    if (l.grid >= (int64_t(1) << 31)) return SCANSCAM_EINVAL;
    return SCANSCAM_OK;
}

bool aligned_to(const void *p, size_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; }

// Address of `scratch` on the current device: looked up once per device, with that device current
// (every GPU holds its own copy of the array at its own address), and kept.
constexpr int kMaxDevices = 64;
int noalloc_scratch(void **out)
{
    static std::mutex lock;
    static void *ptr[kMaxDevices];  // zero-initialised: not looked up yet
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SCANSCAM_ELAUNCH;
    std::lock_guard<std::mutex> hold(lock);
    if (!ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return SCANSCAM_ELAUNCH;
        ptr[dev] = p;
    }
    *out = ptr[dev];
    return SCANSCAM_OK;
}

const scanscam_strides *const kDense[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};

// Tensor order everywhere below: a, x, h, y0, y1 (x = b forwards, gh backwards; y0 = h forwards,
// gb backwards; h and y1 = ga exist only backwards). st[k] == nullptr means dense.
int run(bool rev, const void *a, const void *x, const void *h, void *y0, void *y1,
        const scanscam_strides *const st[5], int64_t n0, int64_t n1, int64_t T, int dtype, void *workspace,
        size_t workspace_bytes, void *stream, const scanscam_plan *plan, void *start_event = nullptr,
        void *stop_event = nullptr, bool use_scratch = false, bool allow_flat = true)
{
    const int esize = elem_size(dtype);
    if (esize == 0) return SCANSCAM_EDTYPE;
    if (n0 < 0 || n1 < 0 || T < 0 || T >= kMaxT) return SCANSCAM_EINVAL;
    if (n0 == 0 || n1 == 0 || T == 0) return SCANSCAM_OK;
    if (n1 > INT64_MAX / n0) return SCANSCAM_EINVAL;
    const int64_t rows = n0 * n1;
    if (!a || !x || !y0 || (rev && (!h || !y1))) return SCANSCAM_EINVAL;

    const void *ptrs[5] = {a, x, rev ? h : a, y0, rev ? y1 : y0};
    const bool used[5] = {true, true, rev, true, rev};
    int64_t s0[5], s1[5];
    for (int k = 0; k < 5; k++) {
        const scanscam_strides *t = used[k] ? st[k] : nullptr;
        s0[k] = t ? t->outer : n1 * T;
        s1[k] = t ? t->row : T;
        if (s0[k] < 0 || s1[k] < 0) return SCANSCAM_EINVAL;
    }
    // Rows are independent, so the two levels may be merged or exchanged freely as long as every
    // tensor is walked the same way: one level when the groups follow each other at the row stride,
    // otherwise the longer level inside (the kernels spread the inner level over blockIdx.x).
    if (n1 == 1) {
        n1 = n0;
        n0 = 1;
        for (int k = 0; k < 5; k++) s1[k] = s0[k];
    }
    bool one_level = true;
    for (int k = 0; k < 5; k++) one_level = one_level && (!used[k] || s0[k] == n1 * s1[k]);
    if (n0 > 1 && one_level) {
        n1 = rows;
        n0 = 1;
    }
    if (n0 > n1) {
        for (int k = 0; k < 5; k++) {
            const int64_t t = s0[k];
            s0[k] = s1[k];
            s1[k] = t;
        }
        const int64_t t = n0;
        n0 = n1;
        n1 = t;
    }
    for (int k = 0; k < 5; k++) {
        if (n0 == 1) s0[k] = 0;
        if (n1 == 1) s1[k] = 0;
    }

    // 16-byte vectors need every row of every tensor to start on a 16-byte border.
    const int full = 16 / esize;
    bool aligned16 = true, aligned128 = true;
    const int line = 128 / esize;  // elements per 128-byte line
    for (int k = 0; k < 5; k++) {
        if (!used[k]) continue;
        if (!aligned_to(ptrs[k], (size_t)esize)) return SCANSCAM_EALIGN;
        aligned16 = aligned16 && aligned_to(ptrs[k], 16) && s0[k] % full == 0 && s1[k] % full == 0;
        aligned128 = aligned128 && aligned_to(ptrs[k], 128) && s0[k] % line == 0 && s1[k] % line == 0;
    }

    // The flat kernel takes dense [rows, T] tensors on 16-byte aligned bases (rows of any length).
    bool flat_ok = allow_flat && n0 == 1;
    for (int k = 0; k < 5; k++) flat_ok = flat_ok && (!used[k] || (aligned_to(ptrs[k], 16) && (n1 == 1 || s1[k] == T)));
    // The flat kernel's workgroups read a halo of their neighbours' spans (and a[e+1] / h[e-1] across span
    // borders backwards), so an output that shares bytes with an input -- an in-place call, which every other
    // kernel family allows because it reads only what it is about to write -- would race there.
    if (flat_ok) {
        const int64_t bytes = rows * T * esize;
        auto overlaps = [&](const void *p, const void *q) {
            const char *pc = static_cast<const char *>(p), *qc = static_cast<const char *>(q);
            return pc < qc + bytes && qc < pc + bytes;
        };
        for (int o = 3; o < 5; o++)
            for (int i = 0; i < 3; i++)
                if (used[o] && used[i] && overlaps(ptrs[o], ptrs[i])) flat_ok = false;
    }
    // One pair of events cannot bracket the flat launch and the launch for the rows it leaves over.
    if ((start_event || stop_event) && flat_rows(rows, T, full) != rows) flat_ok = false;

    Resolved r;
    const int rc = resolve(plan, rows, T, dtype, aligned16, aligned128, rev, &r, flat_ok);
    if (rc != SCANSCAM_OK) return rc;

    if (r.l.mode == kModeFlat) {
        const int64_t taken = flat_rows(rows, T, full);
        scanscam::FlatArgs fa;
        fa.a = a;
        fa.x = x;
        fa.h = h;
        fa.y0 = y0;
        fa.y1 = y1;
        fa.N = taken * T;
        fa.T = (int32_t)T;
        hipStream_t fs = static_cast<hipStream_t>(stream);
        hipEvent_t e0 = static_cast<hipEvent_t>(start_event), e1 = static_cast<hipEvent_t>(stop_event);
        hipError_t e = hipErrorInvalidValue;
        switch (dtype) {
        case SCANSCAM_F32: e = scanscam::launch_scan_flat<float>(fa, r.l.unroll, r.l.waves, rev, fs, e0, e1); break;
        case SCANSCAM_BF16: e = scanscam::launch_scan_flat<__bf16>(fa, r.l.unroll, r.l.waves, rev, fs, e0, e1); break;
        case SCANSCAM_F16: e = scanscam::launch_scan_flat<_Float16>(fa, r.l.unroll, r.l.waves, rev, fs, e0, e1); break;
        case SCANSCAM_F64: e = scanscam::launch_scan_flat<double>(fa, r.l.unroll, r.l.waves, rev, fs, e0, e1); break;
        }
        if (e != hipSuccess) return SCANSCAM_ELAUNCH;
        if (taken == rows) return SCANSCAM_OK;
        // The few rows left over (fewer than a vector has elements): the other kernels, on the tail of every tensor.
        const int64_t off = taken * T * esize;
        auto tail = [&](const void *q) { return q ? static_cast<const void *>(static_cast<const char *>(q) + off) : nullptr; };
        return run(rev, tail(a), tail(x), tail(h), const_cast<void *>(tail(y0)), const_cast<void *>(tail(y1)), kDense, 1,
                   rows - taken, T, dtype, workspace, workspace_bytes, stream, nullptr, nullptr, nullptr, use_scratch,
                   /*allow_flat=*/false);
    }

    ScanArgs args;
    args.a = a;
    args.x = x;
    args.h = h;
    args.y0 = y0;
    args.y1 = y1;
    for (int k = 0; k < 5; k++) {
        args.s0[k] = s0[k];
        args.s1[k] = s1[k];
    }
    args.rows = rows;
    args.n1 = n1;
    args.T = (int32_t)T;
    args.nch = r.nch;
    args.wpr = r.l.wpr;
    args.group = r.l.group;
    args.tiles_per_row = r.tiles_per_row;
    args.counters = r.counters;
    args.row_major = r.row_major;
    args.line_shift = r.line_shift;
    args.desc_base = r.counters * kCounterStride;
    args.super_base = r.super_base;
    args.spin_limit = (plan && plan->spin_limit > 0) ? plan->spin_limit : scanscam::kSpinLimit;
    args.ws = nullptr;

    hipStream_t s = static_cast<hipStream_t>(stream);
    // The caller's events, if any, are bound to the scan kernel itself (its start and end on the GPU).
    hipEvent_t ev0 = static_cast<hipEvent_t>(start_event), ev1 = static_cast<hipEvent_t>(stop_event);
    const bool timed = ev0 || ev1;
    auto launch = [&](const ScanArgs &la, const Launch &l) {
        switch (dtype) {
        case SCANSCAM_F32: return scanscam::launch_scan<float>(la, l, rev, s, ev0, ev1);
        case SCANSCAM_BF16: return scanscam::launch_scan<__bf16>(la, l, rev, s, ev0, ev1);
        case SCANSCAM_F16: return scanscam::launch_scan<_Float16>(la, l, rev, s, ev0, ev1);
        case SCANSCAM_F64: return scanscam::launch_scan<double>(la, l, rev, s, ev0, ev1);
        default: return hipErrorInvalidValue;
        }
    };

    if (r.l.mode == kModeLookback) {
        if (use_scratch) {
            // The library's own fixed array instead of a caller's workspace; every call clears the part
            // it uses (below), whatever the call before left there.
            if (r.ws_bytes > (size_t)SCANSCAM_NOALLOC_SCRATCH_BYTES) return SCANSCAM_ESCRATCH;
            const int src = noalloc_scratch(&workspace);
            if (src != SCANSCAM_OK) return src;
            workspace_bytes = SCANSCAM_NOALLOC_SCRATCH_BYTES;
        }
        if (!workspace || workspace_bytes < r.ws_bytes) return SCANSCAM_EWORKSPACE;
        if (!aligned_to(workspace, 8)) return SCANSCAM_EALIGN;
        args.ws = static_cast<uint64_t *>(workspace);
        const int64_t words = (int64_t)(r.ws_bytes / sizeof(uint64_t));
        if (clear_workspace(args.ws, words, args.desc_base, s) != hipSuccess) return SCANSCAM_ELAUNCH;
        // One launch over all rows; the kernel splits a row index into (group, row). Its grid is far
        // below every launch limit by construction.
        return launch(args, r.l) == hipSuccess ? SCANSCAM_OK : SCANSCAM_ELAUNCH;
    }

    // ROW and SMALL: blockIdx.x walks the n1 rows of a group, blockIdx.y the n0 groups. One launch
    // may hold at most 2^32 - 1 threads and 65535 groups; rows are independent, so a larger problem
    // is issued as several launches over consecutive slabs (only tensors of tens of GB get there).
    const int64_t threads = (int64_t)r.l.waves * kWave;
    const int64_t max_grid = ((int64_t(1) << 32) - 1) / threads;
    int64_t rows_per_wg = 1;
    if (r.l.mode == kModeRow) rows_per_wg = r.l.waves / r.l.wpr;
    if (r.l.mode == kModeSmall) rows_per_wg = (int64_t)r.l.waves * r.l.unroll * (kWave / r.l.group);
    const int64_t grid_x_all = (n1 + rows_per_wg - 1) / rows_per_wg;
    const int64_t slab_rows = grid_x_all <= max_grid ? n1 : max_grid * rows_per_wg;
    if (timed && (grid_x_all > max_grid || n0 > 65535 || n0 * grid_x_all > max_grid))
        return SCANSCAM_EINVAL;  // several launches: one pair of events cannot bracket them

    for (int64_t row0 = 0; row0 < n1; row0 += slab_rows) {
        const int64_t n = n1 - row0 < slab_rows ? n1 - row0 : slab_rows;
        const int64_t grid_x = (n + rows_per_wg - 1) / rows_per_wg;
        int64_t slab_groups = max_grid / grid_x;
        if (slab_groups > 65535) slab_groups = 65535;
        if (slab_groups < 1) slab_groups = 1;
        for (int64_t g0 = 0; g0 < n0; g0 += slab_groups) {
            ScanArgs slab = args;
            Launch l = r.l;
            const void **in[3] = {&slab.a, &slab.x, &slab.h};
            void **out[2] = {&slab.y0, &slab.y1};
            for (int k = 0; k < 5; k++) {
                const int64_t byte_off = (g0 * s0[k] + row0 * s1[k]) * esize;
                if (k < 3 && *in[k]) *in[k] = static_cast<const char *>(*in[k]) + byte_off;
                if (k >= 3 && *out[k - 3]) *out[k - 3] = static_cast<char *>(*out[k - 3]) + byte_off;
            }
            slab.rows = n;
            l.grid = grid_x;
            l.grid_y = (int)(n0 - g0 < slab_groups ? n0 - g0 : slab_groups);
            if (launch(slab, l) != hipSuccess) return SCANSCAM_ELAUNCH;
        }
    }
    return SCANSCAM_OK;
}

// Channels-last: the launch plan. `align`: the largest of 16, 8, 4 and the element size that every tensor's base
// and strides are multiples of (bytes). The choice itself is the cost model of scan_cl_plan.hpp: every field the
// caller's plan leaves at zero is chosen by the smallest estimated duration; this function turns the chosen
// candidate into launch parameters and sizes.
int resolve_cl(const scanscam_plan *user, int64_t batch, int64_t T, int64_t C, int dtype, int align, bool rev,
               scanscam::ClLaunch *l, double *predicted_us = nullptr)
{
    const int esize = elem_size(dtype);
    if (esize == 0) return SCANSCAM_EDTYPE;
    scanscam_plan u = {0, 0, 0, 0, 0, 0};
    if (user) u = *user;
    if (u.mode != SCANSCAM_MODE_AUTO && u.mode != kModeRow && u.mode != kModeLookback) return SCANSCAM_EPLAN;
    const scanscam::ClShape shape = {batch, T, C, esize, compute_size(dtype), align, rev};
    scanscam::ClCandidate c;
    // The choice is a pure function of (shape, caller's plan) and costs about a hundred microseconds (some forty
    // candidates through the cost model), so each thread remembers its last few dozen: a model calls the same shapes
    // over and over. Nothing but speed depends on it.
    struct Remembered {
        bool valid;
        int64_t batch, T, C;
        int dtype, align;
        bool rev;
        int32_t mode, vec, unroll, waves;
        scanscam::ClCandidate c;
        double us;
    };
    constexpr int kRemembered = 64;
    static thread_local Remembered remembered[kRemembered] = {};
    const uint64_t key = (uint64_t)batch * 0x9E3779B97F4A7C15ull ^ (uint64_t)T * 0xC2B2AE3D27D4EB4Full ^ (uint64_t)C * 0x165667B19E3779F9ull ^
                         (uint64_t)(dtype * 64 + align * 2 + (rev ? 1 : 0)) * 0x27D4EB2F165667C5ull ^
                         (uint64_t)(u.mode * 4096 + u.vec * 256 + u.unroll * 16 + u.waves);
    Remembered &slot = remembered[(key >> 32 ^ key) % kRemembered];
    if (slot.valid && slot.batch == batch && slot.T == T && slot.C == C && slot.dtype == dtype && slot.align == align &&
        slot.rev == rev && slot.mode == u.mode && slot.vec == u.vec && slot.unroll == u.unroll && slot.waves == u.waves) {
        c = slot.c;
        if (predicted_us) *predicted_us = slot.us;
    } else {
        double us = 0.0;
        if (!scanscam::cl_choose(shape, u, &c, &us)) return SCANSCAM_EPLAN;
        slot = Remembered{true, batch, T, C, dtype, align, rev, u.mode, u.vec, u.unroll, u.waves, c, us};
        if (predicted_us) *predicted_us = us;
    }

    l->vec = c.vec;
    l->steps = c.steps;
    l->waves = c.waves;
    l->kind = c.kind;
    l->group = c.group;
    l->ragged = c.ragged;
    const int64_t rowgroups = batch * scanscam::cl_groups(C, c.vec);
    const int64_t tile_steps = (int64_t)l->waves * l->steps;
    const int64_t tiles = (T + tile_steps - 1) / tile_steps;
    const int64_t vals = (int64_t)l->vec * kWave * value_words(dtype);  // words of one [vec][64] array of values
    l->lds_bytes = (size_t)(l->kind == 2 ? 7 : 4) * l->waves * l->vec * kWave * compute_size(dtype);
    l->ws_bytes = 0;
    l->segments = 1;
    if (l->kind == 2) {
        if (tiles >= (int64_t(1) << 31)) return SCANSCAM_EINVAL;
        l->segments = (int)tiles;  // the kernel's tiles per row-group
        const int64_t supers = (tiles + l->waves - 1) / l->waves;
        const int64_t pairs = (int64_t)l->vec * kWave * tile_words(dtype);  // words of one [vec][64] array of pairs
        l->ws_bytes = (size_t)(rowgroups * kCounterStride + rowgroups * tiles * pairs + rowgroups * supers * (pairs + vals)) *
                      sizeof(uint64_t);
    }
    if (l->segments <= 1) {  // a forced time split of a single tile: nothing to split after all
        l->kind = 0;
        l->ws_bytes = 0;
    }
    l->grid = rowgroups * l->segments;
    if (l->grid >= (int64_t(1) << 31)) return SCANSCAM_EINVAL;
    return SCANSCAM_OK;
}

int run_cl(bool rev, const void *a, const void *x, const void *h, void *y0, void *y1,
           const scanscam_strides *const st[5], int64_t batch, int64_t T, int64_t C, int dtype, void *workspace,
           size_t workspace_bytes, void *stream, const scanscam_plan *plan)
{
    const int esize = elem_size(dtype);
    if (esize == 0) return SCANSCAM_EDTYPE;
    if (batch < 0 || T < 0 || C < 0 || T >= kMaxT || C >= kMaxT) return SCANSCAM_EINVAL;
    if (batch == 0 || T == 0 || C == 0) return SCANSCAM_OK;
    if (!a || !x || !y0 || (rev && (!h || !y1))) return SCANSCAM_EINVAL;

    // Tensor order a, x, h, y0, y1; the forward pass has no h and no y1 (they alias a and y0).
    const void *ptrs[5] = {a, x, rev ? h : a, y0, rev ? y1 : y0};
    const int src[5] = {0, 1, rev ? 2 : 0, 3, rev ? 4 : 3};
    int64_t sB[5], sT[5];
    int align = 16;  // bytes every base and stride is a multiple of: 16, 8, 4 or the element size
    for (int k = 0; k < 5; k++) {
        const scanscam_strides *t = st[src[k]];
        sB[k] = batch == 1 ? 0 : (t ? t->outer : T * C);
        sT[k] = T == 1 ? 0 : (t ? t->row : C);
        if (sB[k] < 0 || sT[k] < 0 || sT[k] >= kMaxT) return SCANSCAM_EINVAL;
        if (!aligned_to(ptrs[k], (size_t)esize)) return SCANSCAM_EALIGN;
        while (align > esize && !(aligned_to(ptrs[k], (size_t)align) && (sB[k] * esize) % align == 0 && (sT[k] * esize) % align == 0))
            align >>= 1;
    }
    scanscam::ClLaunch l;
    const int rc = resolve_cl(plan, batch, T, C, dtype, align, rev, &l);
    if (rc != SCANSCAM_OK) return rc;
    // A wave addresses its steps (at most 16, and one neighbour on either side backwards) with 32-bit byte
    // offsets from its first one, the lane's channel included.
    for (int k = 0; k < 5; k++)
        if ((uint64_t)sT[k] * (uint64_t)esize * 18u + (uint64_t)C * (uint64_t)esize >= (uint64_t(1) << 32)) return SCANSCAM_EINVAL;

    scanscam::ClArgs args;
    args.a = a;
    args.x = x;
    args.h = rev ? h : a;  // never read in the forward pass
    args.y0 = y0;
    args.y1 = rev ? y1 : y0;
    for (int k = 0; k < 5; k++) {
        args.sB[k] = sB[k];
        args.sT[k] = (int32_t)sT[k];
    }
    args.batch = batch;
    args.T = (int32_t)T;
    args.C = (int32_t)C;
    args.segments = l.segments;
    args.group = l.group;
    // Time steps that are not whole 128-byte lines: neighbouring channel groups on one XCD (see the kernel).
    bool lines = true;
    for (int k = 0; k < 5; k++) lines = lines && (sT[k] * esize) % 128 == 0 && aligned_to(ptrs[k], 128) && (sB[k] * esize) % 128 == 0;
    args.xcd_order = (!lines && l.grid >= 64) ? 1 : 0;
    // Tiles over workgroups: a (batch element, channel group) pair keeps its XCD over all its tiles when their number
    // is a multiple of 8. Otherwise, from 128 pairs on, the XCDs take runs of n / 8 rounded up or down and the grid is
    // padded to 8 equal shares; the workgroups of a short run's last share return at once. (fp32 [9, 5318, 2059], 297
    // pairs dealt round-robin over the XCDs tile by tile: 401 / 706 us.)
    if (args.xcd_order && l.kind == 2) {
        const int64_t pairs = l.grid / l.segments;
        if (pairs % 8 != 0 && pairs >= 128) {
            args.xcd_order = 2;
            l.grid = 8 * ((pairs + 7) / 8) * l.segments;
            if (l.grid >= (int64_t(1) << 31)) return SCANSCAM_EINVAL;
        }
    }
    // Lanes of 8 bytes or less whose time steps are no whole lines write partial lines at both ends of every
    // wave's store; non-temporal stores then cost 20 % of a plain copy's rate and stores left to the caches'
    // normal policy nothing. Measured on the kernels: 16-bit storage 8 to 35 % faster in both directions (bf16
    // [90, 2048, 514] 178 / 341 -> 139 / 298 us, [1000, 500, 130] 157 / 296 -> 120 / 202 us, [700, 300, 257] 112 / 217 ->
    // 85 / 141 us; single channels backwards lose 10 %: [260, 4000, 48]), fp32 forwards and in tiles over workgroups
    // 4 to 19 % ([8, 4096, 1000] 90 / 152 -> 83 / 128 us, [100, 3000, 300] forward 339 -> 276 us; a walk of all of T
    // backwards loses up to 11 %); on whole lines they lose 6 to 14 %, and 16-byte lanes lose 6 to 11 % either way.
    // (Element-aligned lanes of 8 bytes or less always store this way: the kernel's choice, not this flag's.)
    const int lane_bytes = l.vec * esize;
    args.cached_stores = (!lines && lane_bytes <= 8 && esize <= 4 &&
                          (esize == 2 ? (lane_bytes > 2 || !rev) : (!rev || l.kind == 2))) ? 1 : 0;
    args.ws = nullptr;
    args.spin_limit = (plan && plan->spin_limit > 0) ? plan->spin_limit : scanscam::kSpinLimit;

    hipStream_t s = static_cast<hipStream_t>(stream);
    if (l.kind != 0) {
        if (!workspace || workspace_bytes < l.ws_bytes) return SCANSCAM_EWORKSPACE;
        if (!aligned_to(workspace, 8)) return SCANSCAM_EALIGN;
        args.ws = static_cast<uint64_t *>(workspace);
        const int64_t words = (int64_t)(l.ws_bytes / sizeof(uint64_t));
        const int64_t rowgroups = batch * ((C + (int64_t)kWave * l.vec - 1) / ((int64_t)kWave * l.vec));
        if (clear_workspace(args.ws, words, rowgroups * kCounterStride, s) != hipSuccess) return SCANSCAM_ELAUNCH;
    }
    hipError_t e = hipErrorInvalidValue;
    switch (dtype) {
    case SCANSCAM_F32: e = scanscam::launch_scan_cl<float>(args, l, rev, s); break;
    case SCANSCAM_BF16: e = scanscam::launch_scan_cl<__bf16>(args, l, rev, s); break;
    case SCANSCAM_F16: e = scanscam::launch_scan_cl<_Float16>(args, l, rev, s); break;
    case SCANSCAM_F64: e = scanscam::launch_scan_cl<double>(args, l, rev, s); break;
    }
    return e == hipSuccess ? SCANSCAM_OK : SCANSCAM_ELAUNCH;
}

size_t workspace_for(int64_t rows, int64_t T, int dtype, int direction, const scanscam_plan *plan)
{
    // The caller's pointers are not known yet: cover both the 16-byte aligned
    // and the unaligned choice.
    size_t need = 0;
    for (int al = 0; al < 3; al++) {  // element-aligned, 16-byte aligned, 128-byte aligned rows
        Resolved r;
        if (resolve(plan, rows, T, dtype, al >= 1, al == 2, direction == SCANSCAM_BACKWARD, &r) == SCANSCAM_OK &&
            r.ws_bytes > need)
            need = r.ws_bytes;
    }
    return need;
}

}  // namespace

extern "C" {

int scanscam_scan_fwd(const void *a, const void *b, void *h, int64_t rows, int64_t T, int dtype,
                      void *workspace, size_t workspace_bytes, void *stream)
{
    return run(false, a, b, nullptr, h, nullptr, kDense, 1, rows, T, dtype, workspace, workspace_bytes, stream, nullptr);
}

int scanscam_scan_bwd(const void *a, const void *h, const void *gh, void *ga, void *gb, int64_t rows,
                      int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream)
{
    return run(true, a, gh, h, gb, ga, kDense, 1, rows, T, dtype, workspace, workspace_bytes, stream, nullptr);
}

int scanscam_scan_fwd_noalloc(const void *a, const void *b, void *h, int64_t rows, int64_t T, int dtype, void *stream)
{
    return run(false, a, b, nullptr, h, nullptr, kDense, 1, rows, T, dtype, nullptr, 0, stream, nullptr, nullptr, nullptr,
               /*use_scratch=*/true);
}

size_t scanscam_workspace_bytes(int64_t rows, int64_t T, int dtype, int direction)
{
    return workspace_for(rows, T, dtype, direction, nullptr);
}

int scanscam_scan_fwd_plan(const void *a, const void *b, void *h, int64_t rows, int64_t T, int dtype,
                           void *workspace, size_t workspace_bytes, void *stream, const scanscam_plan *plan)
{
    return run(false, a, b, nullptr, h, nullptr, kDense, 1, rows, T, dtype, workspace, workspace_bytes, stream, plan);
}

int scanscam_scan_bwd_plan(const void *a, const void *h, const void *gh, void *ga, void *gb, int64_t rows,
                           int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                           const scanscam_plan *plan)
{
    return run(true, a, gh, h, gb, ga, kDense, 1, rows, T, dtype, workspace, workspace_bytes, stream, plan);
}

size_t scanscam_workspace_bytes_plan(int64_t rows, int64_t T, int dtype, int direction,
                                     const scanscam_plan *plan)
{
    return workspace_for(rows, T, dtype, direction, plan);
}

int scanscam_scan_fwd_timed(const void *a, const void *b, void *h, int64_t rows, int64_t T, int dtype,
                            void *workspace, size_t workspace_bytes, void *stream, const scanscam_plan *plan,
                            void *start_event, void *stop_event)
{
    return run(false, a, b, nullptr, h, nullptr, kDense, 1, rows, T, dtype, workspace, workspace_bytes, stream, plan,
               start_event, stop_event);
}

int scanscam_scan_bwd_timed(const void *a, const void *h, const void *gh, void *ga, void *gb, int64_t rows,
                            int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                            const scanscam_plan *plan, void *start_event, void *stop_event)
{
    return run(true, a, gh, h, gb, ga, kDense, 1, rows, T, dtype, workspace, workspace_bytes, stream, plan, start_event,
               stop_event);
}

int scanscam_scan_fwd_cl(const void *a, const void *b, void *h, int64_t batch, int64_t T, int64_t C, int dtype,
                         void *workspace, size_t workspace_bytes, void *stream, const scanscam_plan *plan)
{
    return run_cl(false, a, b, nullptr, h, nullptr, kDense, batch, T, C, dtype, workspace, workspace_bytes, stream, plan);
}

int scanscam_scan_bwd_cl(const void *a, const void *h, const void *gh, void *ga, void *gb, int64_t batch,
                         int64_t T, int64_t C, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                         const scanscam_plan *plan)
{
    return run_cl(true, a, gh, h, gb, ga, kDense, batch, T, C, dtype, workspace, workspace_bytes, stream, plan);
}

size_t scanscam_workspace_bytes_cl(int64_t batch, int64_t T, int64_t C, int dtype, int direction,
                                   const scanscam_plan *plan)
{
    const int esize = elem_size(dtype);
    if (esize == 0 || batch <= 0 || T <= 0 || C <= 0 || T >= kMaxT || C >= kMaxT) return 0;
    size_t need = 0;
    // The caller's pointers are not known yet: every alignment the tensors may turn out to have.
    for (int align = 16; align >= esize; align >>= 1) {
        scanscam::ClLaunch l;
        if (resolve_cl(plan, batch, T, C, dtype, align, direction == SCANSCAM_BACKWARD, &l) == SCANSCAM_OK && l.ws_bytes > need)
            need = l.ws_bytes;
    }
    return need;
}

int scanscam_scan_fwd_strided(const void *a, const void *b, void *h, const scanscam_strides *sa,
                              const scanscam_strides *sb, const scanscam_strides *sh, int64_t n0, int64_t n1,
                              int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                              const scanscam_plan *plan)
{
    const scanscam_strides *const st[5] = {sa, sb, nullptr, sh, nullptr};
    return run(false, a, b, nullptr, h, nullptr, st, n0, n1, T, dtype, workspace, workspace_bytes, stream, plan);
}

int scanscam_scan_bwd_strided(const void *a, const void *h, const void *gh, void *ga, void *gb,
                              const scanscam_strides *sa, const scanscam_strides *sh, const scanscam_strides *sgh,
                              const scanscam_strides *sga, const scanscam_strides *sgb, int64_t n0, int64_t n1,
                              int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                              const scanscam_plan *plan)
{
    const scanscam_strides *const st[5] = {sa, sgh, sh, sgb, sga};
    return run(true, a, gh, h, gb, ga, st, n0, n1, T, dtype, workspace, workspace_bytes, stream, plan);
}

int scanscam_scan_fwd_cl_strided(const void *a, const void *b, void *h, const scanscam_strides *sa,
                                 const scanscam_strides *sb, const scanscam_strides *sh, int64_t batch, int64_t T,
                                 int64_t C, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                                 const scanscam_plan *plan)
{
    const scanscam_strides *const st[5] = {sa, sb, nullptr, sh, nullptr};
    return run_cl(false, a, b, nullptr, h, nullptr, st, batch, T, C, dtype, workspace, workspace_bytes, stream, plan);
}

int scanscam_scan_bwd_cl_strided(const void *a, const void *h, const void *gh, void *ga, void *gb,
                                 const scanscam_strides *sa, const scanscam_strides *sh,
                                 const scanscam_strides *sgh, const scanscam_strides *sga,
                                 const scanscam_strides *sgb, int64_t batch, int64_t T, int64_t C, int dtype,
                                 void *workspace, size_t workspace_bytes, void *stream, const scanscam_plan *plan)
{
    const scanscam_strides *const st[5] = {sa, sgh, sh, sgb, sga};
    return run_cl(true, a, gh, h, gb, ga, st, batch, T, C, dtype, workspace, workspace_bytes, stream, plan);
}

int scanscam_workspace_timed_out(const void *workspace, void *stream, int *timed_out)
{
    if (!workspace || !timed_out) return SCANSCAM_EINVAL;
    if (!aligned_to(workspace, 8)) return SCANSCAM_EALIGN;
    uint64_t word = 0;
    if (hipStreamSynchronize(static_cast<hipStream_t>(stream)) != hipSuccess) return SCANSCAM_ELAUNCH;
    if (hipMemcpy(&word, static_cast<const uint64_t *>(workspace) + scanscam::kTimeoutWord, sizeof(word),
                  hipMemcpyDeviceToHost) != hipSuccess)
        return SCANSCAM_ELAUNCH;
    *timed_out = word != 0 ? 1 : 0;
    return SCANSCAM_OK;
}

int scanscam_noalloc_timed_out(void *stream, int *timed_out)
{
    if (!timed_out) return SCANSCAM_EINVAL;
    void *ws = nullptr;
    const int rc = noalloc_scratch(&ws);
    if (rc != SCANSCAM_OK) return rc;
    return scanscam_workspace_timed_out(ws, stream, timed_out);
}

int scanscam_resolve_plan(int64_t rows, int64_t T, int dtype, int direction, const scanscam_plan *plan,
                          scanscam_plan *out)
{
    if (!out) return SCANSCAM_EINVAL;
    Resolved r;
    // Dense tensors on allocation borders: rows start on line borders exactly when a row is whole lines.
    const int esize = elem_size(dtype);
    const bool lines = esize != 0 && (T * esize) % 128 == 0;
    const int rc = resolve(plan, rows, T, dtype, true, lines, direction == SCANSCAM_BACKWARD, &r, /*flat_ok=*/true);
    if (rc != SCANSCAM_OK) return rc;
    out->mode = r.l.mode;
    out->vec = r.l.vec;
    out->unroll = r.l.unroll;
    out->waves = r.l.waves;
    out->waves_per_row = r.l.mode == kModeRow ? r.l.wpr : 0;
    out->spin_limit = (plan && plan->spin_limit > 0) ? plan->spin_limit : scanscam::kSpinLimit;
    return SCANSCAM_OK;
}

int scanscam_resolve_plan_cl(int64_t batch, int64_t T, int64_t C, int dtype, int direction,
                             const scanscam_plan *plan, scanscam_plan *out)
{
    if (!out) return SCANSCAM_EINVAL;
    const int esize = elem_size(dtype);
    if (esize == 0) return SCANSCAM_EDTYPE;
    if (batch <= 0 || T <= 0 || C <= 0 || T >= kMaxT || C >= kMaxT) return SCANSCAM_EINVAL;
    // Dense tensors on allocation borders: every time step starts on the largest power of two that divides C elements.
    int align = 16;
    while (align > esize && !(batch == 1 && T == 1) && (C * esize) % align != 0) align >>= 1;
    scanscam::ClLaunch l;
    const int rc = resolve_cl(plan, batch, T, C, dtype, align, direction == SCANSCAM_BACKWARD, &l);
    if (rc != SCANSCAM_OK) return rc;
    out->mode = l.kind == 2 ? kModeLookback : kModeRow;
    out->vec = l.vec;
    out->unroll = l.steps;
    out->waves = l.waves;
    out->waves_per_row = 0;
    out->spin_limit = (plan && plan->spin_limit > 0) ? plan->spin_limit : scanscam::kSpinLimit;
    return SCANSCAM_OK;
}

int scanscam_predict_cl(int64_t batch, int64_t T, int64_t C, int dtype, int direction, const scanscam_plan *plan,
                        double *microseconds)
{
    if (!microseconds) return SCANSCAM_EINVAL;
    const int esize = elem_size(dtype);
    if (esize == 0) return SCANSCAM_EDTYPE;
    if (batch <= 0 || T <= 0 || C <= 0 || T >= kMaxT || C >= kMaxT) return SCANSCAM_EINVAL;
    int align = 16;
    while (align > esize && !(batch == 1 && T == 1) && (C * esize) % align != 0) align >>= 1;
    scanscam::ClLaunch l;
    return resolve_cl(plan, batch, T, C, dtype, align, direction == SCANSCAM_BACKWARD, &l, microseconds);
}

const char *scanscam_strerror(int code)
{
    switch (code) {
    case SCANSCAM_OK: return "ok";
    case SCANSCAM_EINVAL: return "invalid argument (null pointer, negative or too large size)";
    case SCANSCAM_EDTYPE: return "unsupported storage type";
    case SCANSCAM_EALIGN: return "pointer not aligned to its element size (or workspace not to 8 bytes)";
    case SCANSCAM_EPLAN: return "launch plan not valid for this shape or alignment";
    case SCANSCAM_EWORKSPACE: return "workspace missing or smaller than scanscam_workspace_bytes()";
    case SCANSCAM_ELAUNCH: return "HIP runtime refused the kernel launch";
    case SCANSCAM_ESCRATCH:
        return "shape needs more look-back scratch than the library's fixed array (scanscam_scan_fwd_noalloc): "
               "use scanscam_scan_fwd with a workspace";
    default: return "unknown scanscam error code";
    }
}

int scanscam_abi_version(void) { return 3; }

}  // extern "C"

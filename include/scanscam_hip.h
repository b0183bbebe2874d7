/*
 * scanscam_hip.h -- C ABI of libscanscam_hip.so: the first-order gated linear
 * scan h[t] = a[t]*h[t-1] + b[t] and its reverse-time backward pass as HIP
 * kernels for gfx950 (MI355X).
 *
 * These entry points are what a binding of the reference's native layer would
 * call for this path. The reference exposes it through pybind11 functions
 * taking torch tensors (src/scanscam_cuda.cu:725-737); here the same calls take
 * plain device pointers and sizes.
 *
 * Conventions (same as the reference's native functions):
 *   - every tensor is a dense row-major [rows, T] array on the current HIP
 *     device, scanned along T, all of one storage type;
 *   - the caller allocates every output and the workspace; the library
 *     allocates nothing and is re-entrant. It keeps no state between calls,
 *     with one exception: scanscam_scan_fwd_noalloc works in a fixed array of
 *     the library's own in each GPU's memory (see there);
 *   - calls are asynchronous: kernels are enqueued on `stream` (0 = the null
 *     stream) and the call returns at once;
 *   - the return value is 0 on success or a SCANSCAM_E* code; nothing is
 *     launched when an error is returned.
 * rows == 0 or T == 0 is a successful no-op.
 */
#ifndef SCANSCAM_HIP_H
#define SCANSCAM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Storage types. Arithmetic is fp32 for the first three and fp64 for SCANSCAM_F64
 * (the reference dispatches float and double, src/scanscam_cpu.hpp:43, src/scanscam_cuda.cu:288). */
enum {
    SCANSCAM_F32 = 0,
    SCANSCAM_BF16 = 1, /* no counterpart in the reference */
    SCANSCAM_F16 = 2,  /* no counterpart in the reference */
    SCANSCAM_F64 = 3
};

enum { SCANSCAM_FORWARD = 0, SCANSCAM_BACKWARD = 1 };

/* Error codes. */
enum {
    SCANSCAM_OK = 0,
    SCANSCAM_EINVAL = 1,    /* null pointer, negative size, T >= 2^31 - 2^20 */
    SCANSCAM_EDTYPE = 2,    /* unknown storage type */
    SCANSCAM_EALIGN = 3,    /* pointer not aligned to its element size, or workspace not to 8 bytes */
    SCANSCAM_EPLAN = 4,     /* explicit plan not valid for this shape / alignment */
    SCANSCAM_EWORKSPACE = 5,/* workspace missing or smaller than scanscam_workspace_bytes() */
    SCANSCAM_ELAUNCH = 6,   /* the HIP runtime refused the launch */
    SCANSCAM_ESCRATCH = 7   /* scanscam_scan_fwd_noalloc: the shape needs more than SCANSCAM_NOALLOC_SCRATCH_BYTES */
};

/* Kernel families. */
enum {
    SCANSCAM_MODE_AUTO = 0,
    SCANSCAM_MODE_SMALL = 1,   /* T <= 64*vec: several rows per wave, no carries */
    SCANSCAM_MODE_ROW = 2,     /* a workgroup (or part of one) walks a whole row */
    SCANSCAM_MODE_LOOKBACK = 3, /* rows cut into tiles over workgroups, decoupled look-back carries */
    SCANSCAM_MODE_FLAT = 4      /* dense tensors, 16/sizeof(storage) <= T <= 64 * that: all rows scanned as one
                                   stream of aligned vectors with a reset at every row start (unroll 2 or 4) */
};

/*
 * Explicit launch plan, for tuning and for tests that must force one kernel
 * family on a small input. Zero in any field means "choose for me".
 *   vec            elements per lane per load: 16/sizeof(storage) or 1
 *   unroll         64-lane chunks per wave per tile: 1, 2, 3, 4 or 8 (1 or 4 when vec == 1)
 *   waves          waves per workgroup, 1..16 (at most 8 when unroll == 8)
 *   waves_per_row  ROW only: a divisor of `waves` (waves / waves_per_row rows share a workgroup)
 *   spin_limit     kernels that wait for another workgroup's carry poll at most this many times
 *                  (0 = 2^20, about a second); a wait that expires sets word 1 of the workspace to 1
 *                  and poisons the affected outputs with NaN instead of spinning for ever
 */
typedef struct scanscam_plan {
    int32_t mode;
    int32_t vec;
    int32_t unroll;
    int32_t waves;
    int32_t waves_per_row;
    int32_t spin_limit;
} scanscam_plan;

/*
 * Forward scan: h[r,t] = a[r,t]*h[r,t-1] + b[r,t], h[r,-1] = 0.
 * Replaces blocked_linear_scan(gate, value, output), src/scanscam_cuda.cu:260-307
 * (arithmetic of simple_linear_scan_cpu, src/scanscam_cpu.hpp:30-52).
 * h may be the very buffer of a or of b (an in-place call, as the reference's kernel allows,
 * src/scanscam_cuda.cu:205-257); any other overlap of an output with an input is not allowed, and
 * the outputs of the backward call must not share bytes with any of its inputs (a[t+1] and h[t-1] are
 * read across the borders of what a workgroup writes).
 */
int scanscam_scan_fwd(const void *a, const void *b, void *h, int64_t rows, int64_t T, int dtype,
                      void *workspace, size_t workspace_bytes, void *stream);

/*
 * Backward scan: gb[r,t] = gh[r,t] + a[r,t+1]*gb[r,t+1] (gb[r,T] = 0),
 * ga[r,t] = gb[r,t]*h[r,t-1] (h[r,-1] = 0); `h` is the saved forward output.
 * Replaces blocked_linear_scan_backward(gate, output, outGrad, gateGradOut,
 * valueGradOut), src/scanscam_cuda.cu:427-469 (arithmetic of
 * simple_linear_scan_backward_cpu, src/scanscam_cpu.hpp:80-113).
 */
int scanscam_scan_bwd(const void *a, const void *h, const void *gh, void *ga, void *gb, int64_t rows,
                      int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream);

/*
 * scanscam_scan_fwd for callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference, whose
 * kernels need no workspace. Same arguments, results (bit for bit) and
 * errors as scanscam_scan_fwd, without the workspace: where rows are split over workgroups, the
 * look-back descriptors live in a fixed array of SCANSCAM_NOALLOC_SCRATCH_BYTES in the GPU's memory
 * that belongs to the library (one per GPU it runs on, held until the process ends), found once per
 * device on the first call there. The call itself allocates and frees nothing, on the device or
 * through any library. A shape whose descriptors do not fit (more than about 120 000 look-back tiles
 * of fp32 arithmetic, i.e. 1 G elements in long rows) is refused with SCANSCAM_ESCRATCH and nothing is launched.
 * Every call clears the part of the array it uses, with a kernel on `stream`. All calls on one GPU
 * share that GPU's array: calls that may overlap in time on one GPU (two streams, two threads) race
 * and must use scanscam_scan_fwd with separate workspaces instead.
 * The first call on a device asks the runtime for the array's address there (not a stream operation, and
 * it may load the library's code onto the device): make one call per device -- any shape, also rows == 0 --
 * outside of any stream capture before capturing calls into a HIP graph. The device that `stream` belongs
 * to must be the current device, as for every call of this library.
 * scanscam_noalloc_timed_out is scanscam_workspace_timed_out (below) for the current device's array.
 */
#define SCANSCAM_NOALLOC_SCRATCH_BYTES (1 << 20)
int scanscam_scan_fwd_noalloc(const void *a, const void *b, void *h, int64_t rows, int64_t T, int dtype,
                              void *stream);
int scanscam_noalloc_timed_out(void *stream, int *timed_out);

/*
 * Bytes of device workspace the call above of that direction needs for this
 * shape (0 for most shapes; non-zero when rows are split over workgroups, which
 * the two directions decide separately). The
 * reference's kernels need none, so this has no counterpart there. The
 * workspace need not be initialised; its contents are clobbered. Two calls
 * that may overlap in time need separate workspaces.
 */
size_t scanscam_workspace_bytes(int64_t rows, int64_t T, int dtype, int direction);

/* The same three calls with an explicit plan (plan == NULL means automatic). */
int scanscam_scan_fwd_plan(const void *a, const void *b, void *h, int64_t rows, int64_t T, int dtype,
                           void *workspace, size_t workspace_bytes, void *stream, const scanscam_plan *plan);
int scanscam_scan_bwd_plan(const void *a, const void *h, const void *gh, void *ga, void *gb, int64_t rows,
                           int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                           const scanscam_plan *plan);
size_t scanscam_workspace_bytes_plan(int64_t rows, int64_t T, int dtype, int direction,
                                     const scanscam_plan *plan);

/*
 * Measurement aid (no counterpart in the reference): the _plan calls with the scan kernel's own start
 * and end on the GPU recorded into two HIP events the caller created (hipEventCreate), so that
 * hipEventElapsedTime(start, stop) is the kernel's duration, free of launch gaps and of the event
 * packets a hipEventRecord pair would put around it. Either event may be NULL. The kernel that
 * clears the workspace of a long-row launch is not part of the interval. A problem so large that it
 * needs several launches (more than 2^32 threads) returns SCANSCAM_EINVAL here.
 */
int scanscam_scan_fwd_timed(const void *a, const void *b, void *h, int64_t rows, int64_t T, int dtype,
                            void *workspace, size_t workspace_bytes, void *stream, const scanscam_plan *plan,
                            void *start_event, void *stop_event);
int scanscam_scan_bwd_timed(const void *a, const void *h, const void *gh, void *ga, void *gb, int64_t rows,
                            int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                            const scanscam_plan *plan, void *start_event, void *stop_event);

/*
 * Channels-last storage: every tensor is a dense [batch, T, C] array (C
 * fastest) scanned along T -- the layout of a [batch, C, T] tensor whose last
 * two dimensions were transposed. Same arithmetic as the calls above.
 * Replace transposed_linear_scan(gate, value, output, channelsPerBlock),
 * src/scanscam_cuda.cu:556-582, and transposed_linear_scan_backward(gate,
 * output, outGrad, gateGradOut, valueGradOut, channelsPerBlock), :687-723. The
 * reference's trailing tuning argument has its counterpart in `plan` (NULL =
 * automatic): vec = channels per lane (16/sizeof(storage) or 1; also half of
 * the former, an 8-byte lane, for fp32 and 16-bit storage, and 2 for 16-bit
 * storage), unroll = time
 * steps per wave per tile (2, 4, 8 for the full vector; 4, 8, 16 for narrower lanes;
 * with at most 32 * vec channels a wave holds several time steps per load and
 * `unroll` counts those loads), waves = waves per workgroup (1..16). When
 * batch * C is too small to fill the
 * GPU, time is also cut into tiles over workgroups, carried by a look-back
 * chain, which needs a workspace (scanscam_workspace_bytes_cl, same rules as
 * above); mode = SCANSCAM_MODE_ROW forbids that split, SCANSCAM_MODE_LOOKBACK
 * forces it. A time step (C channels, or the time stride of a strided call)
 * must stay below 4 GiB / 18 = 227 MiB (the kernels address a wave's steps with
 * 32-bit offsets from its first one): larger ones return SCANSCAM_EINVAL.
 */
int scanscam_scan_fwd_cl(const void *a, const void *b, void *h, int64_t batch, int64_t T, int64_t C, int dtype,
                         void *workspace, size_t workspace_bytes, void *stream, const scanscam_plan *plan);
int scanscam_scan_bwd_cl(const void *a, const void *h, const void *gh, void *ga, void *gb, int64_t batch,
                         int64_t T, int64_t C, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                         const scanscam_plan *plan);
size_t scanscam_workspace_bytes_cl(int64_t batch, int64_t T, int64_t C, int dtype, int direction,
                                   const scanscam_plan *plan);

/*
 * Strided tensors, so that views need no copy first. The reference's wrappers
 * call .contiguous() on every argument (scanscam/cuda.py:36-37, 60-62), which
 * costs a full extra read and write of each tensor that is a view: a half of a
 * fused projection (chunk along channels), a slice of a longer buffer, a gate
 * broadcast over the batch. These calls replace that copy + kernel pair.
 *
 * Strides are in elements and must be >= 0; 0 is allowed for inputs (a
 * broadcast). Outputs must not overlap themselves or any input.
 *
 * Row layout: the tensors are logical [n0, n1, T] arrays, unit-stride along T;
 * element (r0, r1, t) of a tensor with strides s is at s.outer*r0 + s.row*r1 + t.
 * Channels-last: logical [batch, T, C], unit-stride along C; element (b, t, c)
 * is at s.outer*b + s.row*t + c, with s.row < 2^31.
 * A NULL strides pointer means dense. Workspace: scanscam_workspace_bytes(n0*n1,
 * T, ...) and scanscam_workspace_bytes_cl(batch, T, C, ...).
 */
typedef struct scanscam_strides {
    int64_t outer;
    int64_t row;
} scanscam_strides;

int scanscam_scan_fwd_strided(const void *a, const void *b, void *h, const scanscam_strides *sa,
                              const scanscam_strides *sb, const scanscam_strides *sh, int64_t n0, int64_t n1,
                              int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                              const scanscam_plan *plan);
int scanscam_scan_bwd_strided(const void *a, const void *h, const void *gh, void *ga, void *gb,
                              const scanscam_strides *sa, const scanscam_strides *sh, const scanscam_strides *sgh,
                              const scanscam_strides *sga, const scanscam_strides *sgb, int64_t n0, int64_t n1,
                              int64_t T, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                              const scanscam_plan *plan);
int scanscam_scan_fwd_cl_strided(const void *a, const void *b, void *h, const scanscam_strides *sa,
                                 const scanscam_strides *sb, const scanscam_strides *sh, int64_t batch, int64_t T,
                                 int64_t C, int dtype, void *workspace, size_t workspace_bytes, void *stream,
                                 const scanscam_plan *plan);
int scanscam_scan_bwd_cl_strided(const void *a, const void *h, const void *gh, void *ga, void *gb,
                                 const scanscam_strides *sa, const scanscam_strides *sh,
                                 const scanscam_strides *sgh, const scanscam_strides *sga,
                                 const scanscam_strides *sgb, int64_t batch, int64_t T, int64_t C, int dtype,
                                 void *workspace, size_t workspace_bytes, void *stream, const scanscam_plan *plan);

/*
 * Whether a wait for another workgroup's carry expired in a call that used this workspace (see
 * spin_limit in scanscam_plan): waits for the work on `stream` to finish, reads the workspace's flag
 * word and writes 1 or 0 to *timed_out. A correct launch never sets it; where it is set, the
 * affected outputs hold NaN. Meant for debugging and tests: it blocks the host. No counterpart in
 * the reference.
 */
int scanscam_workspace_timed_out(const void *workspace, void *stream, int *timed_out);

/*
 * Writes the plan the automatic choice resolves to for this shape (assuming
 * 16-byte aligned pointers) into *out. Returns 0 or an error code.
 */
int scanscam_resolve_plan(int64_t rows, int64_t T, int dtype, int direction, const scanscam_plan *plan,
                          scanscam_plan *out);

/*
 * The same for the channels-last calls on dense [batch, T, C] tensors whose bases are 16-byte
 * aligned: mode SCANSCAM_MODE_ROW where a workgroup walks all of T, SCANSCAM_MODE_LOOKBACK where
 * tiles of time steps chain through the workspace; vec channels per lane, unroll time steps per
 * wave and tile, waves per workgroup. No counterpart in the reference, whose kernel has one launch
 * shape (scanscam/cuda.py:69-95 passes channels_per_block only).
 */
int scanscam_resolve_plan_cl(int64_t batch, int64_t T, int64_t C, int dtype, int direction,
                             const scanscam_plan *plan, scanscam_plan *out);

/*
 * The duration in microseconds that the library's cost model estimates for a channels-last call on dense
 * [batch, T, C] tensors with this plan (NULL or zero fields: with what the model itself chooses for them, i.e.
 * the estimate behind scanscam_resolve_plan_cl). The automatic plan is the candidate with the smallest such
 * estimate; the model (a formula of a few physical terms and a learned correction on top of it) is fitted to
 * timings on one MI355X (scanscam_amd/plan_fit.py), so the figure is a ranking aid with an error of about 5 %,
 * not a promise. The first call for a (shape, plan) on a thread takes about 0.1 ms on the host (the choice is
 * remembered per thread after that; nothing but speed depends on what is remembered). No counterpart in the
 * reference.
 */
int scanscam_predict_cl(int64_t batch, int64_t T, int64_t C, int dtype, int direction, const scanscam_plan *plan,
                        double *microseconds);

/* Static, never-freed description of an error code. */
const char *scanscam_strerror(int code);

/* ABI version of this header: bumped on any incompatible change. */
int scanscam_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif /* SCANSCAM_HIP_H */

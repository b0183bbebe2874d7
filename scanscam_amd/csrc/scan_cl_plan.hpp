// Launch plan of the channels-last calls: a cost model (a formula plus a learned correction) in place of rules.
//
// Every launch shape the kernels are instantiated for is a candidate: lanes of 1 channel up to 16 bytes
// (whole, or element-aligned where C or the alignment does not allow whole ones), a workgroup that walks
// all of T or tiles of time handed out over workgroups, 2 to 16 time steps per wave, 4 or 8 waves (a walk
// also 16). For each candidate cl_predict_us() estimates the launch's duration from a few terms, and the plan is the
// candidate with the smallest estimate. Fields that the caller's plan names are taken as given and only
// the others are chosen.
//
// The terms (microseconds):
//   stream   algorithmic bytes / (rate of this kernel variant) x (lines touched / lines used) / fill^alpha
//            `rate`: one measured streaming rate per kernel variant (kernel, lane bytes, storage size,
//            direction, and whether a time step is whole 128-byte lines), the table of scan_cl_model.inc;
//            `lines touched`: every wave access that starts or ends inside a 128-byte line moves the rest of
//            that line as well; `fill`: the part of the lanes of a time step's waves that hold a channel.
//   latency  rounds of workgroups x tiles per workgroup x time of one tile, where a tile takes the memory
//            latency plus the issue time of its waves' instructions (proportional to elements per lane,
//            more backwards, for 16-bit storage and for element-aligned lanes), a tile of the time split
//            also the ticket and the wait for its carry; workgroups resident on a CU (from the
//            registers the kernels were compiled to) cover each other's latency but share its SIMDs.
//   chain    time-split tiles per (batch element, channel group) / waves: the super-tile chain of a
//            row-group advances one memory round trip at a time.
// The formula is their sum plus the launch itself (and the launch that prepares the workspace of a time split).
// (Combined as a p-norm with p = 1.5 to 4, the fitted model chose worse plans on shapes it had not seen.)
// It explains measured durations to about 7 % rms, where two runs of one plan differ by 1 %; what it leaves is
// learned from the same timings by a small network (ClResidual below: ln(measured / formula) from 24 numbers that
// describe shape and plan), and the estimate is the formula times that correction, which is bounded (a factor of
// exp(+-0.7)) and never extrapolates (its inputs are clipped to the range the timings covered). With the formula
// alone the plan picked on unseen shapes is 7 % behind the best measured plan on average, with the correction 2-3 %.
//
// The constants are fitted, not hand-set: `python -m scanscam_amd.plan_search --dump FILE` times every
// candidate on a set of shapes and `python -m scanscam_amd.plan_fit FILE...` fits formula and correction to those
// timings and prints this file's tables (scan_cl_model.inc). No shape has a rule of its own. Two facts about resources are
// constraints on the candidates instead of terms (cl_choose): 16-byte lanes of 16-bit storage spill in the time
// split, and a walk with fewer workgroups than half the compute units cannot keep the chip busy.
#pragma once

#include "scan_launch.hpp"
#include "scanscam_hip.h"

#include <cmath>
#include <cstdint>

namespace scanscam {

constexpr int kClComputeUnits = 256;  // MI355X

// Waves a workgroup of these kernels may have: their LDS arrays of [waves][vec][64] values (2 buffers x (A, B)
// for the walk, 7 for the time split) stay within 64 KiB, and the kernels' launch bounds.
inline int cl_max_waves(int vec, int steps, int kind, int csize)
{
    const int planes = kind == 2 ? 7 : 4;
    int w = (64 * 1024) / (planes * vec * kWave * csize);
    const int by_threads = cl_max_threads(vec, steps) / kWave;
    w = w < by_threads ? w : by_threads;
    return w < kMaxWaves ? w : kMaxWaves;
}

struct ClModel {
    // Streaming rate in bytes per microsecond / 1e6 (= TB/s of algorithmic bytes at full lanes):
    // [kernel: 0 walk, 1 several steps per wave, 2 time split][storage: 2, 4, 8 bytes][lane: 2, 4, 8, 16 bytes][direction]
    // [a time step is a whole number of 128-byte lines]
    double rate[3][3][4][2][2];
    double latency;      // memory latency of a tile's loads
    double latency_w8;   // ... more per 8 waves of the workgroup (the barrier waits for the slowest wave)
    double issue;        // issue time of one wave's instructions per element per lane (fp32, forward)
    double issue_bwd;    // factor backwards
    double issue_16;     // factor for 16-bit storage
    double issue_ragged; // additional part for element-aligned lanes
    double launch;       // the launch
    double launch_split; // the launch that prepares the workspace of a time split
    double carry;        // ticket and carry wait of a time-split tile
    double fill_alpha;   // exponent of 1 / fill in the streaming term
    double chain;        // one hop of a row-group's super-tile chain
    double issue_shared; // additional issue time per doubling of the time steps that share a wave (the lane scan per load)
    double line[4];      // weight of the lines touched beyond the bytes used, for lanes of 2, 4, 8, 16 bytes
};

// What the formula leaves unexplained (about 7 % rms against 1 % of run-to-run noise) a small network has learned
// from the same timings: ln(measured / estimate) as a function of cl_features(), two hidden layers of tanh units.
// The library only evaluates it; scanscam_amd/plan_fit.py trains it and prints its weights.
constexpr int kClInputs = 24, kClHidden1 = 64, kClHidden2 = 32;
constexpr double kClResidualLimit = 0.7;  // the correction of ln(duration) stays within +-0.7

struct ClResidual {
    double lo[kClInputs], hi[kClInputs];      // range of each input in the training timings: inputs are clipped to it
    double mean[kClInputs], scale[kClInputs]; // standardisation
    double w1[kClInputs][kClHidden1], b1[kClHidden1];
    double w2[kClHidden1][kClHidden2], b2[kClHidden2];
    double w3[kClHidden2], b3;
};

#include "scan_cl_model.inc"  // const ClModel kClModel = {...}; const ClResidual kClResidual = {...}: printed by scanscam_amd/plan_fit.py

struct ClShape {
    int64_t batch, T, C;
    int esize;  // bytes per stored element
    int csize;  // bytes of the arithmetic type
    int align;  // the largest of 16, 8, 4 and esize that every base and stride is a multiple of
    bool rev;
};

struct ClCandidate {
    int vec, steps, waves, kind;  // kind 0: a workgroup walks all of T; 2: tiles of time over workgroups
    int group;                    // lanes per time step; below 64: several steps share a wave
    bool ragged;                  // element-aligned lanes
};

inline int cl_pow2_ceil(int64_t v)
{
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

inline int64_t cl_groups(int64_t C, int vec) { return (C + (int64_t)kWave * vec - 1) / ((int64_t)kWave * vec); }

// Whether lanes of `vec` channels can be whole on this shape (C a multiple of them, bases and strides on their borders).
inline bool cl_whole_lanes(const ClShape &s, int vec)
{
    const int bytes = vec * s.esize;
    return vec == 1 || (s.C % vec == 0 && s.align >= (bytes > 16 ? 16 : bytes));
}

// Fills group and ragged of a candidate and says whether the kernels can run it at all.
inline bool cl_complete(const ClShape &s, ClCandidate *c)
{
    const int full = 16 / s.esize, half = s.esize <= 4 ? full / 2 : 0;
    if (!(c->vec == 1 || c->vec == full || (half > 1 && c->vec == half) || (s.esize == 2 && c->vec == 2))) return false;
    c->ragged = !cl_whole_lanes(s, c->vec);
    // Element-aligned lanes: the walk only, and more than half a wave of them per time step.
    if (c->ragged && (c->kind != 0 || s.C <= (int64_t)(kWave / 2) * c->vec)) return false;
    c->group = kWave;
    if (c->kind == 0 && cl_groups(s.C, c->vec) == 1) {
        const int g = cl_pow2_ceil((s.C + c->vec - 1) / c->vec);
        if (g < kWave) c->group = g;
    }
    const bool steps_ok = c->vec == full ? (c->steps == 2 || c->steps == 4 || c->steps == 8)
                                         : (c->steps == 4 || c->steps == 8 || c->steps == 16);
    if (!steps_ok) return false;
    return c->waves >= 1 && c->waves <= cl_max_waves(c->vec, c->steps, c->kind, s.csize);
}

// Vector registers per lane that the kernels compile to, to within a few (from the compiler's resource
// report of this build): base + elements per lane and tile x words per element and stream.
inline double cl_registers(const ClShape &s, const ClCandidate &c)
{
    double per = s.esize == 2 ? (s.rev ? 3.8 : 2.8) : (s.rev ? 3.0 : 2.1), base = c.kind == 2 ? 34.0 : 24.0;
    if (c.group < kWave) {  // several time steps per wave
        base = s.rev ? 36.0 : 32.0;
        per = s.rev ? 5.7 : 4.6;
    }
    return base + c.steps * c.vec * per * (s.esize == 8 ? 2.0 : 1.0);
}

// The formula: launch + stream + latency + chain (see the head of this file). `x`, if given, receives cl_features().
inline double cl_physical_us(const ClShape &s, const ClCandidate &c, const ClModel &m = kClModel, double *x = nullptr)
{
    const int sub = kWave / c.group;  // time steps per wave instruction
    const int64_t G = cl_groups(s.C, c.vec);
    const double fill = c.group == kWave ? (double)s.C / (double)(G * kWave * c.vec) : (double)s.C / (double)(c.group * c.vec);
    const int lane = c.vec * s.esize;
    const int64_t RG = s.batch * G;
    const int64_t tile_steps = (int64_t)c.waves * c.steps * sub;
    const int64_t tiles = (s.T + tile_steps - 1) / tile_steps;
    const double bytes = (double)s.batch * (double)s.T * (double)s.C * s.esize * (s.rev ? 5.0 : 3.0);

    // More than the launch bounds leave a lane (512 threads: 256 registers, 1024: 128) is spilled.
    double regs = cl_registers(s, c);
    const double cap = cl_max_threads(c.vec, c.steps) == 512 ? 256.0 : 128.0;
    const bool spills = regs > cap;
    if (spills) regs = cap;
    int occupancy = (int)(512.0 / regs);
    occupancy = occupancy < 1 ? 1 : (occupancy > 8 ? 8 : occupancy);
    const int resident_max = (4 * occupancy) / c.waves < 1 ? 1 : (4 * occupancy) / c.waves;

    double busy = m.issue * c.steps * c.vec * (c.waves > 4 ? c.waves / 4.0 : 1.0) * (s.rev ? m.issue_bwd : 1.0) *
                  (s.esize == 2 ? m.issue_16 : 1.0);
    if (spills) busy *= 2.0;
    if (c.group < kWave) busy *= 1.0 + m.issue_shared * std::log2((double)sub);
    if (c.ragged) busy *= 1.0 + m.issue_ragged;
    const double tile_us = m.latency + m.latency_w8 * c.waves / 8.0 + busy + (c.kind == 2 ? m.carry : 0.0);
    const int64_t workgroups = c.kind == 2 ? RG * tiles : RG;
    const double per_cu = std::ceil((double)workgroups / kClComputeUnits);
    const double resident = per_cu < resident_max ? per_cu : resident_max;
    const double rounds = std::ceil((double)workgroups / ((double)kClComputeUnits * resident_max));
    const double one = tile_us > resident * busy ? tile_us : resident * busy;
    const double latency_us = rounds * (c.kind == 2 ? 1.0 : (double)tiles) * one;

    const int kernel = c.group < kWave ? 1 : c.kind;
    const int es = s.esize == 2 ? 0 : (s.esize == 4 ? 1 : 2);
    const int ln = lane <= 2 ? 0 : (lane == 4 ? 1 : (lane == 8 ? 2 : 3));
    const int64_t step_bytes = s.C * s.esize;
    const double rate = m.rate[kernel][es][ln][s.rev ? 1 : 0][step_bytes % 128 == 0 ? 1 : 0] * 1e6;
    auto gcd = [](int64_t a, int64_t b) {
        while (b) {
            const int64_t t = a % b;
            a = b;
            b = t;
        }
        return a;
    };
    double lines;
    if (c.group < kWave) {
        const int64_t span = sub * step_bytes;
        lines = 1.0 + m.line[ln] * (double)(128 - gcd(span, 128)) / (double)span;
    } else {
        const int64_t a = gcd(gcd(step_bytes, (int64_t)kWave * lane), 128);
        lines = 1.0 + m.line[ln] * (double)G * (double)(128 - a) / (double)step_bytes;
    }
    const double stream_us = bytes / std::pow(fill, m.fill_alpha) / rate * lines;
    const double chain_us = c.kind == 2 ? m.chain * (double)tiles / c.waves : 0.0;
    const double us = m.launch + (c.kind == 2 ? m.launch_split : 0.0) + stream_us + latency_us + chain_us;
    if (x) {  // cl_features: what the learned correction sees of (shape, plan)
        x[0] = std::log2((double)RG);
        x[1] = std::log2((double)tiles);
        x[2] = std::log2((double)s.T);
        x[3] = std::log2((double)s.C);
        x[4] = std::log2((double)s.batch);
        x[5] = fill;
        x[6] = c.steps;
        x[7] = c.vec;
        x[8] = c.waves;
        x[9] = c.kind;
        x[10] = s.esize;
        x[11] = s.rev ? 1.0 : 0.0;
        x[12] = c.group < kWave ? 1.0 : 0.0;
        x[13] = std::log2((double)sub);
        x[14] = c.ragged ? 1.0 : 0.0;
        x[15] = cl_registers(s, c);
        x[16] = std::log2((double)workgroups);
        x[17] = (double)((workgroups - 1) % kClComputeUnits + 1) / kClComputeUnits;  // how full the last round of workgroups is
        x[18] = step_bytes % 128 == 0 ? 1.0 : 0.0;
        x[19] = step_bytes % 16 == 0 ? 1.0 : 0.0;
        x[20] = std::log2(bytes);
        x[21] = std::log(us);
        x[22] = std::log2((double)lane);
        x[23] = (double)workgroups / kClComputeUnits < 8.0 ? (double)workgroups / kClComputeUnits : 8.0;
    }
    return us;
}

// The learned correction of ln(duration) for one candidate's features.
inline double cl_residual(const double (&x)[kClInputs], const ClResidual &r = kClResidual)
{
    double z[kClInputs], h1[kClHidden1], h2[kClHidden2];
    for (int i = 0; i < kClInputs; i++) {
        const double v = x[i] < r.lo[i] ? r.lo[i] : (x[i] > r.hi[i] ? r.hi[i] : x[i]);
        z[i] = (v - r.mean[i]) / r.scale[i];
    }
    for (int j = 0; j < kClHidden1; j++) h1[j] = r.b1[j];
    for (int i = 0; i < kClInputs; i++)
        for (int j = 0; j < kClHidden1; j++) h1[j] += z[i] * r.w1[i][j];
    for (int j = 0; j < kClHidden1; j++) h1[j] = std::tanh(h1[j]);
    for (int k = 0; k < kClHidden2; k++) h2[k] = r.b2[k];
    for (int j = 0; j < kClHidden1; j++)
        for (int k = 0; k < kClHidden2; k++) h2[k] += h1[j] * r.w2[j][k];
    for (int k = 0; k < kClHidden2; k++) h2[k] = std::tanh(h2[k]);
    double y = r.b3;
    for (int k = 0; k < kClHidden2; k++) y += h2[k] * r.w3[k];
    return y < -kClResidualLimit ? -kClResidualLimit : (y > kClResidualLimit ? kClResidualLimit : y);
}

// Estimated duration of a candidate: the formula times the learned correction.
inline double cl_predict_us(const ClShape &s, const ClCandidate &c)
{
    double x[kClInputs];
    const double physical = cl_physical_us(s, c, kClModel, x);
    return physical * std::exp(cl_residual(x));
}

// The candidate with the smallest estimate among those that agree with the caller's plan `u` (zero fields are
// free; mode ROW forbids the time split, LOOKBACK forces it). Returns false if none can run.
inline bool cl_choose(const ClShape &s, const scanscam_plan &u, ClCandidate *best, double *best_us = nullptr)
{
    const int full = 16 / s.esize, half = s.esize <= 4 ? full / 2 : 0;
    int vecs[4], nv = 0;
    if (u.vec) {
        vecs[nv++] = u.vec;
    } else {
        vecs[nv++] = 1;
        if (s.esize == 2) vecs[nv++] = 2;
        if (half > 1 && half != 2) vecs[nv++] = half;
        if (half == 2 && s.esize != 2) vecs[nv++] = 2;
        if (full > 1) vecs[nv++] = full;
    }
    const int all_steps[4] = {2, 4, 8, 16};
    const int all_waves[3] = {4, 8, 16};  // 16 only for a walk: tiles of 16 waves measured behind 8 throughout
    // A walk keeps one workgroup per batch and channel group: with fewer of them than half the compute units it
    // leaves most of the chip idle however well it streams, so it stands back ("thin") whenever the time can be
    // split instead. Among 328 timed shapes of that kind a walk was the fastest plan once.
    bool found = false, found_thin = false;
    double least = 0.0, least_thin = 0.0;
    ClCandidate thin{};
    for (int iv = 0; iv < nv; iv++) {
        for (int kind = 0; kind <= 2; kind += 2) {
            if ((kind == 2 && u.mode == kModeRow) || (kind == 0 && u.mode == kModeLookback)) continue;
            // Left to itself the choice passes over the time split in 16-byte lanes of 16-bit storage, which the
            // compiler can only build with spills.
            if (!u.vec && kind == 2 && s.esize == 2 && vecs[iv] == 8) continue;
            for (int is = 0; is < 4; is++) {
                if (u.unroll && u.unroll != all_steps[is]) continue;
                for (int iw = 0; iw < (u.waves ? 1 : (kind == 0 ? 3 : 2)); iw++) {
                    ClCandidate c{vecs[iv], all_steps[is], u.waves ? u.waves : all_waves[iw], kind, kWave, false};
                    if (!u.waves) {
                        // No more waves than the LDS arrays and the thread limit allow, nor than there are spans of time.
                        const int most = cl_max_waves(c.vec, c.steps, c.kind, s.csize);
                        if (most < 1) continue;
                        if (c.waves > most) c.waves = most;
                    }
                    if (!cl_complete(s, &c)) continue;
                    if (!u.waves) {
                        const int64_t wave_steps = (int64_t)c.steps * (kWave / c.group);
                        const int64_t spans = (s.T + wave_steps - 1) / wave_steps;
                        if (spans < c.waves) c.waves = cl_pow2_ceil(spans);
                    }
                    const int64_t tile_steps = (int64_t)c.waves * c.steps * (kWave / c.group);
                    if (kind == 2 && u.mode != kModeLookback && s.T <= tile_steps) continue;  // one tile: nothing to split
                    const double us = cl_predict_us(s, c);
                    if (kind == 0 && u.mode == 0 && 2 * s.batch * cl_groups(s.C, c.vec) < kClComputeUnits) {
                        if (!found_thin || us < least_thin) {
                            found_thin = true;
                            least_thin = us;
                            thin = c;
                        }
                        continue;
                    }
                    if (!found || us < least) {
                        found = true;
                        least = us;
                        *best = c;
                    }
                }
            }
        }
    }
    if (!found && found_thin) {
        found = true;
        least = least_thin;
        *best = thin;
    }
    if (found && best_us) *best_us = least;
    return found;
}

}  // namespace scanscam

// Compile-time description of the eight canonical orientations (k * 22.5 degrees).
//
// For a canonical orientation the tap offsets are known when the kernel is compiled, so the
// K-tap gather is emitted as straight-line code: every LDS read has an immediate offset from
// one per-lane base address, every FMA names its weight register directly, and a lane that
// computes L neighbouring outputs along the line's step direction reads each LDS value once
// and feeds it to every output that needs it (a register sliding window).
//
// Step direction e per orientation class:
//   H  (0, 22.5, 157.5 deg)  e = (0, +1)   L outputs side by side in a row
//   V  (67.5, 90, 112.5 deg) e = (+1, 0)   L outputs stacked in a column
//   D  (45 deg)              e = (-1, +1)  L outputs up the anti-diagonal
//   D  (135 deg)             e = (+1, +1)  L outputs down the diagonal
// The "plan" lists, for an item whose first output sits at the origin, every distinct source
// position (sh, sw) = tap + l*e, and for each which tap feeds which of the L outputs.
#pragma once

#include <stdint.h>

#include <utility>

#include "dwo_canon_taps.h"

namespace dwo {

enum { CLS_H = 0, CLS_V = 1, CLS_D = 2 };

constexpr int orient_class(int o) {
    return (o == 0 || o == 1 || o == 7) ? CLS_H : ((o == 2 || o == 6) ? CLS_D : CLS_V);
}
constexpr int step_h(int o) { return orient_class(o) == CLS_H ? 0 : (o == 2 ? -1 : 1); }
constexpr int step_w(int o) { return orient_class(o) == CLS_V ? 0 : 1; }

// taps of kernel size K are the central K entries of the size-63 rows
constexpr int canon_dh(int o, int K, int s) { return kCanon.dh[o][s + (kCanonK - K) / 2]; }
constexpr int canon_dw(int o, int K, int s) { return kCanon.dw[o][s + (kCanonK - K) / 2]; }

constexpr int kMaxSrc = 320;
constexpr int kMaxL = 8;

struct Plan {
    int nsrc = 0;                      // distinct source positions per item
    int ndistinct = 0;                 // distinct tap offsets (duplicates folded)
    int16_t sh[kMaxSrc] = {};          // source position relative to the item origin
    int16_t sw[kMaxSrc] = {};
    int8_t user[kMaxSrc][kMaxL] = {};  // representative tap feeding output l, or -1
    int8_t rep[64] = {};               // rep[s]: first tap with the same offset as tap s,
                                       // -1 for a tap that cannot reach the plane
    int hmin = 0, hmax = 0, wmin = 0, wmax = 0;  // bounding box of the source positions
};

// Taps that can never land inside an H x W plane (|dh| >= H or |dw| >= W) are dropped: they
// only ever read the zero halo.
constexpr Plan make_plan(int o, int K, int L, int H, int W) {
    Plan p{};
    const int eh = step_h(o), ew = step_w(o);
    constexpr int G = 48, GS = 2 * G + 1;
    int8_t grid[GS][GS] = {};
    for (int i = 0; i < GS; i++)
        for (int j = 0; j < GS; j++) grid[i][j] = -1;
    for (int s = 0; s < K; s++) {
        const int dh = canon_dh(o, K, s), dw = canon_dw(o, K, s);
        p.rep[s] = -1;
        if (dh >= H || dh <= -H || dw >= W || dw <= -W) continue;
        if (grid[dh + G][dw + G] < 0) {
            grid[dh + G][dw + G] = (int8_t)s;
            p.ndistinct++;
        }
        p.rep[s] = grid[dh + G][dw + G];
        for (int l = 0; l < L; l++) {
            const int h = dh + l * eh, w = dw + l * ew;
            if (h < p.hmin) p.hmin = h;
            if (h > p.hmax) p.hmax = h;
            if (w < p.wmin) p.wmin = w;
            if (w > p.wmax) p.wmax = w;
        }
    }
    for (int h = p.hmin; h <= p.hmax; h++)
        for (int w = p.wmin; w <= p.wmax; w++) {
            bool any = false;
            int8_t u[kMaxL] = {};
            for (int l = 0; l < kMaxL; l++) u[l] = -1;
            for (int l = 0; l < L; l++) {
                const int th = h - l * eh + G, tw = w - l * ew + G;
                if (th >= 0 && th < GS && tw >= 0 && tw < GS && grid[th][tw] >= 0) {
                    u[l] = grid[th][tw];
                    any = true;
                }
            }
            if (any) {
                p.sh[p.nsrc] = (int16_t)h;
                p.sw[p.nsrc] = (int16_t)w;
                for (int l = 0; l < kMaxL; l++) p.user[p.nsrc][l] = u[l];
                p.nsrc++;
            }
        }
    return p;
}


// Pair plan, for 16-bit activations.  LDS then holds, at every position, the 32-bit word
// (x[pos], x[pos + e]) -- the element and its neighbour along the step direction -- so one read
// feeds two taps of a run through a dot2 instruction (two multiply-adds into an fp32
// accumulator).  Each run of taps t0, t0+e, t0+2e, ... is cut into pairs from its start;
// pair k of a run, for output l, is the word at t0 + (2k + l) * e.
struct PairPlan {
    int nsrc = 0;                      // distinct word positions per item
    int npair = 0;                     // distinct (tap, next tap) weight pairs
    int16_t sh[kMaxSrc] = {};
    int16_t sw[kMaxSrc] = {};
    int8_t user[kMaxSrc][kMaxL] = {};  // weight pair feeding output l, or -1
    int8_t pair_lo[64] = {};           // representative taps of a weight pair (hi may be -1)
    int8_t pair_hi[64] = {};
    int8_t rep[64] = {};
    int hmin = 0, hmax = 0, wmin = 0, wmax = 0;  // box of the words read and of the neighbours
                                                 // written while staging
};

constexpr PairPlan make_pair_plan(int o, int K, int L, int H, int W) {
    PairPlan p{};
    const int eh = step_h(o), ew = step_w(o);
    constexpr int G = 48, GS = 2 * G + 1;
    int8_t grid[GS][GS] = {};
    int16_t src[GS][GS] = {};
    for (int i = 0; i < GS; i++)
        for (int j = 0; j < GS; j++) grid[i][j] = -1, src[i][j] = -1;
    for (int s = 0; s < K; s++) {
        const int dh = canon_dh(o, K, s), dw = canon_dw(o, K, s);
        p.rep[s] = -1;
        if (dh >= H || dh <= -H || dw >= W || dw <= -W) continue;
        if (grid[dh + G][dw + G] < 0) grid[dh + G][dw + G] = (int8_t)s;
        p.rep[s] = grid[dh + G][dw + G];
    }
    // staging writes x[pos] into the words at pos and pos - e of every interior position
    p.hmin = eh > 0 ? -1 : 0, p.hmax = eh < 0 ? 1 : 0, p.wmin = ew > 0 ? -1 : 0, p.wmax = 0;
    for (int h = -G + 1; h < G; h++)
        for (int w = -G + 1; w < G; w++) {
            if (grid[h + G][w + G] < 0) continue;
            const int ph = h - eh + G, pw = w - ew + G;
            if (ph >= 0 && ph < GS && pw >= 0 && pw < GS && grid[ph][pw] >= 0) continue;  // not a run start
            // walk the run from (h, w)
            int ch = h, cw = w;
            while (ch + G < GS && cw + G < GS && ch + G >= 0 && cw + G >= 0 && grid[ch + G][cw + G] >= 0) {
                const int lo = grid[ch + G][cw + G];
                const int nh = ch + eh, nw = cw + ew;
                const bool has = nh + G < GS && nw + G < GS && nh + G >= 0 && nw + G >= 0 &&
                                 grid[nh + G][nw + G] >= 0;
                const int hi = has ? grid[nh + G][nw + G] : -1;
                const int pid = p.npair++;
                p.pair_lo[pid] = (int8_t)lo;
                p.pair_hi[pid] = (int8_t)hi;
                for (int l = 0; l < L; l++) {
                    const int sh = ch + l * eh, sw = cw + l * ew;
                    if (src[sh + G][sw + G] < 0) {
                        src[sh + G][sw + G] = (int16_t)p.nsrc;
                        p.sh[p.nsrc] = (int16_t)sh;
                        p.sw[p.nsrc] = (int16_t)sw;
                        for (int q = 0; q < kMaxL; q++) p.user[p.nsrc][q] = -1;
                        p.nsrc++;
                    }
                    p.user[src[sh + G][sw + G]][l] = (int8_t)pid;
                    if (sh < p.hmin) p.hmin = sh;
                    if (sh > p.hmax) p.hmax = sh;
                    if (sw < p.wmin) p.wmin = sw;
                    if (sw > p.wmax) p.wmax = sw;
                }
                ch += 2 * eh, cw += 2 * ew;
                if (!has) break;
            }
        }
    return p;
}
constexpr int pair_plan_dot_count(const PairPlan &p, int L) {
    int n = 0;
    for (int m = 0; m < p.nsrc; m++)
        for (int l = 0; l < L; l++) n += p.user[m][l] >= 0 ? 1 : 0;
    return n;
}

constexpr int round_up(int v, int m) { return (v + m - 1) / m * m; }
constexpr int cmax(int a, int b) { return a > b ? a : b; }
constexpr int cmin(int a, int b) { return a < b ? a : b; }

// Smallest r >= need with (mult * r - target) divisible by 32, or need rounded to odd when
// no such r exists within one period.  Used to pick LDS row strides for which the flattened
// item -> address map is linear modulo the 32 banks.
constexpr int bank_stride(int need, int mult, int target) {
    for (int r = need; r < need + 32; r++)
        if ((mult * r - target) % 32 == 0) return r;
    return need | 1;
}

template <bool PAIR>
struct PlanFor {
    static constexpr Plan make(int o, int K, int L, int H, int W) { return make_plan(o, K, L, H, W); }
};
template <>
struct PlanFor<true> {
    static constexpr PairPlan make(int o, int K, int L, int H, int W) {
        return make_pair_plan(o, K, L, H, W);
    }
};

// LDS geometry of one (orientation, K, L, H, W) variant.  All sizes in 32-bit words (floats, or
// element pairs when PAIR).
template <int O, int K, int L, int H, int W, bool PAIR = false>
struct Geo {
    static constexpr int CLS = orient_class(O);
    static constexpr int L_ = L;
    static constexpr int EH = step_h(O), EW = step_w(O);
    static constexpr auto plan = PlanFor<PAIR>::make(O, K, L, H, W);

    static constexpr int LR = CLS == CLS_H ? 1 : L;              // rows per row-block
    static constexpr int RB = (H + LR - 1) / LR;                 // row-blocks per plane
    static constexpr int IPR = CLS == CLS_H ? W / L              // items per row-block
                               : (CLS == CLS_V ? W : round_up(W + L - 1, 8));
    static constexpr int IPP = RB * IPR;                         // items per plane
    static constexpr int P0 = (CLS == CLS_D && EH < 0) ? L - 1 : 0;  // origin row in the block
    static constexpr int PT = cmax(0, -(P0 + plan.hmin));        // zero rows above the plane
    static constexpr int ROWS = cmax(H + PT, (RB - 1) * LR + P0 + plan.hmax + PT + 1);

    // columns
    static constexpr int Q0 = CLS == CLS_D ? L - 1 : 0;  // item j's origin column is j - Q0
    static constexpr int PL =
        CLS == CLS_H ? round_up(cmax(0, -plan.wmin), L) : round_up(cmax(0, Q0 - plan.wmin), 4);
    // H class: a padded row is split into L sub-rows, column u lives in sub-row u % L at u / L
    static constexpr int SUB = (PL + W - 1 + cmax(0, plan.wmax)) / L + 1;
    static constexpr int WIDTH =
        CLS == CLS_H ? L * SUB
                     : (CLS == CLS_V ? PL + W + cmax(0, plan.wmax)
                                     : PL + cmax(W, IPR - Q0) + cmax(0, plan.wmax));
    static constexpr int RS = bank_stride(WIDTH, LR, IPR);
    static constexpr int PLANE = ROWS * RS;  // floats per staged plane

    // LDS offset of column u (already including PL) within a row
    static constexpr int col(int u) { return CLS == CLS_H ? (u % L) * SUB + u / L : u; }
    // immediate offset of source (sh, sw) from the item base  rb*LR*RS + j
    static constexpr int imm(int sh, int sw) {
        return (sh + P0 + PT) * RS + (CLS == CLS_H ? col(sw + PL) : sw + PL - Q0);
    }
    // LDS index of interior element (r, w) of the plane
    static constexpr int interior_row(int r) { return (r + PT) * RS; }
};

// Work decomposition per plane extent: outputs per lane (L) for each orientation class, planes
// staged per batch (PB) and threads per workgroup (NT), chosen so that one batch yields close
// to NT items for every class (items per plane: H class H*W/LH, V class ceil(H/LV)*W, D class
// ceil(H/LD)*round_up(W+LD-1, 8)).
template <int H, int W>
struct Tile {
    static constexpr int LH = W % 4 == 0 ? 4 : (W % 2 == 0 ? 2 : 1);
    static constexpr int LV = LH, LD = LH;
    static constexpr int PB = 1, NT = 256;
};
template <>
struct Tile<56, 56> {  // 784 / 448 / 448 items per plane
    static constexpr int LH = 4, LV = 7, LD = 8, PB = 1, NT = 448;
};
template <>
struct Tile<64, 64> {  // 1024 / 1024 / 1152
    static constexpr int LH = 4, LV = 4, LD = 4, PB = 1, NT = 512;
};
template <>
struct Tile<32, 32> {  // 256 / 256 / 320
    static constexpr int LH = 4, LV = 4, LD = 4, PB = 2, NT = 512;
};
template <>
struct Tile<16, 16> {  // 64 / 64 / 96 (wgrad only: fprop and dgrad run on the register planes)
    static constexpr int LH = 4, LV = 4, LD = 4, PB = 4, NT = 256;
};
template <>
struct Tile<28, 28> {  // 196 / 196 / 224
    static constexpr int LH = 4, LV = 4, LD = 4, PB = 2, NT = 448;
};
template <>
struct Tile<14, 14> {  // 98 / 98 / 112
    static constexpr int LH = 2, LV = 2, LD = 2, PB = 4, NT = 448;
};
template <>
struct Tile<7, 7> {  // 49 / 49 / 56
    static constexpr int LH = 1, LV = 1, LD = 1, PB = 8, NT = 448;
};
template <int H, int W>
constexpr int tile_L(int o) {
    return orient_class(o) == CLS_H ? Tile<H, W>::LH
                                    : (orient_class(o) == CLS_V ? Tile<H, W>::LV : Tile<H, W>::LD);
}

// wgrad has no outputs to store, so its row-direction items need not be a whole number of
// 16-byte chunks: at 56 x 56 seven outputs per item make 448 items per plane, one per thread
// (four make 784: a second pass with a quarter of the lanes idle), and a source feeds up to
// seven running sums instead of four.  Measured with all channels at one angle: 0 degrees
// 46.8 -> 42.3 us; 22.5 degrees (99 sources per item instead of 62) 46.7 -> 55 us, so only the
// horizontal orientation takes it.
template <int H, int W>
constexpr int wgrad_L(int o) {
    return (H == 56 && W == 56 && o == 0) ? 7 : tile_L<H, W>(o);
}

// Planes of at most 16 x 16 are handled in registers, one plane per 16-lane DPP row
// (dwo_regplane.h), instead of being staged in LDS.
constexpr bool reg_plane_shape_rt(int H, int W) { return H <= 16 && W <= 16; }
template <int H, int W>
constexpr bool reg_plane_shape() {
    return reg_plane_shape_rt(H, W);
}

// NHWC slice kernels: a workgroup owns kSliceCh consecutive channels.
constexpr int kSliceCh = 4;
// Plane extents the NHWC slice kernels are built for (four haloed planes per image must fit a
// workgroup's LDS next to the staging of their results); other extents run NHWC on the tile
// kernels.
constexpr bool nhwc_plane_shape_rt(int H, int W) {
    return H == W && (H == 56 || H == 28 || H == 14 || H == 7);
}
template <int H, int W>
constexpr bool nhwc_plane_shape() {
    return nhwc_plane_shape_rt(H, W);
}
// Threads per workgroup and images staged per batch: the planes of a batch must fit in LDS, and
// as many workgroups as possible should be resident per CU (at 14 x 14 one image per batch, four
// workgroups per CU, measured 23 % faster than two images per batch and two workgroups).
template <int H, int W>
struct NhwcTile {
    static constexpr int NT = 256, PBI = 1;
};
template <>
struct NhwcTile<56, 56> {
    static constexpr int NT = 1024, PBI = 1;
};
template <>
struct NhwcTile<28, 28> {
    static constexpr int NT = 512, PBI = 1;
};
template <>
struct NhwcTile<14, 14> {
    static constexpr int NT = 512, PBI = 1;
};
template <>
struct NhwcTile<7, 7> {
    static constexpr int NT = 512, PBI = 4;
};

}  // namespace dwo

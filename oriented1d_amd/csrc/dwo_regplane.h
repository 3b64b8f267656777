// Register-plane NCHW fprop / dgrad kernels for stride 1 on planes of at most 16 x 16 (the
// 14 x 14 and 7 x 7 stages): LDS only as a turntable between the coalesced global accesses and
// the lanes' rows (wave-private and without barriers where a plane is a whole number of
// four-element chunks).  (wgrad of these planes stays on the LDS-staged
// plane kernels: its 32 running sums next to two planes in registers did not fit without
// spilling, and measured slower.)
//
// A plane lives in the registers of one 16-lane DPP row: lane i of the row holds row i of the
// plane (W registers) for the row-direction and diagonal orientations, or column i (H registers)
// for the stacked ones.  A tap (dh, dw) then is a compile-time register index (the offset along
// the registers) plus a DPP row shift by the offset across the lanes, applied as a modifier of
// the multiply-add's source operand: lanes shifted in from outside the 16-lane row read zero
// (bound_ctrl), which is exactly the operator's out-of-image rule, and the unused lanes of a row
// hold zeros.  A wave works on four planes (images n .. n+3 of one channel); the waves of a
// workgroup take consecutive channels of the same images, so a workgroup reads and writes one
// contiguous run of memory per image (whole cache lines when the channel block starts on one),
// each wave running the body of its own channel's orientation.
#pragma once

#include "dwo_common.h"
#include "dwo_dispatch.h"
#include "dwo_plan.h"
#include "dwo_static.h"

namespace dwo {

// Register budget of the NHWC whole-line kernel: its weights differ from row to row of a wave
// and sit in vector registers, which does not fit the 80 registers of six waves per SIMD
// (measured at 384 x 14 x 14 fp32: 21 us with spills at six, 15.0 at five, 13.7 at four).
#ifndef DWO_LINE_WPE
#define DWO_LINE_WPE 4
#endif
constexpr int kRegPlanesPerWave = 4;   // one per 16-lane DPP row
constexpr int kRegWavesPerGroup = 8;   // consecutive channels per workgroup
constexpr int kRegThreads = 64 * kRegWavesPerGroup;

// lanes hold rows for the row-direction and diagonal classes, columns for the stacked ones
constexpr bool reg_lane_is_row(int o) { return orient_class(o) != CLS_V; }

// value of `v` in lane (own lane + SH) of the same 16-lane row, zero beyond the row
template <int SH>
__device__ __forceinline__ float row_shift(float v) {
    if constexpr (SH == 0) {
        return v;
    } else {
        constexpr int ctrl = SH > 0 ? 0x100 + SH : 0x110 - SH;  // row_shl:SH / row_shr:-SH
        return __builtin_bit_cast(
            float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true));
    }
}

// taps of orientation O on an H x W plane: rep[s] = first tap with the same offset (duplicates
// fold into it), -1 for a tap that cannot reach the plane
template <int O, int K, int H, int W>
struct RegPlan {
    static constexpr Plan plan = make_plan(O, K, 1, H, W);
};

// does any live, representative tap of orientation O shift by SH lanes?
template <int O, int K, int H, int W>
constexpr bool reg_shift_used(int sh) {
    for (int s = 0; s < K; s++)
        if (RegPlan<O, K, H, W>::plan.rep[s] == s &&
            (reg_lane_is_row(O) ? canon_dh(O, K, s) : canon_dw(O, K, s)) == sh)
            return true;
    return false;
}

// The four planes of a wave travel between HBM and the registers through a wave-private piece
// of LDS (fp32, planes back to back, no halo): global accesses are whole 16-byte (8-byte for
// 16-bit types) chunks at consecutive addresses from consecutive lanes, whatever way the lanes
// then pick their rows or columns out of LDS.  (Rows fetched from HBM directly, 56 bytes apart
// from lane to lane, ran 1.7 times slower at 14 x 14.)  Only one wave touches the region and a
// wave's LDS operations complete in order, so no barrier is involved.
template <typename T, int H, int W>
struct RegIO {
    static constexpr int E = H * W, VL = E % 4 == 0 ? 4 : 1;
    static constexpr int NCH = E / VL, NIT = (NCH + 63) / 64;
    static constexpr int kWaveFloats = kRegPlanesPerWave * E;
    Chunk<T, VL> reg[kRegPlanesPerWave][NIT];

    // base = plane (n0, c); planes n0 .. n0+nvalid-1 exist, `stride` elements apart
    __device__ __forceinline__ void fetch(const T *__restrict__ base, size_t stride, int nvalid) {
        const unsigned lane = threadIdx.x & 63;
#pragma unroll
        for (int p = 0; p < kRegPlanesPerWave; p++)
#pragma unroll
            for (int it = 0; it < NIT; it++) {
                const unsigned l = lane + 64 * it;
                if (l < NCH && p < nvalid) reg[p][it].load(base + p * stride + l * VL);
            }
    }
    __device__ __forceinline__ void put(float *wl, int nvalid) const {
        const unsigned lane = threadIdx.x & 63;
#pragma unroll
        for (int p = 0; p < kRegPlanesPerWave; p++)
#pragma unroll
            for (int it = 0; it < NIT; it++) {
                const unsigned l = lane + 64 * it;
                if (l < NCH && p < nvalid) {
                    float *q = wl + p * E + l * VL;
                    if constexpr (VL == 4) {
                        typedef float f4 __attribute__((ext_vector_type(4)));
                        *reinterpret_cast<f4 *>(__builtin_assume_aligned(q, 16)) =
                            f4{reg[p][it].get(0), reg[p][it].get(1), reg[p][it].get(2),
                               reg[p][it].get(3)};
                    } else {
                        q[0] = reg[p][it].get(0);
                    }
                }
            }
        __builtin_amdgcn_wave_barrier();
    }
    // results in the wave's LDS region -> HBM
    static __device__ __forceinline__ void write_out(const float *wl, T *__restrict__ base,
                                                     size_t stride, int nvalid) {
        __builtin_amdgcn_wave_barrier();
        const unsigned lane = threadIdx.x & 63;
#pragma unroll
        for (int p = 0; p < kRegPlanesPerWave; p++)
#pragma unroll
            for (int it = 0; it < NIT; it++) {
                const unsigned l = lane + 64 * it;
                if (l < NCH && p < nvalid) {
                    const float *q = wl + p * E + l * VL;
                    if constexpr (VL == 4) {
                        const lds_f4 v = lds_read4(q);
                        Vec4<T> r;
                        r.set(v[0], v[1], v[2], v[3]);
                        r.store(base + p * stride + l * VL);
                    } else {
                        st_out(base + p * stride + l, from_float<T>(q[0]));
                    }
                }
            }
    }
};

// Planes whose size is not a multiple of four elements (7 x 7) travel as single elements per
// lane.  For 16-bit activations those 2-byte accesses cost more than two workgroup barriers
// (7 x 7 bf16: 9.3 us per launch against 7.2 us; fp32 measured 4 % slower this way and keeps the
// barrier-free path): when the channel count is a multiple of the workgroup's eight channels,
// the eight planes of one image are one contiguous, aligned run of 8 * H * W elements, and the
// workgroup moves the runs of its four images as whole four-element chunks, one per thread,
// through all the waves' LDS regions.
template <typename T, int H, int W>
struct GroupIO {
    static constexpr int E = H * W;
    static constexpr bool kUse = E % 4 != 0 && sizeof(T) == 2;  // (8 * E is a multiple of four)
    static constexpr int RUN = kRegWavesPerGroup * E / 4;      // chunks per image
    static constexpr int kWaveFloats = kRegPlanesPerWave * E;
    static_assert(!kUse || kRegPlanesPerWave * RUN <= kRegThreads, "one chunk per thread");
    Vec4<T> reg;

    // LDS index of element `idx` of image p's run: channel idx / E, element idx % E
    static __device__ __forceinline__ unsigned slot(unsigned p, unsigned idx) {
        const unsigned w = idx / E;
        return w * kWaveFloats + p * E + (idx - w * E);
    }
    // base = plane (n0, c0) of the workgroup's first channel
    __device__ __forceinline__ void fetch(const T *__restrict__ base, size_t stride, int nvalid) {
        const unsigned p = threadIdx.x / RUN, i = threadIdx.x % RUN;
        if (p < kRegPlanesPerWave && (int)p < nvalid) reg.load(base + p * stride + i * 4);
    }
    __device__ __forceinline__ void put(float *lds, int nvalid) const {
        const unsigned p = threadIdx.x / RUN, i = threadIdx.x % RUN;
        if (p < kRegPlanesPerWave && (int)p < nvalid) {
#pragma unroll
            for (int e = 0; e < 4; e++) lds[slot(p, i * 4 + e)] = reg.get(e);
        }
        __syncthreads();
    }
    static __device__ __forceinline__ void write_out(const float *lds, T *__restrict__ base,
                                                     size_t stride, int nvalid) {
        __syncthreads();
        const unsigned p = threadIdx.x / RUN, i = threadIdx.x % RUN;
        if (p < kRegPlanesPerWave && (int)p < nvalid) {
            Vec4<T> r;
            r.set(lds[slot(p, i * 4)], lds[slot(p, i * 4 + 1)], lds[slot(p, i * 4 + 2)],
                  lds[slot(p, i * 4 + 3)]);
            r.store(base + p * stride + i * 4);
        }
    }
};

// How the planes of a workgroup (eight channels c0 .. c0+7 of images n0 .. n0+3) travel between
// global memory and the waves' LDS regions; `nvalid` = images of the block that exist.  The
// kernels call start() before they know their orientation, put() before a wave reads its planes
// out of its region `wl` and finish() after it wrote its results there.
//
// NCHW, every wave its own four planes, no workgroup barrier.
template <typename T, int H, int W>
struct WavePlanes {
    static constexpr bool kBarriers = false;
    static constexpr int kPlaneStride = H * W;
    RegIO<T, H, W> io;
    T *out;
    size_t stride;
    __device__ __forceinline__ void start(const T *__restrict__ src, T *__restrict__ dst, int c,
                                          int C, int n0, int nvalid) {
        const size_t off = ((size_t)n0 * C + c) * (H * W);
        stride = (size_t)C * (H * W);
        out = dst + off;
        io.fetch(src + off, stride, nvalid);
    }
    __device__ __forceinline__ void put(float *, float *wl, int nvalid) const { io.put(wl, nvalid); }
    __device__ __forceinline__ void finish(const float *, const float *wl, int nvalid) const {
        RegIO<T, H, W>::write_out(wl, out, stride, nvalid);
    }
};
// NCHW, the workgroup moves its images' runs of eight planes (GroupIO)
template <typename T, int H, int W>
struct GroupPlanes {
    static constexpr bool kBarriers = true;
    static constexpr int kPlaneStride = H * W;
    GroupIO<T, H, W> io;
    T *out;
    size_t stride;
    __device__ __forceinline__ void start(const T *__restrict__ src, T *__restrict__ dst, int c,
                                          int C, int n0, int nvalid) {
        const size_t off = ((size_t)n0 * C + (c - c % kRegWavesPerGroup)) * (H * W);
        stride = (size_t)C * (H * W);
        out = dst + off;
        io.fetch(src + off, stride, nvalid);
    }
    __device__ __forceinline__ void put(float *lds, float *, int nvalid) const { io.put(lds, nvalid); }
    __device__ __forceinline__ void finish(const float *lds, const float *, int nvalid) const {
        GroupIO<T, H, W>::write_out(lds, out, stride, nvalid);
    }
};
// NHWC, 32 channels of one image per workgroup (C a multiple of 32): a pixel's slice is 128 (64)
// contiguous bytes, read as 16 bytes by each of eight (four) lanes, so whole cache lines move.
// DPP row r of wave w holds channel c0 + w + 8 r: with the networks' angle assignments
// (round-robin over eight orientations, or eight contiguous groups) the four channels of a wave
// share their orientation, which the straight-line bodies need.  Planes sit kPlaneStride words
// apart, a stride that is 8 modulo 32: the 64 slices a wave scatters at a time then fall on
// every bank twice, the minimum.
template <typename T, int H, int W>
struct NhwcLinePlanes {
    static constexpr bool kBarriers = true;
    static constexpr int E = H * W;
    static constexpr int kPlaneStride = (E + 23) / 32 * 32 + 8;
    static constexpr int kWaveFloats = kRegPlanesPerWave * kPlaneStride;
    static constexpr int kBlockCh = kRegWavesPerGroup * kRegPlanesPerWave;  // 32
    static constexpr int CPL = 16 / (int)sizeof(T);  // channels per lane: 4 or 8
    static constexpr int LPP = kBlockCh / CPL;       // lanes per pixel: 8 or 4
    static constexpr int NCH = (E * LPP + kRegThreads - 1) / kRegThreads;
    static_assert(kPlaneStride >= E && kPlaneStride % 32 == 8, "plane stride");
    Vec4<T> v[NCH][CPL / 4];
    T *out;
    unsigned C;
    __device__ __forceinline__ bool chunk(int k, unsigned &px, unsigned &sub) const {
        const unsigned t = threadIdx.x + k * kRegThreads;
        px = t / LPP, sub = t % LPP;
        return t < E * LPP;
    }
    // LDS index of channel ch (0 .. 31) of the block at pixel px
    static __device__ __forceinline__ unsigned slot(unsigned ch, unsigned px) {
        return (ch % kRegWavesPerGroup) * kWaveFloats + (ch / kRegWavesPerGroup) * kPlaneStride + px;
    }
    // c0 = first channel of the block, n = the image
    __device__ __forceinline__ void start(const T *__restrict__ src, T *__restrict__ dst, int c0,
                                          int C_, int n, int) {
        C = (unsigned)C_;
        const size_t off = (size_t)n * E * C + c0;
        out = dst + off;
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            unsigned px, sub;
            if (chunk(k, px, sub)) {
                const T *a = src + off + (size_t)px * C + sub * CPL;
#pragma unroll
                for (int q = 0; q < CPL / 4; q++) v[k][q].load_cached(a + 4 * q);
            }
        }
    }
    __device__ __forceinline__ void put(float *lds, float *, int) const {
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            unsigned px, sub;
            if (chunk(k, px, sub)) {
#pragma unroll
                for (int q = 0; q < CPL / 4; q++)
#pragma unroll
                    for (int e = 0; e < 4; e++) lds[slot(sub * CPL + q * 4 + e, px)] = v[k][q].get(e);
            }
        }
        __syncthreads();
    }
    __device__ __forceinline__ void finish(const float *lds, const float *, int) const {
        __syncthreads();
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            unsigned px, sub;
            if (chunk(k, px, sub)) {
                T *o = out + (size_t)px * C + sub * CPL;
#pragma unroll
                for (int q = 0; q < CPL / 4; q++) {
                    const unsigned ch = sub * CPL + q * 4;
                    Vec4<T> r;
                    r.set(lds[slot(ch, px)], lds[slot(ch + 1, px)], lds[slot(ch + 2, px)],
                          lds[slot(ch + 3, px)]);
                    r.store_cached(o + 4 * q);
                }
            }
        }
    }
};

// A plane in registers: lane i of 16-lane row `ps` holds row i (ROW) or column i of plane ps;
// PS = distance between the planes of a wave in its LDS region.
template <bool ROW, int H, int W, int PS = H * W>
struct RegPlane {
    static constexpr int NREG = ROW ? W : H, NLANE = ROW ? H : W;
    float v[NREG];
    // wl = the wave's LDS region; lanes beyond the plane (and the rows of missing planes) hold zeros
    __device__ __forceinline__ void load(const float *wl, unsigned ps, unsigned i, bool plane_ok) {
        const bool live = plane_ok && i < NLANE;
        const float *p = wl + ps * PS + (ROW ? i * W : i);
#pragma unroll
        for (int q = 0; q < NREG; q++) v[q] = live ? p[ROW ? q : q * W] : 0.f;
    }
    __device__ __forceinline__ void store(float *wl, unsigned ps, unsigned i, bool plane_ok) const {
        const bool live = plane_ok && i < NLANE;
        float *p = wl + ps * PS + (ROW ? i * W : i);
        if (live) {
#pragma unroll
            for (int q = 0; q < NREG; q++) p[ROW ? q : q * W] = v[q];
        }
    }
};

// ---------------------------------------------------------------------------------------------
// fprop / dgrad
// ---------------------------------------------------------------------------------------------
// `pio` moves the planes (see WavePlanes); `lds` is the workgroup's whole LDS array, `wl` the
// wave's region of it.  `mine`: this lane's plane exists and has orientation O; `io`
// (wave-uniform): this call also moves the planes (false when a wave makes several passes over
// planes of different orientations and moves them itself).
template <int O, int OP, class PIO, int K, int H, int W>
__device__ __forceinline__ void regplane_conv_body(const float *__restrict__ wt,
                                                   const float *__restrict__ bias, float *lds,
                                                   float *wl, PIO &pio, int c, int nvalid, bool mine,
                                                   bool io) {
    constexpr bool ROW = reg_lane_is_row(O);
    using P = RegPlane<ROW, H, W, PIO::kPlaneStride>;
    constexpr int NREG = P::NREG;
    using RP = RegPlan<O, K, H, W>;  // rep[]: duplicate and dead taps
    const unsigned lane = threadIdx.x & 63, i = lane & 15, ps = lane >> 4;

    // weights with duplicates folded into their representative tap (dgrad: reversed, the
    // offsets are odd-symmetric)
    float w[K];
#pragma unroll
    for (int s = 0; s < K; s++) w[s] = wt[(size_t)c * K + (OP == OP_DGRAD ? K - 1 - s : s)];
    static_for<K>([&](auto s) {
        constexpr int r = RP::plan.rep[s];
        if constexpr (r >= 0 && r != s) w[r] += w[s];
    });
    const float bv = (OP == OP_FPROP && bias != nullptr) ? bias[c] : 0.f;
    if (io) pio.put(lds, wl, nvalid);
    P x;
    x.load(wl, ps, i, mine);
    // (results go back into the wave's own region, which only this wave reads before finish())
    // Shift by shift: the plane shifted by SH lanes (one DPP move per register), then every
    // multiply-add whose tap has that shift.  The empty asm at the end of a shift pins the
    // running sums there, so the shifted copies die with their shift (left to itself the
    // compiler makes the copies of all shifts first and spills them).
    P y;
#pragma unroll
    for (int q = 0; q < NREG; q++) y.v[q] = bv;
    static_for<31>([&](auto idx) {
        constexpr int sh = idx - 15;
        if constexpr (reg_shift_used<O, K, H, W>(sh)) {
            float xs[NREG];
#pragma unroll
            for (int j = 0; j < NREG; j++) xs[j] = row_shift<sh>(x.v[j]);
            static_for<K>([&](auto s) {
                if constexpr (RP::plan.rep[s] == s && (ROW ? canon_dh(O, K, s) : canon_dw(O, K, s)) == sh) {
                    constexpr int o = ROW ? canon_dw(O, K, s) : canon_dh(O, K, s);
                    static_for<NREG>([&](auto q) {
                        constexpr int j = q + o;
                        if constexpr (j >= 0 && j < NREG) y.v[q] = __builtin_fmaf(xs[j], w[s], y.v[q]);
                    });
                }
            });
#pragma unroll
            for (int q = 0; q < NREG; q++) asm volatile("" : "+v"(y.v[q]));
        }
    });
    y.store(wl, ps, i, mine);
    if (io) pio.finish(lds, wl, nvalid);
}

// any angle: same plane movement; lane i of row ps gathers row i of plane ps from the wave's
// LDS region with the taps of the device table (rare: the networks only use the canonical
// orientations)
template <int OP, class PIO, int K, int H, int W>
__device__ __forceinline__ void regplane_conv_table(const float *__restrict__ wt,
                                                    const float *__restrict__ bias,
                                                    const int8_t *__restrict__ dhdw, float *lds,
                                                    float *wl, PIO &pio, int c, int nvalid, bool mine,
                                                    bool io) {
    const unsigned lane = threadIdx.x & 63, i = lane & 15, ps = lane >> 4;
    if (io) pio.put(lds, wl, nvalid);
    const float bv = (OP == OP_FPROP && bias != nullptr) ? bias[c] : 0.f;
    const bool live = mine && i < H;
    const float *plane = wl + ps * PIO::kPlaneStride;
    float y[W];
#pragma unroll
    for (int q = 0; q < W; q++) y[q] = bv;
    for (int s = 0; s < K; s++) {
        const int sgn = OP == OP_DGRAD ? -1 : 1;
        const int dh = sgn * dhdw[((size_t)c * K + s) * 2], dw = sgn * dhdw[((size_t)c * K + s) * 2 + 1];
        const float ws = wt[(size_t)c * K + s];
        const int h = (int)i + dh;
        if (live && h >= 0 && h < H) {
#pragma unroll
            for (int q = 0; q < W; q++) {
                const int ww = q + dw;
                if (ww >= 0 && ww < W) y[q] = __builtin_fmaf(plane[h * W + ww], ws, y[q]);
            }
        }
    }
    // every lane of the wave has read its sources before any row is overwritten
    __builtin_amdgcn_wave_barrier();
    if (live) {
#pragma unroll
        for (int q = 0; q < W; q++) wl[ps * PIO::kPlaneStride + i * W + q] = y[q];
    }
    if (io) pio.finish(lds, wl, nvalid);
}

// one wave: planes of channel c (wave-uniform, or one channel per 16-lane row), orientation
// class cls (8 and above: table-driven body), wave-uniform; PIO::start has been called
template <int OP, class PIO, int K, int H, int W>
__device__ __forceinline__ void regplane_dispatch(const float *__restrict__ wt,
                                                  const float *__restrict__ bias,
                                                  const void *__restrict__ blob, float *lds,
                                                  float *wl, PIO &pio, int c, int cls, int nvalid,
                                                  bool mine, bool io) {
#define DWO_CASE(O)                                                                              \
    case O:                                                                                      \
        regplane_conv_body<O, OP, PIO, K, H, W>(wt, bias, lds, wl, pio, c, nvalid, mine, io); \
        break;
    switch (cls) {
        DWO_CASE(0)
        DWO_CASE(1)
        DWO_CASE(2)
        DWO_CASE(3)
        DWO_CASE(4)
        DWO_CASE(5)
        DWO_CASE(6)
        DWO_CASE(7)
        default:
            regplane_conv_table<OP, PIO, K, H, W>(wt, bias, taps_dhdw(blob), lds, wl, pio, c, nvalid,
                                                  mine, io);
    }
#undef DWO_CASE
}

// Blocks of four images a wave of regplane_kernel works through.  The smallest planes have so
// little arithmetic per block that one block per wave leaves every wave waiting out its own HBM
// latency; the workgroup-barrier path (GroupPlanes) keeps one block.
#ifndef DWO_REG_BLOCKS
#define DWO_REG_BLOCKS 2
#endif
template <typename T, int H, int W>
constexpr int reg_blocks_per_wave() {
    return (!GroupIO<T, H, W>::kUse && H * W <= 64) ? DWO_REG_BLOCKS : 1;
}

template <int OP, typename T, int K, int H, int W>
__global__ __launch_bounds__(kRegThreads) __attribute__((amdgpu_waves_per_eu(6, 8))) void regplane_kernel(
    const T *__restrict__ src, const float *__restrict__ wt, const float *__restrict__ bias,
    const void *__restrict__ blob, T *__restrict__ dst, int N, int C) {
    // (wave-uniform: the weights and the class are fetched with scalar loads)
    const int c = blockIdx.x * kRegWavesPerGroup + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    __shared__ __align__(16) float lds[kRegWavesPerGroup * RegIO<T, H, W>::kWaveFloats];
    float *wl = lds + (threadIdx.x >> 6) * RegIO<T, H, W>::kWaveFloats;
    const int n0 = blockIdx.y * kRegPlanesPerWave * reg_blocks_per_wave<T, H, W>();
    if constexpr (GroupIO<T, H, W>::kUse) {
        // (uniform over the grid: with whole channel blocks no wave leaves before the barriers)
        if (C % kRegWavesPerGroup == 0) {
            GroupPlanes<T, H, W> pio;
            pio.start(src, dst, c, C, n0, N - n0);
            const int cls = __builtin_amdgcn_readfirstlane(taps_class(blob, C, K)[c]);
            regplane_dispatch<OP, GroupPlanes<T, H, W>, K, H, W>(
                wt, bias, blob, lds, wl, pio, c, cls, N - n0,
                (int)((threadIdx.x & 63) >> 4) < N - n0, true);
            return;
        }
    }
    if (c >= C) return;  // whole wave; this path has no workgroup barriers
    // kRegBlocksPerWave image blocks per wave, all fetched up front: the later blocks' HBM latency
    // overlaps the earlier ones' arithmetic (the wave's LDS region is reused block after block;
    // a wave's LDS operations complete in order)
    constexpr int NB = reg_blocks_per_wave<T, H, W>();
    WavePlanes<T, H, W> pio[NB];
#pragma unroll
    for (int q = 0; q < NB; q++)
        if (n0 + q * kRegPlanesPerWave < N)
            pio[q].start(src, dst, c, C, n0 + q * kRegPlanesPerWave, N - n0 - q * kRegPlanesPerWave);
    const int cls = __builtin_amdgcn_readfirstlane(taps_class(blob, C, K)[c]);
#pragma unroll
    for (int q = 0; q < NB; q++) {
        const int left = N - n0 - q * kRegPlanesPerWave;
        if (left > 0)
            regplane_dispatch<OP, WavePlanes<T, H, W>, K, H, W>(
                wt, bias, blob, lds, wl, pio[q], c, cls, left, (int)((threadIdx.x & 63) >> 4) < left, true);
    }
}

// NHWC tensors, C a multiple of 32: workgroup = 32 channels of one image (NhwcLinePlanes)
template <int OP, typename T, int K, int H, int W>
__global__ __launch_bounds__(kRegThreads) __attribute__((amdgpu_waves_per_eu(DWO_LINE_WPE, 8))) void regplane_nhwc_line_kernel(
    const T *__restrict__ src, const float *__restrict__ wt, const float *__restrict__ bias,
    const void *__restrict__ blob, T *__restrict__ dst, int N, int C) {
    using PIO = NhwcLinePlanes<T, H, W>;
    __shared__ __align__(16) float lds[kRegWavesPerGroup * PIO::kWaveFloats];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float *wl = lds + wave * PIO::kWaveFloats;
    // Workgroup -> (channel block, image).  With 2-byte elements a block's pixel slices are half
    // cache lines, and the other halves belong to the neighbouring channel block: hardware hands
    // consecutive workgroup ids to the eight XCDs round-robin, so inside every aligned run of 16
    // ids the two workgroups an XCD receives take neighbouring tasks, i.e. (with an even number
    // of channel blocks) the two halves of the same lines, and the second one finds them in
    // that XCD's L2.
    unsigned task = blockIdx.x + blockIdx.y * gridDim.x;
    if (sizeof(T) == 2 && (task | 15u) < gridDim.x * gridDim.y)
        task = (task & ~15u) + 2 * (task & 7u) + ((task >> 3) & 1u);
    const int block_x = task % gridDim.x, image = task / gridDim.x;
    const int c0 = block_x * PIO::kBlockCh;
    const int c = c0 + wave + kRegWavesPerGroup * (int)((threadIdx.x & 63) >> 4);  // per 16-lane row
    PIO pio;
    pio.start(src, dst, c0, C, image, kRegPlanesPerWave);
    // The straight-line bodies need one orientation per pass.  A wave whose four channels share
    // theirs (the usual case) makes one pass that also moves the planes; otherwise it moves them
    // itself and makes one pass per distinct class, each over the rows of that class only.
    // (One loop, not unrolled, for both cases: every pass site is a copy of all nine bodies.)
    const int cls_row = taps_class(blob, C, K)[c];
    constexpr int NP = kRegPlanesPerWave;
    const bool uniform = __ballot(cls_row != __builtin_amdgcn_readfirstlane(cls_row)) == 0;
    if (!uniform) pio.put(lds, wl, NP);
#pragma nounroll
    for (int r = 0; r < (uniform ? 1 : NP); r++) {
        const int cls = __builtin_amdgcn_readlane(cls_row, 16 * r);
        bool done = false;
        for (int q = 0; q < r; q++) done = done || __builtin_amdgcn_readlane(cls_row, 16 * q) == cls;
        if (!done)
            regplane_dispatch<OP, PIO, K, H, W>(wt, bias, blob, lds, wl, pio, c, cls, NP,
                                                uniform || cls_row == cls, uniform);
    }
    if (!uniform) pio.finish(lds, wl, NP);
}

// ---------------------------------------------------------------------------------------------
// host launcher (same contract as launch_plane_conv)
// ---------------------------------------------------------------------------------------------
template <typename T, int K, int H, int W>
int launch_regplane_conv(int op, const void *src, const float *w, const float *bias,
                         const void *taps, void *dst, int N, int C, hipStream_t st) {
    if (N == 0) return 0;  // set-up only: nothing to prepare
    constexpr int per_wave = kRegPlanesPerWave * reg_blocks_per_wave<T, H, W>();
    const dim3 grid((C + kRegWavesPerGroup - 1) / kRegWavesPerGroup, (N + per_wave - 1) / per_wave),
        block(kRegThreads);
    if (grid.y > 65535) return -100;  // not covered: the dispatch goes on to the tile kernels
    if (op == OP_FPROP)
        regplane_kernel<OP_FPROP, T, K, H, W><<<grid, block, 0, st>>>((const T *)src, w, bias, taps,
                                                                     (T *)dst, N, C);
    else
        regplane_kernel<OP_DGRAD, T, K, H, W><<<grid, block, 0, st>>>((const T *)src, w, bias, taps,
                                                                     (T *)dst, N, C);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

// NHWC; the caller has checked that C is a multiple of NhwcLinePlanes::kBlockCh
template <typename T, int K, int H, int W>
int launch_regplane_nhwc_conv(int op, const void *src, const float *w, const float *bias,
                              const void *taps, void *dst, int N, int C, hipStream_t st) {
    if (N == 0) return 0;
    if (N > 65535) return DWO_ERR_BAD_SHAPE;
    const dim3 grid(C / NhwcLinePlanes<T, H, W>::kBlockCh, N), block(kRegThreads);
    if (op == OP_FPROP)
        regplane_nhwc_line_kernel<OP_FPROP, T, K, H, W><<<grid, block, 0, st>>>((const T *)src, w, bias,
                                                                               taps, (T *)dst, N, C);
    else
        regplane_nhwc_line_kernel<OP_DGRAD, T, K, H, W><<<grid, block, 0, st>>>((const T *)src, w, bias,
                                                                               taps, (T *)dst, N, C);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

}  // namespace dwo

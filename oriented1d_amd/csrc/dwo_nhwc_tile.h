// NHWC fprop for any plane extent and stride (channel count a multiple of 4): the stem
// convolutions of the ConvNeXt-1D networks (224 -> 112 -> 56, stride 2) and every other NHWC
// shape without compile-time planes.
//
// A workgroup owns four consecutive channels of a band of output rows of one image and walks
// the band in sub-tiles.  Per sub-tile it loads the pixel slices of the input window (8 or 16
// bytes per pixel), stores them as one plane per channel in LDS in the activation's own type
// (out-of-image positions as zeros), lets sub-group k (128 threads) evaluate channel k's taps
// for the sub-tile's outputs from that plane, and writes the results back as pixel slices.
// The sub-tile shape is chosen per workgroup from its channels' tap extents: wide row strips
// for near-horizontal taps, tall column strips for near-vertical ones, squares in between, so
// the window read per output stays small for every orientation.  The extents are bounded by
// K / 2 in each direction, whatever the angles.
#pragma once

#include "dwo_static.h"

namespace dwo {

constexpr int kTileThreads = 512;                          // four sub-groups of two waves
constexpr int kTileSub = kTileThreads / kSliceCh;          // threads per channel
constexpr int kTilePlaneElems = 7680;                      // LDS elements per channel plane (two
                                                           // workgroups of 16-bit planes per CU)
constexpr int kTileOutputs = 1024;                         // most outputs per sub-tile
constexpr int kTileBandRows = 32;                          // output rows per workgroup

// planes, fp32 results, per-channel tap table (offset, weight) and tap extents
template <typename T>
constexpr size_t nhwc_tile_lds_bytes() {
    return (size_t)kSliceCh * kTilePlaneElems * sizeof(T) + (size_t)kSliceCh * kTileOutputs * 4 +
           (size_t)kSliceCh * DWO_MAX_K * 8 + 64;
}

// One pixel slice at byte offset `off` of a raw buffer descriptor (zeros when off lies outside).
__device__ __forceinline__ void slice_load(Vec4<float> &v, __amdgpu_buffer_rsrc_t r, unsigned off) {
    v.v = __builtin_bit_cast(Vec4<float>::f4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
}
__device__ __forceinline__ void slice_load(Vec4<bf16_t> &v, __amdgpu_buffer_rsrc_t r, unsigned off) {
    v.v = __builtin_bit_cast(Vec4<bf16_t>::u2, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
}
__device__ __forceinline__ void slice_load(Vec4<f16_t> &v, __amdgpu_buffer_rsrc_t r, unsigned off) {
    v.v = __builtin_bit_cast(Vec4<f16_t>::h4, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
}

// floor(n / d) for n < 2^16 and 2 <= d < 2^16, with m = ceil(2^32 / d)
__device__ __forceinline__ unsigned fast_div(unsigned n, unsigned m) { return __umulhi(n, m); }
__device__ __forceinline__ unsigned div_magic(unsigned d) {
    return (unsigned)((0x100000000ull + d - 1) / d);
}

template <typename T>
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void nhwc_tile_fprop_kernel(
    const T *__restrict__ x, const float *__restrict__ wt, const float *__restrict__ bias,
    const int8_t *__restrict__ dhdw, T *__restrict__ y, ConvDims d, int nbands, int tasks_per_image) {
    extern __shared__ float lds_f[];
    T *planes = reinterpret_cast<T *>(lds_f);
    float *lout = reinterpret_cast<float *>(planes + kSliceCh * kTilePlaneElems);
    int2 *tapt = reinterpret_cast<int2 *>(lout + kSliceCh * kTileOutputs);  // [ch][K] (offset, weight)
    int *halo = reinterpret_cast<int *>(tapt + kSliceCh * DWO_MAX_K);       // [ch][2]

    // image n of XCD n % 8: hardware deals consecutive workgroup ids to the XCDs in turn, so the
    // slices and bands of one image share one L2
    const int xcd = blockIdx.x % 8, local = blockIdx.x / 8;
    const int n = xcd + 8 * (local / tasks_per_image);
    if (n >= d.N) return;
    const int task = local % tasks_per_image;
    const int nslices = d.C / kSliceCh;
    const int slice = task % nslices, band = task / nslices;
    const int c0 = slice * kSliceCh;
    const int sub = __builtin_amdgcn_readfirstlane(threadIdx.x / kTileSub);
    const unsigned stid = threadIdx.x % kTileSub;
    const int c = c0 + sub;
    const int s_ = d.stride, K = d.K;

    // tap extents of this sub-group's channel (uniform), then of the four channels together
    const int8_t *mytaps = dhdw + (size_t)c * K * 2;
    int hh = 0, hw = 0;
    for (int s = 0; s < K; s++) {
        hh = max(hh, abs((int)mytaps[2 * s]));
        hw = max(hw, abs((int)mytaps[2 * s + 1]));
    }
    if (stid == 0) halo[sub * 2] = hh, halo[sub * 2 + 1] = hw;
    __syncthreads();
    hh = max(max(halo[0], halo[2]), max(halo[4], halo[6]));
    hw = max(max(halo[1], halo[3]), max(halo[5], halo[7]));
    hh = __builtin_amdgcn_readfirstlane(hh);
    hw = __builtin_amdgcn_readfirstlane(hw);
    const float bv = bias != nullptr ? bias[c] : 0.f;

    // Window rows/columns step by the stride when no tap of the slice leaves its row/column
    // (0 and 90 degrees): the positions in between are never read.
    const int rstep = hh == 0 ? s_ : 1, cstep = hw == 0 ? s_ : 1;
    const int srow = s_ / rstep, scol = s_ / cstep;  // plane rows/columns per output row/column

    // sub-tile shape: th rows x tw columns of outputs; window ih x iw of inputs.  Cost per
    // output = window positions plus a fixed per-sub-tile charge (barriers, pipeline fill).
    // (widths of at least 2, also for a one-column plane: the index arithmetic divides by them)
    const int p_lo = band * kTileBandRows, p_hi = min(d.P, p_lo + kTileBandRows);
    const int RH = p_hi - p_lo;
    const int Qe = max(d.Q, 2);
    int th = 1, tw = 2;
    {
        float best = 1e30f;
        for (int a = RH; a >= 1; a = (a + 1) / 2) {
            for (int k = 0; k < 6; k++) {
                const int b = k == 0 ? Qe : (256 >> k);  // full width, 128, 64, 32, 16, 8
                if (b > Qe || a * b > kTileOutputs) continue;
                const int ih = (a - 1) * srow + 1 + 2 * hh, iw = ((b - 1) * scol + 1 + 2 * hw) | 1;
                if (ih * iw > kTilePlaneElems) continue;
                const float cost = (float)(ih * iw + 1536) / (float)(a * b);
                if (cost < best) best = cost, th = a, tw = b;
            }
            if (a == 1) break;
        }
    }
    const int ih = (th - 1) * srow + 1 + 2 * hh;
    const int iw = (tw - 1) * scol + 1 + 2 * hw;
    const int iwp = iw | 1;
    const unsigned m_iw = div_magic(iw), m_tw = div_magic(tw);
    // the channel's taps as (LDS element offset, weight) pairs, read back as broadcasts
    int2 *mytab = tapt + sub * DWO_MAX_K;
    if ((int)stid < K)
        mytab[stid] = make_int2(((int)mytaps[2 * stid] / rstep) * iwp + (int)mytaps[2 * stid + 1] / cstep,
                                __float_as_int(wt[(size_t)c * K + stid]));

    const T *xn = x + (size_t)n * d.H * d.W * d.C + c0;
    T *yn = y + (size_t)n * d.P * d.Q * d.C + c0;
    const T *plane = planes + sub * kTilePlaneElems;
    const unsigned nwin = ih * iw, nout = th * tw;

    // window of sub-tile (pt, qt) -> registers: rows pt*s - hh .., columns qt*s - hw ..
    // (through a buffer descriptor over the image: positions outside it get an offset beyond
    // the descriptor and read as zeros, so the loads need no predicates)
    constexpr int PRE = kTilePlaneElems / kTileThreads;  // slices per thread, at most
    Vec4<T> pre[PRE];
    const __amdgpu_buffer_rsrc_t img = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T *>(xn), 0, (unsigned)(((size_t)d.H * d.W * d.C - c0) * sizeof(T)), 0x00020000);
    auto load_window = [&](int pt, int qt) {
        const int r0 = pt * s_ - hh, q0 = qt * s_ - hw;
#pragma unroll
        for (int u = 0; u < PRE; u++) {
            if (u * kTileThreads >= (int)nwin) break;
            unsigned v = u * kTileThreads + threadIdx.x;
            asm volatile("" : "+v"(v));  // recompute per window: hoisting 16 index sets spills
            const unsigned i = fast_div(v, m_iw), j = v - i * iw;
            const unsigned r = (unsigned)(r0 + (int)i * rstep), q = (unsigned)(q0 + (int)j * cstep);
            const bool inside = v < nwin && r < (unsigned)d.H && q < (unsigned)d.W;
            slice_load(pre[u], img, inside ? (r * d.W + q) * d.C * (unsigned)sizeof(T) : 0xffffffffu);
        }
    };
    load_window(p_lo, 0);
    for (int pt = p_lo; pt < p_hi; pt += th) {
        for (int qt = 0; qt < d.Q; qt += tw) {
#pragma unroll
            for (int u = 0; u < PRE; u++) {
                if (u * kTileThreads >= (int)nwin) break;
                unsigned v = u * kTileThreads + threadIdx.x;
                asm volatile("" : "+v"(v));
                if (v < nwin) {
                    const unsigned i = fast_div(v, m_iw), j = v - i * iw;
                    const unsigned at = i * iwp + j;
#pragma unroll
                    for (int ch = 0; ch < kSliceCh; ch++)
                        planes[ch * kTilePlaneElems + at] = pre[u].elem(ch);
                }
            }
            __syncthreads();
            // the next window travels while this one is being evaluated
            if (qt + tw < d.Q)
                load_window(pt, qt + tw);
            else if (pt + th < p_hi)
                load_window(pt + th, 0);
            // sub-group: one channel; a thread takes four outputs at a time so that each tap's
            // (offset, weight) is fetched once for the four
            for (unsigned o0 = stid; o0 < nout; o0 += 4 * kTileSub) {
                const T *base[4];
                float acc[4];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const unsigned o = min(o0 + k * kTileSub, nout - 1);
                    const unsigned pl = fast_div(o, m_tw), ql = o - pl * tw;
                    base[k] = plane + ((pl * srow + hh) * iwp + ql * scol + hw);
                    acc[k] = bv;
                }
#pragma unroll 4
                for (int s = 0; s < K; s++) {
                    const int2 t = mytab[s];
                    const float w = __int_as_float(t.y);
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        acc[k] = __builtin_fmaf(to_float(base[k][t.x]), w, acc[k]);
                }
#pragma unroll
                for (int k = 0; k < 4; k++)
                    if (o0 + k * kTileSub < nout) lout[sub * kTileOutputs + o0 + k * kTileSub] = acc[k];
            }
            __syncthreads();
            for (unsigned o = threadIdx.x; o < nout; o += kTileThreads) {
                const unsigned pl = fast_div(o, m_tw), ql = o - pl * tw;
                const int p = pt + (int)pl, q = qt + (int)ql;
                if (p < p_hi && q < d.Q) {
                    Vec4<T> out;
                    out.set(lout[o], lout[kTileOutputs + o], lout[2 * kTileOutputs + o],
                            lout[3 * kTileOutputs + o]);
                    out.store_cached(yn + ((size_t)p * d.Q + q) * d.C);
                }
            }
        }
    }
}

// grid: 8 * ceil(N / 8) * bands * slices workgroups
template <typename T>
int launch_nhwc_tile_fprop(const void *x, const float *w, const float *bias, const void *taps,
                           void *y, const ConvDims &d, hipStream_t st) {
    const size_t lds = nhwc_tile_lds_bytes<T>();
    static const bool once = [&] {
        allow_large_lds(nhwc_tile_fprop_kernel<T>, lds);
        return true;
    }();
    (void)once;
    const int nbands = (d.P + kTileBandRows - 1) / kTileBandRows;
    const int tpi = nbands * (d.C / kSliceCh);
    const long grid = 8L * ((d.N + 7) / 8) * tpi;
    if (grid > 0x7fffffffL) return DWO_ERR_BAD_SHAPE;
    nhwc_tile_fprop_kernel<T><<<dim3((unsigned)grid), dim3(kTileThreads), lds, st>>>(
        (const T *)x, w, bias, taps_dhdw(taps), (T *)y, d, nbands, tpi);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

}  // namespace dwo

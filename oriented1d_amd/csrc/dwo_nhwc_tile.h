// fprop (and, with reversed weights, stride-1 dgrad) for any plane extent, stride and kernel
// size: the stem convolutions of the ConvNeXt-1D networks (NHWC, 224 -> 112 -> 56, stride 2),
// the stages of inputs other than 224 x 224 (NCHW), and every other shape without compile-time
// planes.  NHWC needs a channel count that is a multiple of 4.  Described for NHWC; NCHW differs
// only in how the window is loaded and the results are stored (PlaneSource).
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

// Where the window's pixels come from.  SliceSource: an NHWC tensor with the convolution's own
// channel count; a pixel's payload is the workgroup's four-channel slice.  PointwiseSource: an
// NHWC tensor of CIN channels (the network's input image) to which a pointwise linear layer
// CIN -> C is applied on the way into LDS (the stem's first layer, models/convnext.py:143,177:
// the C-channel tensor is never written to memory); out-of-image positions are zeros of the
// *projected* tensor, and the projection is rounded to the activation type as the separate layer's
// output would be.
template <typename T>
struct SliceSource {
    static constexpr bool kNchw = false;
    typedef Vec4<T> Payload;
    struct Params {
        const T *x;
    };
    __amdgpu_buffer_rsrc_t img;
    unsigned pix_bytes;
    __device__ __forceinline__ void init(const Params &p, int n, int c0, const ConvDims &d) {
        const T *xn = p.x + (size_t)n * d.H * d.W * d.C + c0;
        img = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<T *>(xn), 0, (unsigned)(((size_t)d.H * d.W * d.C - c0) * sizeof(T)), 0x00020000);
        pix_bytes = d.C * (unsigned)sizeof(T);
    }
    // (positions outside the image get an offset beyond the descriptor and read as zeros, so the
    // loads need no predicates)
    __device__ __forceinline__ void load(Payload &v, bool inside, unsigned pixel) const {
        slice_load(v, img, inside ? pixel * pix_bytes : 0xffffffffu);
    }
    __device__ __forceinline__ T elem(const Payload &v, int ch, bool) const { return v.elem(ch); }
};

__device__ __forceinline__ float buffer_value(__amdgpu_buffer_rsrc_t r, unsigned off, float);
__device__ __forceinline__ float buffer_value(__amdgpu_buffer_rsrc_t r, unsigned off, bf16_t);
__device__ __forceinline__ float buffer_value(__amdgpu_buffer_rsrc_t r, unsigned off, f16_t);

// PlaneSource: an NCHW tensor; a pixel's payload is one element from each of the workgroup's
// four channel planes (consecutive lanes read consecutive pixels of a row, so every plane's
// loads are contiguous).  Channels beyond C (a last, partial group of four) read as zeros.
template <typename T>
struct PlaneSource {
    static constexpr bool kNchw = true;
    struct Payload {
        float v[kSliceCh];
    };
    struct Params {
        const T *x;
    };
    __amdgpu_buffer_rsrc_t img;
    unsigned plane_bytes, c0_bytes;
    __device__ __forceinline__ void init(const Params &p, int n, int c0, const ConvDims &d) {
        const T *xn = p.x + (size_t)n * d.C * d.H * d.W;
        img = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<T *>(xn), 0, (unsigned)((size_t)d.C * d.H * d.W * sizeof(T)), 0x00020000);
        plane_bytes = (unsigned)(d.H * d.W) * (unsigned)sizeof(T);
        c0_bytes = (unsigned)c0 * plane_bytes;
    }
    __device__ __forceinline__ void load(Payload &v, bool inside, unsigned pixel) const {
#pragma unroll
        for (int ch = 0; ch < kSliceCh; ch++)
            v.v[ch] = buffer_value(
                img, inside ? c0_bytes + ch * plane_bytes + pixel * (unsigned)sizeof(T) : 0xffffffffu, T{});
    }
    __device__ __forceinline__ T elem(const Payload &v, int ch, bool) const {
        return from_float<T>(v.v[ch]);  // exact: the value came from a T
    }
};

__device__ __forceinline__ float buffer_value(__amdgpu_buffer_rsrc_t r, unsigned off, float) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
}
__device__ __forceinline__ float buffer_value(__amdgpu_buffer_rsrc_t r, unsigned off, bf16_t) {
    return __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0) << 16);
}
__device__ __forceinline__ float buffer_value(__amdgpu_buffer_rsrc_t r, unsigned off, f16_t) {
    return (float)__builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0));
}

template <typename T, int CIN>
struct PointwiseSource {
    static constexpr bool kNchw = false;
    struct Payload {
        float v[CIN];
    };
    struct Params {
        const T *x;         // [N,H,W,CIN]
        const float *pw_w;  // [C,CIN]
        const float *pw_b;  // [C] or null
    };
    __amdgpu_buffer_rsrc_t img;
    float w[kSliceCh][CIN], b[kSliceCh];
    __device__ __forceinline__ void init(const Params &p, int n, int c0, const ConvDims &d) {
        const T *xn = p.x + (size_t)n * d.H * d.W * CIN;
        img = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<T *>(xn), 0, (unsigned)((size_t)d.H * d.W * CIN * sizeof(T)), 0x00020000);
#pragma unroll
        for (int ch = 0; ch < kSliceCh; ch++) {
            b[ch] = p.pw_b != nullptr ? p.pw_b[c0 + ch] : 0.f;
#pragma unroll
            for (int k = 0; k < CIN; k++) w[ch][k] = p.pw_w[(size_t)(c0 + ch) * CIN + k];
        }
    }
    __device__ __forceinline__ void load(Payload &v, bool inside, unsigned pixel) const {
#pragma unroll
        for (int k = 0; k < CIN; k++)
            v.v[k] = buffer_value(img, inside ? (pixel * CIN + k) * (unsigned)sizeof(T) : 0xffffffffu, T{});
    }
    __device__ __forceinline__ T elem(const Payload &v, int ch, bool inside) const {
        float a = b[ch];
#pragma unroll
        for (int k = 0; k < CIN; k++) a = __builtin_fmaf(v.v[k], w[ch][k], a);
        return inside ? from_float<T>(a) : T{};
    }
};

// floor(n / d) for n < 2^16 and 2 <= d < 2^16, with m = ceil(2^32 / d)
__device__ __forceinline__ unsigned fast_div(unsigned n, unsigned m) { return __umulhi(n, m); }
__device__ __forceinline__ unsigned div_magic(unsigned d) {
    return (unsigned)((0x100000000ull + d - 1) / d);
}

template <typename T, class Src>
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void nhwc_tile_fprop_kernel(
    typename Src::Params sp, const float *__restrict__ wt, const float *__restrict__ bias,
    const int8_t *__restrict__ dhdw, T *__restrict__ y, ConvDims d, int nbands, int tasks_per_image,
    int flip) {
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
    const int nslices = (d.C + kSliceCh - 1) / kSliceCh;
    const int slice = task % nslices, band = task / nslices;
    const int c0 = slice * kSliceCh;
    const int sub = __builtin_amdgcn_readfirstlane(threadIdx.x / kTileSub);
    const unsigned stid = threadIdx.x % kTileSub;
    const int c = min(c0 + sub, d.C - 1);  // (a partial last group repeats its last channel)
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
                                __float_as_int(wt[(size_t)c * K + (flip ? K - 1 - (int)stid : (int)stid)]));

    T *yn = Src::kNchw ? y + ((size_t)n * d.C + c0) * d.P * d.Q : y + (size_t)n * d.P * d.Q * d.C + c0;
    const T *plane = planes + sub * kTilePlaneElems;
    const unsigned nwin = ih * iw, nout = th * tw;

    // window of sub-tile (pt, qt) -> registers: rows pt*s - hh .., columns qt*s - hw ..
    constexpr int PRE = kTilePlaneElems / kTileThreads;  // pixels per thread, at most
    typename Src::Payload pre[PRE];
    Src source;
    source.init(sp, n, c0, d);
    auto window_pixel = [&](int pt, int qt, unsigned v, unsigned &pixel) {
        const unsigned i = fast_div(v, m_iw), j = v - i * iw;
        const unsigned r = (unsigned)(pt * s_ - hh + (int)i * rstep);
        const unsigned q = (unsigned)(qt * s_ - hw + (int)j * cstep);
        pixel = r * d.W + q;
        return v < nwin && r < (unsigned)d.H && q < (unsigned)d.W;
    };
    auto load_window = [&](int pt, int qt) {
#pragma unroll
        for (int u = 0; u < PRE; u++) {
            if (u * kTileThreads >= (int)nwin) break;
            unsigned v = u * kTileThreads + threadIdx.x;
            asm volatile("" : "+v"(v));  // recompute per window: hoisting 16 index sets spills
            unsigned pixel;
            const bool inside = window_pixel(pt, qt, v, pixel);
            source.load(pre[u], inside, pixel);
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
                    unsigned pixel;
                    const bool inside = window_pixel(pt, qt, v, pixel);
#pragma unroll
                    for (int ch = 0; ch < kSliceCh; ch++)
                        planes[ch * kTilePlaneElems + at] = source.elem(pre[u], ch, inside);
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
            if constexpr (Src::kNchw) {
                // rows of each channel plane: consecutive lanes, consecutive columns
                const int nch = min(kSliceCh, d.C - c0);
                for (unsigned i = threadIdx.x; i < nout * nch; i += kTileThreads) {
                    const unsigned ch = i / nout, o = i - ch * nout;
                    const unsigned pl = fast_div(o, m_tw), ql = o - pl * tw;
                    const int p = pt + (int)pl, q = qt + (int)ql;
                    if (p < p_hi && q < d.Q)
                        yn[((size_t)ch * d.P + p) * d.Q + q] = from_float<T>(lout[ch * kTileOutputs + o]);
                }
            } else {
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
}

// grid: 8 * ceil(N / 8) * bands * slices workgroups
template <typename T, class Src>
int launch_nhwc_tile(const typename Src::Params &sp, const float *w, const float *bias,
                     const void *taps, void *y, const ConvDims &d, int flip, hipStream_t st) {
    const size_t lds = nhwc_tile_lds_bytes<T>();
    static const bool once = [&] {
        allow_large_lds(nhwc_tile_fprop_kernel<T, Src>, lds);
        return true;
    }();
    (void)once;
    const int nbands = (d.P + kTileBandRows - 1) / kTileBandRows;
    const int tpi = nbands * ((d.C + kSliceCh - 1) / kSliceCh);
    const long grid = 8L * ((d.N + 7) / 8) * tpi;
    if (grid > 0x7fffffffL) return DWO_ERR_BAD_SHAPE;
    nhwc_tile_fprop_kernel<T, Src><<<dim3((unsigned)grid), dim3(kTileThreads), lds, st>>>(
        sp, w, bias, taps_dhdw(taps), (T *)y, d, nbands, tpi, flip);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

// flip = 1 reverses the weights: with stride 1 that is dgrad (the offsets are odd-symmetric)
template <typename T>
int launch_nhwc_tile_fprop(const void *x, const float *w, const float *bias, const void *taps,
                           void *y, const ConvDims &d, int flip, hipStream_t st) {
    return launch_nhwc_tile<T, SliceSource<T>>({(const T *)x}, w, bias, taps, y, d, flip, st);
}
template <typename T>
int launch_nchw_tile_fprop(const void *x, const float *w, const float *bias, const void *taps,
                           void *y, const ConvDims &d, int flip, hipStream_t st) {
    return launch_nhwc_tile<T, PlaneSource<T>>({(const T *)x}, w, bias, taps, y, d, flip, st);
}

// fprop of the C-channel tensor pw(x): x [N,H,W,CIN], pw_w [C,CIN], pw_b [C] or null
template <typename T, int CIN>
int launch_nhwc_tile_pointwise_fprop(const void *x, const float *pw_w, const float *pw_b,
                                     const float *w, const float *bias, const void *taps, void *y,
                                     const ConvDims &d, hipStream_t st) {
    return launch_nhwc_tile<T, PointwiseSource<T, CIN>>({(const T *)x, pw_w, pw_b}, w, bias, taps, y,
                                                         d, 0, st);
}

}  // namespace dwo

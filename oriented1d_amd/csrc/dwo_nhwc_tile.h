// Tile kernels: fprop, dgrad and wgrad for any plane extent, stride, kernel size and angle, in
// both layouts: the stem convolutions of the ConvNeXt-1D networks (NHWC, 224 -> 112 -> 56,
// stride 2), the stages of inputs other than 224 x 224 (NCHW), and every other shape without
// compile-time planes.  NHWC needs a channel count that is a multiple of 4.  The layouts differ
// only in how a window is loaded (SliceSource, PlaneSource; PointwiseSource applies the stem's
// pointwise projection on the way in) and in how results are stored (tile_flush).
//
// fprop (nhwc_tile_fprop_kernel; with reversed weights also dgrad at stride 1): a workgroup owns
// four consecutive channels of a band of output rows of one image and walks the band in
// sub-tiles.  Per sub-tile it loads the input window, stores it as one plane per channel in LDS in
// the activation's own type (out-of-image positions as zeros), lets sub-group k (128 threads)
// evaluate channel k's taps for the sub-tile's outputs from that plane, and writes the results
// out.  The sub-tile shape is chosen per workgroup from its channels' tap extents: wide row
// strips for near-horizontal taps, tall column strips for near-vertical ones, squares in
// between, so the window read per output stays small for every orientation.  The extents are
// bounded by K / 2 in each direction, whatever the angles.
//
// tile_dgrad_strided_kernel (strides 2 and 4) and tile_wgrad_kernel are described where they
// are defined.
#pragma once

#include <type_traits>

#include "dwo_static.h"

namespace dwo {

constexpr int kTileThreads = 512;                          // four sub-groups of two waves
constexpr int kTileSub = kTileThreads / kSliceCh;          // threads per channel
// LDS elements per channel plane: two workgroups per CU for every element type
template <typename T>
constexpr int tile_plane_elems() {
    return sizeof(T) == 2 ? 7680 : 3584;
}
constexpr int kTileOutputs = 1024;                         // most outputs per sub-tile
constexpr int kTileTapSlots = (DWO_MAX_K + 3) / 4 * 4 + 4;  // tap table: whole groups of four taps
                                                           // plus one group read ahead
constexpr int kTileBandRows = 32;                          // most output rows per workgroup

// planes, fp32 results, per-channel tap table (offset, weight) and tap extents
template <typename T>
constexpr size_t nhwc_tile_lds_bytes() {
    return (size_t)kSliceCh * tile_plane_elems<T>() * sizeof(T) + (size_t)kSliceCh * kTileOutputs * 4 +
           (size_t)kSliceCh * kTileTapSlots * 8 + 64;
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

// PlaneSource: an NCHW tensor; a pixel's payload is one element from each of the workgroup's
// four channel planes (consecutive lanes read consecutive pixels of a row, so every plane's
// loads are contiguous).  Channels beyond C (a last, partial group of four) read as zeros.
// one element from each of four planes: fp32 as they are, 16-bit types packed in pairs
template <typename T>
struct PlanePixels {
    unsigned v[kSliceCh / 2];
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned off, unsigned plane_bytes) {
#pragma unroll
        for (int k = 0; k < kSliceCh / 2; k++) {
            const unsigned lo = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0);
            const unsigned hi = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, off + plane_bytes, 0, 0);
            v[k] = lo | hi << 16;
            off += 2 * plane_bytes;
        }
    }
    __device__ __forceinline__ T elem(int ch) const {
        return __builtin_bit_cast(T, (uint16_t)(v[ch / 2] >> (16 * (ch % 2))));
    }
};
template <>
struct PlanePixels<float> {
    float v[kSliceCh];
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned off, unsigned plane_bytes) {
#pragma unroll
        for (int k = 0; k < kSliceCh; k++)
            v[k] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off + k * plane_bytes, 0, 0));
    }
    __device__ __forceinline__ float elem(int ch) const { return v[ch]; }
};

// PlaneSource: an NCHW tensor; a pixel's payload is one element from each of the workgroup's
// four channel planes (consecutive lanes read consecutive pixels of a row, so every plane's
// loads are contiguous).  Channels beyond C (a last, partial group of four) read as zeros: the
// descriptor ends with the image.
template <typename T>
struct PlaneSource {
    static constexpr bool kNchw = true;
    typedef PlanePixels<T> Payload;
    struct Params {
        const T *x;
    };
    __amdgpu_buffer_rsrc_t img;
    unsigned plane_bytes;
    __device__ __forceinline__ void init(const Params &p, int n, int c0, const ConvDims &d) {
        const T *xn = p.x + ((size_t)n * d.C + c0) * d.H * d.W;
        img = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<T *>(xn), 0, (unsigned)((size_t)(d.C - c0) * d.H * d.W * sizeof(T)), 0x00020000);
        plane_bytes = (unsigned)(d.H * d.W) * (unsigned)sizeof(T);
    }
    __device__ __forceinline__ void load(Payload &v, bool inside, unsigned pixel) const {
        // (an offset that stays beyond the descriptor after the three plane steps)
        v.load(img, inside ? pixel * (unsigned)sizeof(T) : 0x80000000u, plane_bytes);
    }
    __device__ __forceinline__ T elem(const Payload &v, int ch, bool) const { return v.elem(ch); }
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
__device__ __forceinline__ unsigned div_magic(unsigned d) { return 0xffffffffu / d + 1; }

// Results of a th x tw sub-tile at (pt, qt), one fp32 plane of `stride` floats per channel in
// `lout`, to the image at `yn` (rows below p_hi, columns below Q): NCHW as rows of each channel
// plane (consecutive lanes, consecutive columns), NHWC as four-channel pixel slices.
template <typename T, bool NCHW>
__device__ __forceinline__ void tile_flush(const float *lout, int stride, T *yn, unsigned nout,
                                           unsigned tw, unsigned m_tw, int pt, int qt, int p_hi, int P,
                                           int Q, int C, int c0) {
    if constexpr (NCHW) {
        const int nch = min(kSliceCh, C - c0);
        for (int ch = 0; ch < nch; ch++)
            for (unsigned o = threadIdx.x; o < nout; o += kTileThreads) {
                const unsigned pl = fast_div(o, m_tw), ql = o - pl * tw;
                const int p = pt + (int)pl, q = qt + (int)ql;
                if (p < p_hi && q < Q)
                    yn[((size_t)ch * P + p) * Q + q] = from_float<T>(lout[ch * stride + o]);
            }
    } else {
        for (unsigned o = threadIdx.x; o < nout; o += kTileThreads) {
            const unsigned pl = fast_div(o, m_tw), ql = o - pl * tw;
            const int p = pt + (int)pl, q = qt + (int)ql;
            if (p < p_hi && q < Q) {
                Vec4<T> out;
                out.set(lout[o], lout[stride + o], lout[2 * stride + o], lout[3 * stride + o]);
                out.store_cached(yn + ((size_t)p * Q + q) * C);
            }
        }
    }
}

// Largest |dh| and |dw| over the taps of channels c0 .. c0+3 (uniform), from the tap blob's
// per-channel extents.
__device__ __forceinline__ void slice_extent(const int8_t *__restrict__ extent, int c0, int C, int &hh,
                                             int &hw) {
    hh = 0, hw = 0;
#pragma unroll
    for (int ch = 0; ch < kSliceCh; ch++) {
        const int c = min(c0 + ch, C - 1);
        hh = max(hh, (int)extent[2 * c]);
        hw = max(hw, (int)extent[2 * c + 1]);
    }
    hh = __builtin_amdgcn_readfirstlane(hh);
    hw = __builtin_amdgcn_readfirstlane(hw);
}

// Sub-tile shape for a band of RH output rows: th rows x tw columns of outputs with a window
// of ((th-1)*srow + 1 + 2*hh) x ((tw-1)*scol + 1 + 2*hw) inputs.  Cost per output = window
// positions plus a fixed per-sub-tile charge (barriers, pipeline fill), compared as integer
// cross products.  Widths: the full width `wfull` or a power of two from 8 to 128; widths of at
// least 2, also for a one-column plane: the index arithmetic divides by them.
__device__ __forceinline__ void choose_tile(int RH, int wfull, int srow, int scol, int hh, int hw,
                                            int plane_elems, int &th, int &tw) {
    th = 1, tw = min(wfull, 8);
    int best_num = 0x7fffffff / kTileOutputs, best_den = 1;
    for (int a = RH; a >= 1; a = (a + 1) / 2) {
        for (int k = 0; k < 6; k++) {
            const int b = k == 0 ? wfull : (256 >> k);
            if (b > wfull || a * b > kTileOutputs) continue;
            const int ih = (a - 1) * srow + 1 + 2 * hh, iw = ((b - 1) * scol + 1 + 2 * hw) | 1;
            if (ih * iw > plane_elems) continue;
            const int num = ih * iw + 1536, den = a * b;
            if (num * best_den < best_num * den) best_num = num, best_den = den, th = a, tw = b;
        }
        if (a == 1) break;
    }
}

// Rows per band: 32, fewer while the grid would not fill the chip's workgroup slots twice.
inline int tile_band_rows(int N, int rows, int nslices) {
    int band = kTileBandRows;
    while (band > 8 && (long)N * ((rows + band - 1) / band) * nslices < 1024) band /= 2;
    return band;
}

template <typename T, class Src>
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void nhwc_tile_fprop_kernel(
    typename Src::Params sp, const float *__restrict__ wt, const float *__restrict__ bias,
    const int8_t *__restrict__ dhdw, const int8_t *__restrict__ extent, T *__restrict__ y, ConvDims d,
    int nbands, int band_rows, int flip) {
    extern __shared__ float lds_f[];
    T *planes = reinterpret_cast<T *>(lds_f);
    float *lout = reinterpret_cast<float *>(planes + kSliceCh * tile_plane_elems<T>());
    int2 *tapt = reinterpret_cast<int2 *>(lout + kSliceCh * kTileOutputs);  // [ch][K] (offset, weight)

    // Unit (image, band) u runs on XCD u % 8: hardware deals consecutive workgroup ids to the
    // XCDs in turn, so the slices of one band (which share every cache line they touch, NHWC)
    // meet in one L2.
    const int nslices = (d.C + kSliceCh - 1) / kSliceCh;
    const int unit = blockIdx.x % 8 + 8 * (blockIdx.x / 8 / nslices);
    if (unit >= d.N * nbands) return;
    const int slice = blockIdx.x / 8 % nslices;
    const int n = unit / nbands, band = unit - n * nbands;
    const int c0 = slice * kSliceCh;
    const int sub = __builtin_amdgcn_readfirstlane(threadIdx.x / kTileSub);
    const unsigned stid = threadIdx.x % kTileSub;
    const int c = min(c0 + sub, d.C - 1);  // (a partial last group repeats its last channel)
    const int s_ = d.stride, K = d.K;

    // tap extents of the four channels together
    const int8_t *mytaps = dhdw + (size_t)c * K * 2;
    int hh, hw;
    slice_extent(extent, c0, d.C, hh, hw);
    const float bv = bias != nullptr ? bias[c] : 0.f;

    // Window rows/columns step by the stride when no tap of the slice leaves its row/column
    // (0 and 90 degrees): the positions in between are never read.
    const int rstep = hh == 0 ? s_ : 1, cstep = hw == 0 ? s_ : 1;
    const int srow = hh == 0 ? 1 : s_, scol = hw == 0 ? 1 : s_;  // plane rows/columns per output row/column

    // sub-tile shape: th rows x tw columns of outputs; window ih x iw of inputs.  Cost per
    // output = window positions plus a fixed per-sub-tile charge (barriers, pipeline fill).
    // (widths of at least 2, also for a one-column plane: the index arithmetic divides by them)
    const int p_lo = band * band_rows, p_hi = min(d.P, p_lo + band_rows);
    const int RH = p_hi - p_lo;
    const int Qe = max((d.Q + 1) & ~1, 2);  // even widths: a thread evaluates pairs of columns
    int th, tw;
    choose_tile(RH, Qe, srow, scol, hh, hw, tile_plane_elems<T>(), th, tw);
    const int ih = (th - 1) * srow + 1 + 2 * hh;
    const int iw = (tw - 1) * scol + 1 + 2 * hw;
    const int iwp = iw | 1;
    const unsigned m_iw = div_magic(iw), m_tw = div_magic(tw);
    // the channel's taps as (LDS byte offset, weight) pairs, read back as broadcasts; padded with
    // weightless taps to whole groups of four plus the group that is read ahead
    int2 *mytab = tapt + sub * kTileTapSlots;
    const int K4 = (K + 3) & ~3;
    if ((int)stid < K4 + 4) {
        int2 e = make_int2(0, 0);
        if ((int)stid < K)
            // (the steps exceed 1 only where every offset of the slice is 0: no division needed)
            e = make_int2(((int)mytaps[2 * stid] * iwp + (int)mytaps[2 * stid + 1]) *
                              (int)sizeof(T),
                          __float_as_int(wt[(size_t)c * K + (flip ? K - 1 - (int)stid : (int)stid)]));
        mytab[stid] = e;
    }
    const unsigned long long *mytab64 = reinterpret_cast<const unsigned long long *>(mytab);
    const unsigned tw2 = tw >> 1, m_tw2 = div_magic(max(tw2, 2u)), npairs = th * tw2;

    T *yn = Src::kNchw ? y + ((size_t)n * d.C + c0) * d.P * d.Q : y + (size_t)n * d.P * d.Q * d.C + c0;
    const T *plane = planes + sub * tile_plane_elems<T>();
    const unsigned nwin = ih * iw, nout = th * tw;

    // window of sub-tile (pt, qt) -> registers: rows pt*s - hh .., columns qt*s - hw ..
    constexpr int PRE = tile_plane_elems<T>() / kTileThreads;  // pixels per thread, at most
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
                        planes[ch * tile_plane_elems<T>() + at] = source.elem(pre[u], ch, inside);
                }
            }
            __syncthreads();
            // the next window travels while this one is being evaluated
            if (qt + tw < d.Q)
                load_window(pt, qt + tw);
            else if (pt + th < p_hi)
                load_window(pt + th, 0);
            // sub-group: one channel; a thread takes two pairs of neighbouring outputs at a time:
            // each tap's (offset, weight) is fetched once for the four, each pair shares one
            // address, and the next four taps travel while these are used
            auto eval = [&](auto sc) {
                constexpr int SB = decltype(sc)::value * (int)sizeof(T);  // bytes between the pair
                for (unsigned i0 = stid; i0 < npairs; i0 += 2 * kTileSub) {
                    const char *base[2];
                    unsigned at[2];
                    float acc[4] = {bv, bv, bv, bv};
#pragma unroll
                    for (int k = 0; k < 2; k++) {
                        const unsigned i = min(i0 + k * kTileSub, npairs - 1);
                        const unsigned pl = tw2 == 1 ? i : fast_div(i, m_tw2), ql = 2 * (i - pl * tw2);
                        base[k] = reinterpret_cast<const char *>(
                            plane + ((pl * srow + hh) * iwp + ql * decltype(sc)::value + hw));
                        at[k] = pl * tw + ql;
                    }
                    unsigned long long cur[4], nxt[4];
#pragma unroll
                    for (int j = 0; j < 4; j++) cur[j] = mytab64[j];
                    for (int s = 0; s < K4; s += 4) {
#pragma unroll
                        for (int j = 0; j < 4; j++) nxt[j] = mytab64[s + 4 + j];
                        T v[4][4];
#pragma unroll
                        for (int j = 0; j < 4; j++) {
#pragma unroll
                            for (int k = 0; k < 2; k++) {
                                const char *a = base[k] + (int)cur[j];
                                v[j][2 * k] = *reinterpret_cast<const T *>(a);
                                v[j][2 * k + 1] = *reinterpret_cast<const T *>(a + SB);
                            }
                        }
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const float w = __int_as_float((int)(cur[j] >> 32));
#pragma unroll
                            for (int k = 0; k < 4; k++) acc[k] = __builtin_fmaf(to_float(v[j][k]), w, acc[k]);
                        }
#pragma unroll
                        for (int j = 0; j < 4; j++) cur[j] = nxt[j];
                    }
#pragma unroll
                    for (int k = 0; k < 2; k++)
                        if (i0 + k * kTileSub < npairs)
                            *reinterpret_cast<float2 *>(lout + sub * kTileOutputs + at[k]) =
                                make_float2(acc[2 * k], acc[2 * k + 1]);
                }
            };
            if (scol == 1)
                eval(std::integral_constant<int, 1>{});
            else if (scol == 2)
                eval(std::integral_constant<int, 2>{});
            else
                eval(std::integral_constant<int, 4>{});
            __syncthreads();
            tile_flush<T, Src::kNchw>(lout, kTileOutputs, yn, nout, tw, m_tw, pt, qt, p_hi, d.P, d.Q, d.C,
                                      c0);
        }
    }
}

// grid: 8 * ceil(N * bands / 8) * slices workgroups
template <typename T, class Src>
int launch_nhwc_tile(const typename Src::Params &sp, const float *w, const float *bias,
                     const void *taps, void *y, const ConvDims &d, int flip, hipStream_t st) {
    const size_t lds = nhwc_tile_lds_bytes<T>();
    static int cache[kMaxDevices];
    per_device_once(cache, [&] {
        allow_large_lds(nhwc_tile_fprop_kernel<T, Src>, lds);
        return 1;
    });
    if (d.N == 0) return 0;  // set-up only
    const int nslices = (d.C + kSliceCh - 1) / kSliceCh;
    const int band_rows = tile_band_rows(d.N, d.P, nslices);
    const int nbands = (d.P + band_rows - 1) / band_rows;
    const long grid = 8L * (((long)d.N * nbands + 7) / 8) * nslices;
    if (grid > 0x7fffffffL) return DWO_ERR_BAD_SHAPE;
    nhwc_tile_fprop_kernel<T, Src><<<dim3((unsigned)grid), dim3(kTileThreads), lds, st>>>(
        sp, w, bias, taps_dhdw(taps), taps_extent(taps, d.C, d.K), (T *)y, d, nbands, band_rows, flip);
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

// ---------------------------------------------------------------------------------------------
// dgrad with stride 2 or 4 (ops.py:64-88 with the strides of models/convnext.py:141-150).
// dx(h, w) sums w_t * dy((h - dh_t) / s, (w - dw_t) / s) over the taps t whose offsets have h's
// and w's residues modulo s.  The dx pixels of one residue class (a, b) therefore are a
// stride-1 gather over dy with that class's taps at offsets (-floor(dh_t / s), -floor(dw_t / s)),
// and every tap belongs to exactly one class: 1 / s^2 of the multiply-adds of a gather that
// tests all taps at every pixel.  A workgroup owns four channels of a band of dx rows; per
// sub-tile it stages the dy window as one plane per channel in LDS, lets sub-group k evaluate
// channel k class after class (its tap table is sorted by class), places the sums at their dx
// positions in LDS and writes the sub-tile out in raster order.
// LDS elements per channel plane (dy window): two workgroups per CU for every element type
template <typename T>
constexpr int dgrad_plane_elems() {
    return sizeof(T) == 2 ? 4096 : 2048;
}
constexpr int kDgradOutputs = 2048;     // most dx pixels per sub-tile
constexpr int kDgradClasses = 16;       // residue classes at stride 4

template <typename T>
constexpr size_t tile_dgrad_lds_bytes() {
    return (size_t)kSliceCh * dgrad_plane_elems<T>() * sizeof(T) + (size_t)kSliceCh * kDgradOutputs * 4 +
           (size_t)kSliceCh * DWO_MAX_K * 12 + (size_t)kSliceCh * (kDgradClasses + 1) * 4 + 64;
}

template <typename T, class Src>
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void tile_dgrad_strided_kernel(
    typename Src::Params sp, const float *__restrict__ wt, const int8_t *__restrict__ dhdw,
    const int8_t *__restrict__ extent, T *__restrict__ dx, ConvDims d, int nbands, int band_rows) {
    extern __shared__ float lds_f[];
    T *planes = reinterpret_cast<T *>(lds_f);
    float *lout = reinterpret_cast<float *>(planes + kSliceCh * dgrad_plane_elems<T>());
    int2 *tapt = reinterpret_cast<int2 *>(lout + kSliceCh * kDgradOutputs);  // [ch][K], by class
    int *cstart = reinterpret_cast<int *>(tapt + kSliceCh * DWO_MAX_K);     // [ch][classes + 1]
    int *halo = cstart + kSliceCh * (kDgradClasses + 1);                    // [ch][K] taps

    const int nslices = (d.C + kSliceCh - 1) / kSliceCh;
    const int unit = blockIdx.x % 8 + 8 * (blockIdx.x / 8 / nslices);
    if (unit >= d.N * nbands) return;
    const int slice = blockIdx.x / 8 % nslices;
    const int n = unit / nbands, band = unit - n * nbands;
    const int c0 = slice * kSliceCh;
    const int sub = __builtin_amdgcn_readfirstlane(threadIdx.x / kTileSub);
    const unsigned stid = threadIdx.x % kTileSub;
    const int c = min(c0 + sub, d.C - 1);
    const int s_ = d.stride, sh = d.shift, K = d.K, ncls = s_ * s_;

    // the channel's taps into LDS (each is looked at K times below); tap t: residue class and
    // offset in dy
    const int8_t *mytaps = dhdw + (size_t)c * K * 2;
    int *ltap = halo + sub * DWO_MAX_K;
    if ((int)stid < K) ltap[stid] = ((int)mytaps[2 * stid] << 16) | ((int)mytaps[2 * stid + 1] & 0xffff);
    auto tap_class = [&](int t, int &eh, int &ew) {
        const int packed = ltap[t];
        const int dh = packed >> 16, dw = (int)(short)packed;
        eh = -(dh >> sh), ew = -(dw >> sh);  // (arithmetic shifts: floor)
        return (dh & (s_ - 1)) * s_ + (dw & (s_ - 1));
    };
    // extents in dy: the taps are symmetric about the centre, so |floor(-e / s)| = ceil(e / s)
    int hh, hw;
    slice_extent(extent, c0, d.C, hh, hw);
    hh = (hh + s_ - 1) >> sh, hw = (hw + s_ - 1) >> sh;
    __syncthreads();

    // sub-tile: th x tw dx pixels (multiples of the stride), window ih x iw of dy
    const int h_lo = band * band_rows, h_hi = min(d.H, h_lo + band_rows);
    const int RH = (h_hi - h_lo + s_ - 1) & ~(s_ - 1);
    const int We = max((d.W + s_ - 1) & ~(s_ - 1), 2 * s_);
    int th = s_, tw = 8;
    {
        int best_num = 0x7fffffff / kDgradOutputs, best_den = 1;
        for (int a = RH;; a = (((a + 1) / 2) + s_ - 1) & ~(s_ - 1)) {
            for (int k = -1; k < 6; k++) {
                const int b = k < 0 ? We : (256 >> k);  // full width, 256, 128, 64, 32, 16, 8
                if (b > We || a * b > kDgradOutputs) continue;
                const int ih = (a >> sh) + 2 * hh, iw = ((b >> sh) + 2 * hw) | 1;
                if (ih * iw > dgrad_plane_elems<T>()) continue;
                const int num = ih * iw + 1536, den = a * b;
                if (num * best_den < best_num * den) best_num = num, best_den = den, th = a, tw = b;
            }
            if (a <= s_) break;
        }
    }
    const int csh = th >> sh, csw = tw >> sh;  // a class's pixels in the sub-tile
    const int ih = csh + 2 * hh, iw = csw + 2 * hw, iwp = iw | 1;
    const unsigned m_iw = div_magic(iw), m_tw = div_magic(tw), m_csw = div_magic(csw);
    const unsigned nwin = ih * iw, nout = th * tw, csz = csh * csw;

    // the channel's taps sorted by class as (LDS element offset, weight), and the class ranges
    int2 *mytab = tapt + sub * DWO_MAX_K;
    int *mystart = cstart + sub * (kDgradClasses + 1);
    if ((int)stid < K) {
        int eh, ew, fh, fw;
        const int cls = tap_class(stid, eh, ew);
        int rank = 0;
#pragma unroll 8
        for (int t = 0; t < K; t++) {
            const int other = tap_class(t, fh, fw);
            rank += (other < cls || (other == cls && t < (int)stid)) ? 1 : 0;
        }
        mytab[rank] = make_int2(eh * iwp + ew, __float_as_int(wt[(size_t)c * K + stid]));
    }
    if ((int)stid <= ncls) {
        int below = 0, fh, fw;
#pragma unroll 8
        for (int t = 0; t < K; t++) below += tap_class(t, fh, fw) < (int)stid ? 1 : 0;
        mystart[stid] = below;
    }

    T *dxn = Src::kNchw ? dx + ((size_t)n * d.C + c0) * d.H * d.W : dx + (size_t)n * d.H * d.W * d.C + c0;
    const T *plane = planes + sub * dgrad_plane_elems<T>();
    float *myout = lout + sub * kDgradOutputs;

    constexpr int PRE = dgrad_plane_elems<T>() / kTileThreads;
    typename Src::Payload pre[PRE];
    Src source;
    ConvDims ds = d;  // the source tensor is dy: P x Q
    ds.H = d.P, ds.W = d.Q;
    source.init(sp, n, c0, ds);
    auto window_pixel = [&](int ht, int wt_, unsigned v, unsigned &pixel) {
        const unsigned i = fast_div(v, m_iw), j = v - i * iw;
        const unsigned r = (unsigned)((ht >> sh) - hh + (int)i);
        const unsigned q = (unsigned)((wt_ >> sh) - hw + (int)j);
        pixel = r * d.Q + q;
        return v < nwin && r < (unsigned)d.P && q < (unsigned)d.Q;
    };
    auto load_window = [&](int ht, int wt_) {
#pragma unroll
        for (int u = 0; u < PRE; u++) {
            if (u * kTileThreads >= (int)nwin) break;
            unsigned v = u * kTileThreads + threadIdx.x;
            asm volatile("" : "+v"(v));
            unsigned pixel;
            const bool inside = window_pixel(ht, wt_, v, pixel);
            source.load(pre[u], inside, pixel);
        }
    };
    // R pixels of class (a, b) per thread, 128 apart in the class's raster order
    auto eval = [&](auto rc, unsigned e0, int a, int b, int t0, int t1) {
        constexpr int R = decltype(rc)::value;
        const T *base[R];
        float acc[R];
        unsigned at[R];
#pragma unroll
        for (int k = 0; k < R; k++) {
            const unsigned e = min(e0 + k * kTileSub, csz - 1);
            const unsigned i = fast_div(e, m_csw), j = e - i * csw;
            base[k] = plane + ((i + hh) * iwp + j + hw);
            at[k] = ((i << sh) + a) * tw + (j << sh) + b;
            acc[k] = 0.f;
        }
#pragma unroll 4
        for (int t = t0; t < t1; t++) {
            const int2 tp = mytab[t];
            const float w = __int_as_float(tp.y);
#pragma unroll
            for (int k = 0; k < R; k++) acc[k] = __builtin_fmaf(to_float(base[k][tp.x]), w, acc[k]);
        }
#pragma unroll
        for (int k = 0; k < R; k++)
            if (e0 + k * kTileSub < csz) myout[at[k]] = acc[k];
    };

    load_window(h_lo, 0);
    for (int ht = h_lo; ht < h_hi; ht += th) {
        for (int wt_ = 0; wt_ < d.W; wt_ += tw) {
#pragma unroll
            for (int u = 0; u < PRE; u++) {
                if (u * kTileThreads >= (int)nwin) break;
                unsigned v = u * kTileThreads + threadIdx.x;
                asm volatile("" : "+v"(v));
                if (v < nwin) {
                    const unsigned i = fast_div(v, m_iw), j = v - i * iw;
                    const unsigned at = i * iwp + j;
                    unsigned pixel;
                    const bool inside = window_pixel(ht, wt_, v, pixel);
#pragma unroll
                    for (int ch = 0; ch < kSliceCh; ch++)
                        planes[ch * dgrad_plane_elems<T>() + at] = source.elem(pre[u], ch, inside);
                }
            }
            __syncthreads();
            if (wt_ + tw < d.W)
                load_window(ht, wt_ + tw);
            else if (ht + th < h_hi)
                load_window(ht + th, 0);
            for (int cls = 0; cls < ncls; cls++) {
                const int t0 = __builtin_amdgcn_readfirstlane(mystart[cls]);
                const int t1 = __builtin_amdgcn_readfirstlane(mystart[cls + 1]);
                const int a = cls >> sh, b = cls & (s_ - 1);
                if (csz > 2 * kTileSub)
                    for (unsigned e0 = stid; e0 < csz; e0 += 4 * kTileSub)
                        eval(std::integral_constant<int, 4>{}, e0, a, b, t0, t1);
                else if (csz > kTileSub)
                    for (unsigned e0 = stid; e0 < csz; e0 += 2 * kTileSub)
                        eval(std::integral_constant<int, 2>{}, e0, a, b, t0, t1);
                else if (stid < csz)
                    eval(std::integral_constant<int, 1>{}, stid, a, b, t0, t1);
            }
            __syncthreads();
            tile_flush<T, Src::kNchw>(lout, kDgradOutputs, dxn, nout, tw, m_tw, ht, wt_, h_hi, d.H, d.W,
                                      d.C, c0);
        }
    }
}

template <typename T, class Src>
int launch_tile_dgrad_strided_src(const void *dy, const float *w, const void *taps, void *dx,
                                  const ConvDims &d, hipStream_t st) {
    const size_t lds = tile_dgrad_lds_bytes<T>();
    static int cache[kMaxDevices];
    per_device_once(cache, [&] {
        allow_large_lds(tile_dgrad_strided_kernel<T, Src>, lds);
        return 1;
    });
    if (d.N == 0) return 0;  // set-up only
    const int nslices = (d.C + kSliceCh - 1) / kSliceCh;
    const int band_rows = tile_band_rows(d.N, d.H, nslices);
    const int nbands = (d.H + band_rows - 1) / band_rows;
    const long grid = 8L * (((long)d.N * nbands + 7) / 8) * nslices;
    if (grid > 0x7fffffffL) return DWO_ERR_BAD_SHAPE;
    tile_dgrad_strided_kernel<T, Src><<<dim3((unsigned)grid), dim3(kTileThreads), lds, st>>>(
        {(const T *)dy}, w, taps_dhdw(taps), taps_extent(taps, d.C, d.K), (T *)dx, d, nbands, band_rows);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

// dgrad at stride 2 or 4: dy [N,C,P,Q] or [N,P,Q,C] -> dx [N,C,H,W] or [N,H,W,C]
template <typename T>
int launch_tile_dgrad_strided(const void *dy, const float *w, const void *taps, void *dx,
                              const ConvDims &d, bool nchw, hipStream_t st) {
    return nchw ? launch_tile_dgrad_strided_src<T, PlaneSource<T>>(dy, w, taps, dx, d, st)
                : launch_tile_dgrad_strided_src<T, SliceSource<T>>(dy, w, taps, dx, d, st);
}

// ---------------------------------------------------------------------------------------------
// wgrad for any plane extent, stride and kernel size (ops.py:91-118): dw[c, t] = sum over
// images and output positions of dy(p, q) * x(p*s + dh_t, q*s + dw_t), db[c] = sum of dy.
// A workgroup owns four channels and every G-th (image, band) unit.  Per sub-tile it stages the
// x window as planes (as fprop does) and the dy sub-tile as fp32 rows in LDS (zeros beyond the
// image).  In sub-group k (channel k) a thread is (tap, part): it keeps the one running sum of
// its tap over the part's share of the positions, four consecutive positions of a row at a time
// (one 16-byte read of dy, broadcast to the taps, and four window elements).  The parts are
// added at the end and the workgroup writes one partial per (channel, tap); db comes from the
// threads that staged dy.
template <typename T>
constexpr size_t tile_wgrad_lds_bytes() {
    return (size_t)kSliceCh * tile_plane_elems<T>() * sizeof(T) + (size_t)kSliceCh * kTileOutputs * 4 + 64;
}

// Groups of (image, band) units: a multiple of 8 (unit u runs on XCD u % 8), about 8192
// workgroups at most.
inline int tile_wgrad_groups(const ConvDims &d, int *band_rows, int *nbands) {
    const int nslices = (d.C + kSliceCh - 1) / kSliceCh;
    *band_rows = tile_band_rows(d.N, d.P, nslices);
    *nbands = (d.P + *band_rows - 1) / *band_rows;
    const long units = ((long)d.N * *nbands + 7) / 8 * 8;
    const long cap = (8192 / nslices + 7) / 8 * 8;
    return (int)(units < cap ? units : cap);
}

template <typename T, class Src>
__global__ __launch_bounds__(kTileThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void tile_wgrad_kernel(
    typename Src::Params spx, typename Src::Params spy, const int8_t *__restrict__ dhdw,
    const int8_t *__restrict__ extent, float *__restrict__ part, ConvDims d, int nbands, int band_rows,
    int G, int slots_log2) {
    extern __shared__ float lds_f[];
    T *planes = reinterpret_cast<T *>(lds_f);
    float *ldy = reinterpret_cast<float *>(planes + kSliceCh * tile_plane_elems<T>());  // [ch][th * tw]

    const int nslices = (d.C + kSliceCh - 1) / kSliceCh;
    const int g = blockIdx.x % 8 + 8 * (blockIdx.x / 8 / nslices);
    const int slice = blockIdx.x / 8 % nslices;
    const int c0 = slice * kSliceCh;
    const int sub = __builtin_amdgcn_readfirstlane(threadIdx.x / kTileSub);
    const unsigned stid = threadIdx.x % kTileSub;
    const int c = min(c0 + sub, d.C - 1);
    const int s_ = d.stride, K = d.K;
    const int slots = 1 << slots_log2, parts = kTileSub >> slots_log2;
    const int ts = stid & (slots - 1), prt = stid >> slots_log2;

    const int8_t *mytaps = dhdw + (size_t)c * K * 2;
    int hh, hw;
    slice_extent(extent, c0, d.C, hh, hw);
    const int rstep = hh == 0 ? s_ : 1, cstep = hw == 0 ? s_ : 1;
    const int srow = hh == 0 ? 1 : s_, scol = hw == 0 ? 1 : s_;
    // this thread's tap, in plane rows and columns (spare slots repeat tap 0 and are dropped)
    // (the steps exceed 1 only where every offset of the slice is 0: no division needed)
    const int my_dh = ts < K ? (int)mytaps[2 * ts] : 0;
    const int my_dw = ts < K ? (int)mytaps[2 * ts + 1] : 0;

    const T *plane = planes + sub * tile_plane_elems<T>();
    const float *mydy = ldy + sub * kTileOutputs;
    constexpr int PRE = tile_plane_elems<T>() / kTileThreads, PREY = kTileOutputs / kTileThreads;
    typename Src::Payload pre[PRE], prey[PREY];
    Src srcx, srcy;
    ConvDims dyd = d;  // dy as a source tensor: P x Q
    dyd.H = d.P, dyd.W = d.Q;
    float acc = 0.f, dsum[kSliceCh] = {0.f, 0.f, 0.f, 0.f};
    const int Qe = max((d.Q + 3) & ~3, 8);  // sub-tile widths are multiples of 4

    for (int unit = g; unit < d.N * nbands; unit += G) {
        const int n = unit / nbands, band = unit - n * nbands;
        const int p_lo = band * band_rows, p_hi = min(d.P, p_lo + band_rows);
        int th, tw;
        choose_tile(p_hi - p_lo, Qe, srow, scol, hh, hw, tile_plane_elems<T>(), th, tw);
        const int ih = (th - 1) * srow + 1 + 2 * hh;
        const int iw = (tw - 1) * scol + 1 + 2 * hw;
        const int iwp = iw | 1;
        const int tw4 = tw >> 2;
        const unsigned m_iw = div_magic(iw), m_tw = div_magic(tw), m_tw4 = div_magic(tw4);
        const unsigned nwin = ih * iw, nout = th * tw, nquads = th * tw4;
        const T *tapped = plane + (my_dh + hh) * iwp + my_dw + hw;
        srcx.init(spx, n, c0, d);
        srcy.init(spy, n, c0, dyd);

        auto window_pixel = [&](int pt, int qt, unsigned v, unsigned &pixel) {
            const unsigned i = fast_div(v, m_iw), j = v - i * iw;
            const unsigned r = (unsigned)(pt * s_ - hh + (int)i * rstep);
            const unsigned q = (unsigned)(qt * s_ - hw + (int)j * cstep);
            pixel = r * d.W + q;
            return v < nwin && r < (unsigned)d.H && q < (unsigned)d.W;
        };
        auto dy_pixel = [&](int pt, int qt, unsigned o, unsigned &pixel) {
            const unsigned pl = fast_div(o, m_tw), ql = o - pl * tw;
            const unsigned p = pt + pl, q = qt + ql;
            pixel = p * d.Q + q;
            return o < nout && p < (unsigned)p_hi && q < (unsigned)d.Q;
        };
        auto load_tiles = [&](int pt, int qt) {
#pragma unroll
            for (int u = 0; u < PRE; u++) {
                if (u * kTileThreads >= (int)nwin) break;
                unsigned v = u * kTileThreads + threadIdx.x;
                asm volatile("" : "+v"(v));
                unsigned pixel;
                const bool inside = window_pixel(pt, qt, v, pixel);
                srcx.load(pre[u], inside, pixel);
            }
#pragma unroll
            for (int u = 0; u < PREY; u++) {
                if (u * kTileThreads >= (int)nout) break;
                unsigned o = u * kTileThreads + threadIdx.x;
                asm volatile("" : "+v"(o));
                unsigned pixel;
                const bool inside = dy_pixel(pt, qt, o, pixel);
                srcy.load(prey[u], inside, pixel);
            }
        };
        load_tiles(p_lo, 0);
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
                            planes[ch * tile_plane_elems<T>() + at] = srcx.elem(pre[u], ch, inside);
                    }
                }
#pragma unroll
                for (int u = 0; u < PREY; u++) {
                    if (u * kTileThreads >= (int)nout) break;
                    const unsigned o = u * kTileThreads + threadIdx.x;
                    if (o < nout) {
#pragma unroll
                        for (int ch = 0; ch < kSliceCh; ch++) {
                            // (positions outside the image were loaded as zeros)
                            const float v = to_float(srcy.elem(prey[u], ch, true));
                            ldy[ch * kTileOutputs + o] = v;
                            dsum[ch] += v;
                        }
                    }
                }
                __syncthreads();
                if (qt + tw < d.Q)
                    load_tiles(pt, qt + tw);
                else if (pt + th < p_hi)
                    load_tiles(pt + th, 0);
#pragma unroll 2
                for (unsigned qd = prt; qd < nquads; qd += parts) {
                    const unsigned pl = fast_div(qd, m_tw4), qc = qd - pl * tw4;
                    const float4 gy = *reinterpret_cast<const float4 *>(mydy + pl * tw + 4 * qc);
                    const T *a = tapped + pl * srow * iwp + 4 * qc * scol;
                    acc = __builtin_fmaf(gy.x, to_float(a[0]), acc);
                    acc = __builtin_fmaf(gy.y, to_float(a[scol]), acc);
                    acc = __builtin_fmaf(gy.z, to_float(a[2 * scol]), acc);
                    acc = __builtin_fmaf(gy.w, to_float(a[3 * scol]), acc);
                }
                __syncthreads();
            }
        }
    }

    // parts -> one sum per (channel, tap); the dy sums of all threads -> one per channel
    float *red = ldy;                       // [ch][128]
    float *redb = ldy + kTileThreads;       // [wave][ch]
    red[threadIdx.x] = acc;
#pragma unroll
    for (int ch = 0; ch < kSliceCh; ch++) {
        float v = dsum[ch];
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
        if (threadIdx.x % 64 == 0) redb[(threadIdx.x / 64) * kSliceCh + ch] = v;
    }
    __syncthreads();
    if (c0 + sub >= d.C) return;
    const size_t row = (size_t)c * (K + 1);
    if (prt == 0 && ts < K) {
        float total = 0.f;
        for (int j = 0; j < parts; j++) total += red[sub * kTileSub + ts + (j << slots_log2)];
        part[(row + ts) * G + g] = total;
    }
    if (stid == 0) {
        float total = 0.f;
        for (int wv = 0; wv < kTileThreads / 64; wv++) total += redb[wv * kSliceCh + sub];
        part[(row + K) * G + g] = total;
    }
}

// partial sums part[(c * (K + 1) + t) * G + g], t = K for db; returns G through `groups`
template <typename T, class Src>
int launch_tile_wgrad_src(const void *x, const void *dy, const void *taps, float *part, int *groups,
                          const ConvDims &d, hipStream_t st) {
    const size_t lds = tile_wgrad_lds_bytes<T>();
    static int cache[kMaxDevices];
    per_device_once(cache, [&] {
        allow_large_lds(tile_wgrad_kernel<T, Src>, lds);
        return 1;
    });
    if (d.N == 0) return 0;  // set-up only
    int band_rows, nbands;
    const int G = tile_wgrad_groups(d, &band_rows, &nbands);
    *groups = G;
    const int nslices = (d.C + kSliceCh - 1) / kSliceCh;
    int slots_log2 = 0;
    while ((1 << slots_log2) < d.K) slots_log2++;
    tile_wgrad_kernel<T, Src><<<dim3((unsigned)(G * nslices)), dim3(kTileThreads), lds, st>>>(
        {(const T *)x}, {(const T *)dy}, taps_dhdw(taps), taps_extent(taps, d.C, d.K), part, d, nbands,
        band_rows, G, slots_log2);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

template <typename T>
int launch_tile_wgrad(const void *x, const void *dy, const void *taps, float *part, int *groups,
                      const ConvDims &d, bool nchw, hipStream_t st) {
    return nchw ? launch_tile_wgrad_src<T, PlaneSource<T>>(x, dy, taps, part, groups, d, st)
                : launch_tile_wgrad_src<T, SliceSource<T>>(x, dy, taps, part, groups, d, st);
}

}  // namespace dwo

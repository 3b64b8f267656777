// NHWC-native kernels: lane = channel, so all global accesses are coalesced along C and no
// transposed copy of the tensor is ever made.  Every lane keeps the K tap offsets and weights
// of its own channel in registers (adjacent channels usually have different orientations),
// walks a strip of pixels in row-major order and gathers its taps through the vector caches,
// which hold the neighbouring taps of a line between consecutive pixels.
//
// Taps are fetched with raw buffer loads over a descriptor that spans exactly one image: a tap
// above or below the image falls outside the descriptor and the hardware returns zero, so only
// taps that leave the image sideways (and would wrap into the neighbouring row) need masking,
// and only for pixels within K/2 columns of the left or right edge.
//
//   fprop : dst[n,p,q,c] = sum_s src[n, p*str+dh_c(s), q*str+dw_c(s), c] * w[c,s] (+ bias[c])
//   dgrad : (stride 1)   = fprop over dy with every offset negated
//   wgrad : part[c,s,g]  = sum over the pixels of workgroup g of x[..tap..] * dy[n,p,q,c]
#pragma once

#include "dwo_common.h"

namespace dwo {

enum { NHWC_FPROP = 0, NHWC_DGRAD = 1 };

constexpr int kNhwcThreads = 256;  // 4 waves: one 64-channel slab, four pixel strips

// Buffer descriptor over [base, base + bytes): raw (stride 0), 32-bit data format.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t image_rsrc(const void *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}
// One element at byte offset `off` (zero when off is outside the descriptor).
__device__ __forceinline__ float buffer_elem(__amdgpu_buffer_rsrc_t r, unsigned off, float) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
}
__device__ __forceinline__ float buffer_elem(__amdgpu_buffer_rsrc_t r, unsigned off, bf16_t) {
    const unsigned short v = __builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0);
    return __uint_as_float((unsigned)v << 16);
}
__device__ __forceinline__ float buffer_elem(__amdgpu_buffer_rsrc_t r, unsigned off, f16_t) {
    const unsigned short v = __builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0);
    return (float)__builtin_bit_cast(_Float16, v);
}

// Tap loop of one pixel: the K gathers are issued in chunks of eight, chunk k+1 before the
// arithmetic of chunk k, with scheduling fences in between -- eight to sixteen loads in flight
// per wave, and no more live registers than that (left alone, the scheduler either hoists all
// K loads and spills the lane's tap state or serialises load -> wait -> FMA).
// `use(s, value)` consumes tap s.
template <typename T, int K, class Use>
__device__ __forceinline__ void gather_taps(__amdgpu_buffer_rsrc_t img, unsigned centre,
                                            const int (&off)[K], Use use) {
    constexpr int CH = 8, NC = (K + CH - 1) / CH;
    float v[2][CH];
#pragma unroll
    for (int j = 0; j < CH; j++)
        if (j < K) v[0][j] = buffer_elem(img, centre + off[j], T{});
#pragma unroll
    for (int k = 0; k < NC; k++) {
#pragma unroll
        for (int j = 0; j < CH; j++)
            if ((k + 1) * CH + j < K)
                v[(k + 1) & 1][j] = buffer_elem(img, centre + off[(k + 1) * CH + j], T{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < CH; j++)
            if (k * CH + j < K) use(k * CH + j, v[k & 1][j]);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Per-lane tap state of channel c for a source image of width SW (elements of `esize` bytes).
template <int K>
struct LaneTaps {
    int off[K];               // byte offset of tap s from the pixel's own element
    unsigned dwp[(K + 3) / 4];  // column offsets, four signed bytes per register
    __device__ __forceinline__ void load(const int8_t *__restrict__ dhdw, int c, int C, int SW,
                                         int esize, bool negate) {
#pragma unroll
        for (int s = 0; s < (K + 3) / 4; s++) dwp[s] = 0;
#pragma unroll
        for (int s = 0; s < K; s++) {
            int h = dhdw[((size_t)c * K + s) * 2], w = dhdw[((size_t)c * K + s) * 2 + 1];
            if (negate) h = -h, w = -w;
            off[s] = (h * SW + w) * C * esize;
            dwp[s / 4] |= (unsigned)(w & 0xff) << (8 * (s % 4));
        }
    }
    // (the empty asm keeps the unpacked value from being hoisted out of the pixel loop, where
    // all K of them would occupy registers again)
    __device__ __forceinline__ int dw(int s) const {
        unsigned p = dwp[s / 4];
        asm volatile("" : "+v"(p));
        return (int)(signed char)(p >> (8 * (s % 4)));
    }
};

// Uniform walk over destination pixels of an [N, DH, DW] grid in row-major order.
struct PixelWalk {
    int n, a, b;
    __device__ __forceinline__ void start(int idx, int DH, int DW) {
        b = idx % DW;
        const int t = idx / DW;
        a = t % DH;
        n = t / DH;
    }
    __device__ __forceinline__ void next(int DH, int DW) {
        if (++b == DW) {
            b = 0;
            if (++a == DH) a = 0, n++;
        }
    }
};

// fprop (any stride) and stride-1 dgrad.  SH x SW is the source image, DH x DW the destination.
template <typename T, int K, int MODE>
__global__ __launch_bounds__(kNhwcThreads) __attribute__((amdgpu_waves_per_eu(4, 8))) void
nhwc_conv_kernel(const T *__restrict__ src, const float *__restrict__ wt,
                 const float *__restrict__ bias, const int8_t *__restrict__ dhdw,
                 T *__restrict__ dst, ConvDims d, int pix_per_wave) {
    constexpr int PAD = K / 2;
    constexpr int ES = sizeof(T);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int DH = MODE == NHWC_DGRAD ? d.H : d.P, DW = MODE == NHWC_DGRAD ? d.W : d.Q;
    const int SH = MODE == NHWC_DGRAD ? d.P : d.H, SW = MODE == NHWC_DGRAD ? d.Q : d.W;
    const int step = MODE == NHWC_FPROP ? d.stride : 1;
    // Workgroup -> (image, strip group).  Consecutive workgroup ids go to the eight XCDs in turn,
    // each with its own L2; all strips of one image are given to one XCD (image n -> XCD n % 8)
    // and walked in order, so an image is fetched from HBM once, by one L2.
    const int per_image = (DH * DW + 4 * pix_per_wave - 1) / (4 * pix_per_wave);
    const int slabs = (d.C + 63) / 64;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int slab = slot % slabs, strip = (slot / slabs) % per_image;
    const int n_img = (slot / slabs / per_image) * 8 + xcd;
    if (n_img >= d.N) return;
    const int first = n_img * DH * DW;
    const int lo = first + (strip * 4 + wave) * pix_per_wave;
    const int hi = min(lo + pix_per_wave, first + DH * DW);
    if (lo >= hi) return;
    const int c = slab * 64 + lane;
    const bool cok = c < d.C;
    const int cc = cok ? c : d.C - 1;  // idle lanes shadow a real channel and never store

    LaneTaps<K> tp;
    tp.load(dhdw, cc, d.C, SW, ES, MODE == NHWC_DGRAD);
    float w[K];
#pragma unroll
    for (int s = 0; s < K; s++) w[s] = wt[(size_t)cc * K + s];
    const float bv = (MODE == NHWC_FPROP && bias != nullptr) ? bias[cc] : 0.f;
    const unsigned image_bytes = (unsigned)SH * SW * d.C * ES;
    const unsigned lane_off = (unsigned)cc * ES;

    PixelWalk px;
    px.start(lo, DH, DW);
    for (int i = lo; i < hi; i++, px.next(DH, DW)) {
        const int h0 = px.a * step, w0 = px.b * step;  // tap centre in the source image
        const __amdgpu_buffer_rsrc_t img =
            image_rsrc(src + (size_t)px.n * SH * SW * d.C, image_bytes);
        const unsigned centre = (unsigned)((h0 * SW + w0) * d.C) * ES + lane_off;
        float acc = bv;
        if (w0 >= PAD && w0 + PAD < SW) {
            gather_taps<T, K>(img, centre, tp.off,
                              [&](int s, float v) { acc = __builtin_fmaf(v, w[s], acc); });
        } else {
            gather_taps<T, K>(img, centre, tp.off, [&](int s, float v) {
                const float ws = (unsigned)(w0 + tp.dw(s)) < (unsigned)SW ? w[s] : 0.f;
                acc = __builtin_fmaf(v, ws, acc);
            });
        }
        if (cok) (dst + (size_t)i * d.C)[(unsigned)c] = from_float<T>(acc);
    }
}

// wgrad stage 1.  Workgroup (slab, g): 64 channels, pixels [g*4*ppw, (g+1)*4*ppw) of the output
// grid split over its four waves; the four per-lane partial sums meet in LDS and one partial per
// (channel, tap) goes to part[(c*(K+1)+s)*NG + g] (column K: sum of dy, the bias gradient).
template <typename T, int K>
__global__ __launch_bounds__(kNhwcThreads) __attribute__((amdgpu_waves_per_eu(4, 8))) void
nhwc_wgrad_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                  const int8_t *__restrict__ dhdw, float *__restrict__ part, ConvDims d,
                  int pix_per_wave, int NG) {
    constexpr int PAD = K / 2;
    constexpr int ES = sizeof(T);
    __shared__ float red[3][K + 1][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = blockIdx.x * 64 + lane;
    const bool cok = c < d.C;
    const int cc = cok ? c : d.C - 1;
    const int npix = d.N * d.P * d.Q;
    const int lo = min((blockIdx.y * 4 + wave) * pix_per_wave, npix);
    const int hi = min(lo + pix_per_wave, npix);

    LaneTaps<K> tp;
    tp.load(dhdw, cc, d.C, d.W, ES, false);
    float acc[K + 1];
#pragma unroll
    for (int s = 0; s <= K; s++) acc[s] = 0.f;
    const unsigned image_bytes = (unsigned)d.H * d.W * d.C * ES;
    const unsigned lane_off = (unsigned)cc * ES;

    PixelWalk px;
    px.start(lo, d.P, d.Q);
    for (int i = lo; i < hi; i++, px.next(d.P, d.Q)) {
        const int h0 = px.a * d.stride, w0 = px.b * d.stride;
        const __amdgpu_buffer_rsrc_t img =
            image_rsrc(x + (size_t)px.n * d.H * d.W * d.C, image_bytes);
        const unsigned centre = (unsigned)((h0 * d.W + w0) * d.C) * ES + lane_off;
        const float gy = to_float((dy + (size_t)i * d.C)[(unsigned)cc]);
        acc[K] += gy;
        if (w0 >= PAD && w0 + PAD < d.W) {
            gather_taps<T, K>(img, centre, tp.off,
                              [&](int s, float v) { acc[s] = __builtin_fmaf(v, gy, acc[s]); });
        } else {
            gather_taps<T, K>(img, centre, tp.off, [&](int s, float v) {
                const float gs = (unsigned)(w0 + tp.dw(s)) < (unsigned)d.W ? gy : 0.f;
                acc[s] = __builtin_fmaf(v, gs, acc[s]);
            });
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int s = 0; s <= K; s++) red[wave - 1][s][lane] = acc[s];
    }
    __syncthreads();
    if (wave == 0 && cok) {
#pragma unroll
        for (int s = 0; s <= K; s++)
            part[((size_t)c * (K + 1) + s) * NG + blockIdx.y] =
                (acc[s] + red[0][s][lane]) + (red[1][s][lane] + red[2][s][lane]);
    }
}

// Strip length per wave: long enough to amortise loading a lane's K taps and weights, short
// enough to give every CU several workgroups.
inline int nhwc_pix_per_wave(long npix, int slabs) {
    long ppw = npix * slabs / (4L * 256 * 16);
    if (ppw < 16) ppw = 16;
    if (ppw > 256) ppw = 256;
    return (int)ppw;
}
// 1-D grid of nhwc_conv_kernel: (image group of 8, strip group, slab) x 8 XCDs
inline unsigned nhwc_conv_grid(int N, long pix_per_image, int ppw, int slabs) {
    const long per_image = (pix_per_image + 4L * ppw - 1) / (4L * ppw);
    return (unsigned)(((N + 7) / 8) * per_image * slabs * 8);
}
constexpr int kNhwcMaxGroups = 1024;
// wgrad: pixel groups (workgroups along the pixel axis), at most kNhwcMaxGroups partials per tap
inline int nhwc_wgrad_groups(long npix, int slabs, int *ppw_out) {
    long groups = (4L * 256) / slabs;
    if (groups < 1) groups = 1;
    if (groups > kNhwcMaxGroups) groups = kNhwcMaxGroups;
    long ppw = (npix + 4 * groups - 1) / (4 * groups);
    if (ppw < 16) ppw = 16;
    groups = (npix + 4 * ppw - 1) / (4 * ppw);
    *ppw_out = (int)ppw;
    return (int)groups;
}

}  // namespace dwo

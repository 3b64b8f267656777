// Generic (any K, stride, extent, layout, orientation) kernels: one output element per
// thread, taps read from the device table, sources gathered straight from global memory
// through the vector caches.  They are the correctness floor every shape can fall back
// to; the LDS-staged kernels in the sibling headers take over the shapes they cover.
#pragma once

#include "dwo_common.h"

namespace dwo {

template <int LAYOUT>
__device__ __forceinline__ int elem_index(int n, int c, int h, int w, int C, int H, int W) {
    if (LAYOUT == DWO_NCHW) return ((n * C + c) * H + h) * W + w;
    return ((n * H + h) * W + w) * C + c;
}

// fprop (DGRAD=false): dst[N,C,P,Q] gathers src[N,C,H,W] at (p*stride+dh, q*stride+dw).
// dgrad (DGRAD=true) : dst[N,C,H,W] gathers src[N,C,P,Q] at ((h-dh)/stride, (w-dw)/stride)
//                      for taps whose numerators are divisible by the stride.
template <typename T, int LAYOUT, bool DGRAD>
__global__ __launch_bounds__(256) void gather_generic_kernel(
    const T *__restrict__ src, const float *__restrict__ wt, const float *__restrict__ bias,
    const int8_t *__restrict__ dhdw, T *__restrict__ dst, ConvDims d, int total) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int DH = DGRAD ? d.H : d.P, DW = DGRAD ? d.W : d.Q;  // destination extents
    int n, c, a, b;
    if (LAYOUT == DWO_NCHW) {
        b = idx % DW;
        int t = idx / DW;
        a = t % DH;
        t /= DH;
        c = t % d.C;
        n = t / d.C;
    } else {
        c = idx % d.C;
        int t = idx / d.C;
        b = t % DW;
        t /= DW;
        a = t % DH;
        n = t / DH;
    }
    const int8_t *tp = dhdw + (size_t)c * d.K * 2;
    const float *wc = wt + (size_t)c * d.K;
    float acc = 0.f;
    for (int s = 0; s < d.K; s++) {
        const int dh = tp[2 * s], dw = tp[2 * s + 1];
        if (!DGRAD) {
            const int h = a * d.stride + dh, w = b * d.stride + dw;
            if (h >= 0 && h < d.H && w >= 0 && w < d.W)
                acc += to_float(src[elem_index<LAYOUT>(n, c, h, w, d.C, d.H, d.W)]) * wc[s];
        } else {
            const int pp = a - dh, qq = b - dw;
            if (((pp | qq) & (d.stride - 1)) != 0) continue;  // stride is a power of two
            const int p = pp >> d.shift, q = qq >> d.shift;
            if (p >= 0 && p < d.P && q >= 0 && q < d.Q)
                acc += to_float(src[elem_index<LAYOUT>(n, c, p, q, d.C, d.P, d.Q)]) * wc[s];
        }
    }
    if (!DGRAD && bias != nullptr) acc += bias[c];
    dst[idx] = from_float<T>(acc);
}

// wgrad stage 1, generic.  Workgroup (cb, g): channel block cb (CPB channels) and slice g of
// the N*P*Q positions.  NCHW: CPB = 1, 256 threads stride over positions.  NHWC: CPB = 64,
// thread (lane = channel, ty = position phase).  For every tap s (and the pseudo-tap K that
// sums dy alone for the bias gradient) the workgroup writes one partial to
// part[(c*(K+1)+s)*G + g].
template <typename T, int LAYOUT>
__global__ __launch_bounds__(256) void wgrad_generic_kernel(
    const T *__restrict__ dy, const T *__restrict__ x, const int8_t *__restrict__ dhdw,
    float *__restrict__ part, ConvDims d, int G, int per_slice) {
    __shared__ float red[256];
    const int g = blockIdx.y;
    const int npos = d.N * d.P * d.Q;
    const int lo = g * per_slice;
    const int hi = min(lo + per_slice, npos);
    int c, first, step;
    if (LAYOUT == DWO_NCHW) {
        c = blockIdx.x;
        first = lo + threadIdx.x;
        step = 256;
    } else {
        c = blockIdx.x * 64 + (threadIdx.x & 63);
        first = lo + (threadIdx.x >> 6);
        step = 4;
    }
    const bool cok = c < d.C;
    const int8_t *tp = dhdw + (size_t)(cok ? c : 0) * d.K * 2;
    for (int s = 0; s <= d.K; s++) {
        const int dh = s < d.K ? tp[2 * s] : 0, dw = s < d.K ? tp[2 * s + 1] : 0;
        float acc = 0.f;
        if (cok) {
            for (int i = first; i < hi; i += step) {
                const int q = i % d.Q;
                int t = i / d.Q;
                const int p = t % d.P;
                const int n = t / d.P;
                const float gy = to_float(dy[elem_index<LAYOUT>(n, c, p, q, d.C, d.P, d.Q)]);
                if (s == d.K) {
                    acc += gy;
                } else {
                    const int h = p * d.stride + dh, w = q * d.stride + dw;
                    if (h >= 0 && h < d.H && w >= 0 && w < d.W)
                        acc += to_float(x[elem_index<LAYOUT>(n, c, h, w, d.C, d.H, d.W)]) * gy;
                }
            }
        }
        if (LAYOUT == DWO_NCHW) {
            acc = wave_sum(acc);
            __syncthreads();
            if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
            __syncthreads();
            if (threadIdx.x == 0)
                part[((size_t)c * (d.K + 1) + s) * G + g] = (red[0] + red[1]) + (red[2] + red[3]);
        } else {
            __syncthreads();
            red[threadIdx.x] = acc;
            __syncthreads();
            if (threadIdx.x < 64 && cok)
                part[((size_t)c * (d.K + 1) + s) * G + g] =
                    (red[threadIdx.x] + red[threadIdx.x + 64]) +
                    (red[threadIdx.x + 128] + red[threadIdx.x + 192]);
        }
    }
}

// wgrad stage 2: the single cross-workgroup reduction.  One thread per (c, s) adds the G
// partials in index order (deterministic) and writes dw[c,s]; column K goes to db[c].
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float *__restrict__ part,
                                                           float *__restrict__ dw,
                                                           float *__restrict__ db, int C, int K,
                                                           int G) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= C * (K + 1)) return;
    const int c = idx / (K + 1), s = idx % (K + 1);
    if (s == K && db == nullptr) return;
    const float *p = part + (size_t)idx * G;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int g = 0;
    for (; g + 4 <= G; g += 4) {
        a0 += p[g];
        a1 += p[g + 1];
        a2 += p[g + 2];
        a3 += p[g + 3];
    }
    for (; g < G; g++) a0 += p[g];
    const float total = (a0 + a1) + (a2 + a3);
    if (s == K)
        db[c] = total;
    else
        dw[(size_t)c * K + s] = total;
}

}  // namespace dwo

// Layout-changing glue around the operator in a ConvNeXt-1D block, forward only: the passes the
// reference spends in PyTorch between its convolution and its pointwise layers
// (models/convnext.py:306-318: permute + LayerNorm before, layer scale + permute + residual
// after; :176-190 in the stem), each as one pass over HBM.
//
//   nchw_layernorm_nhwc   out[n,h,w,:] = LN_c(x[n,:,h,w]) * gamma + beta         NCHW -> NHWC
//   layernorm_nhwc        out[r,:]     = act(LN_c(x[r,:]) * gamma + beta)        rows of C
//   nhwc_scale_add_nchw   out[n,c,h,w] = res[n,c,h,w] + scale[c] * y[n,h,w,c]    NHWC -> NCHW
//
// LayerNorm is over the channel dimension with the biased variance, statistics in fp32 (mean
// first, then the variance around it).  A wave normalises one pixel at a time; lane l holds
// channels 2l, 2l+1 (+128, +256, ..) so that NHWC accesses are 4- or 8-byte per lane and
// contiguous over the wave.  The transposing kernels go through an LDS tile of P pixels x C
// channels so that both their NCHW and their NHWC side are contiguous.
#pragma once

#include "dwo_static.h"

namespace dwo {

constexpr int kFusedThreads = 256;
constexpr int kFusedMaxC = 2048;          // 16 channel pairs per lane
constexpr int kFusedMaxTileC = 1536;      // transposing LayerNorm: 8 pixels x C floats within 64 KB
constexpr int kFusedChanTile = 64;        // channels per workgroup of the transposing scale-add

// Pixels per LDS tile [C][P + 1] of elements of `esize` bytes: the largest power of two up to 64
// whose tile stays near 26 KB (six workgroups per CU), but not below 32 pixels -- shorter channel
// rows waste most of every 128-byte line on the NCHW side -- while 32 still fit in 56 KB.
inline int fused_tile_pixels(int C, int esize) {
    int p = 64;
    while (p > 8 && (long)C * (p + 1) * esize > 26 * 1024) p >>= 1;
    if (p < 32 && (long)C * 33 * esize <= 40 * 1024) p = 32;
    return p;
}

__device__ __forceinline__ float wave_total(float v) {
    v = wave_sum_dpp(v);  // total in lane 63
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

template <typename T>
__device__ __forceinline__ void store_pair(T *p, float a, float b);
template <>
__device__ __forceinline__ void store_pair<float>(float *p, float a, float b) {
    *reinterpret_cast<float2 *>(p) = make_float2(a, b);
}
template <>
__device__ __forceinline__ void store_pair<bf16_t>(bf16_t *p, float a, float b) {
    *reinterpret_cast<uint32_t *>(p) = pack_bf16(a, b);
}
template <>
__device__ __forceinline__ void store_pair<f16_t>(f16_t *p, float a, float b) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 v;
    v[0] = (_Float16)a, v[1] = (_Float16)b;
    *reinterpret_cast<h2 *>(p) = v;
}
template <typename T>
__device__ __forceinline__ void load_pair(const T *p, float &a, float &b);
template <>
__device__ __forceinline__ void load_pair<float>(const float *p, float &a, float &b) {
    const float2 v = *reinterpret_cast<const float2 *>(p);
    a = v.x, b = v.y;
}
template <>
__device__ __forceinline__ void load_pair<bf16_t>(const bf16_t *p, float &a, float &b) {
    const uint32_t v = *reinterpret_cast<const uint32_t *>(p);
    a = __uint_as_float(v << 16), b = __uint_as_float(v & 0xffff0000u);
}
template <>
__device__ __forceinline__ void load_pair<f16_t>(const f16_t *p, float &a, float &b) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 v = *reinterpret_cast<const h2 *>(p);
    a = (float)v[0], b = (float)v[1];
}

__device__ __forceinline__ float gelu_erf(float v) { return 0.5f * v * (1.f + erff(v * 0.70710678118654752f)); }

// Normalises the values a wave holds for one pixel (v[2k], v[2k+1] = channels 2*lane + 128*k
// and the next one; `live` pairs exist) and writes them as pairs to out_px.  C is even.
template <typename T, int NP>
__device__ __forceinline__ void normalise_and_store(float (&v)[2 * NP], int C, float eps,
                                                    const float *__restrict__ gamma,
                                                    const float *__restrict__ beta, bool gelu,
                                                    T *out_px) {
    const int lane = threadIdx.x & 63;
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NP; k++)
        if (2 * lane + 128 * k < C) s += v[2 * k] + v[2 * k + 1];
    const float mean = wave_total(s) / (float)C;
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < NP; k++)
        if (2 * lane + 128 * k < C) {
            const float a = v[2 * k] - mean, b = v[2 * k + 1] - mean;
            q += a * a + b * b;
        }
    const float rstd = rsqrtf(wave_total(q) / (float)C + eps);
#pragma unroll
    for (int k = 0; k < NP; k++) {
        const int c = 2 * lane + 128 * k;
        if (c < C) {
            float a = (v[2 * k] - mean) * rstd * gamma[c] + beta[c];
            float b = (v[2 * k + 1] - mean) * rstd * gamma[c + 1] + beta[c + 1];
            if (gelu) a = gelu_erf(a), b = gelu_erf(b);
            store_pair<T>(out_px + c, a, b);
        }
    }
}

// Sums over each half of a wave (lanes 0-31 and 32-63): the DPP reduction without its last
// step; every lane gets its half's total.
__device__ __forceinline__ float half_wave_total(float v) {
#define DWO_DPP_ADD(ctrl, row_mask)                                                              \
    v += __builtin_bit_cast(                                                                     \
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, row_mask, 0xf, true))
    DWO_DPP_ADD(0x111, 0xf);  // row_shr:1
    DWO_DPP_ADD(0x112, 0xf);  // row_shr:2
    DWO_DPP_ADD(0x114, 0xf);  // row_shr:4
    DWO_DPP_ADD(0x118, 0xf);  // row_shr:8
    DWO_DPP_ADD(0x142, 0xa);  // row_bcast:15 into rows 1 and 3: lanes 31 and 63 hold the halves
#undef DWO_DPP_ADD
    const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 31));
    const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
    return (threadIdx.x & 32) ? hi : lo;
}

// Rows of at most 64 channels: two rows per wave, one per half, a lane holding one channel pair.
template <typename T>
__global__ __launch_bounds__(kFusedThreads) void layernorm_nhwc_narrow_kernel(
    const T *__restrict__ x, const float *__restrict__ gamma, const float *__restrict__ beta,
    T *__restrict__ out, long rows, int C, float eps, int gelu) {
    const int c = 2 * (threadIdx.x & 31);
    const bool live = c < C;
    float g0 = 0.f, g1 = 0.f, b0 = 0.f, b1 = 0.f;
    if (live) g0 = gamma[c], g1 = gamma[c + 1], b0 = beta[c], b1 = beta[c + 1];
    const long first = ((long)blockIdx.x * (kFusedThreads / 64) + (threadIdx.x >> 6)) * 2 +
                       ((threadIdx.x >> 5) & 1);
    const long step = (long)gridDim.x * (kFusedThreads / 64) * 2;
    const long last = (rows + 1) & ~1L;  // both halves of a wave run the same number of rounds
    for (long r = first; r < last; r += step) {
        float a = 0.f, b = 0.f;
        const bool ok = live && r < rows;
        if (ok) load_pair<T>(x + r * C + c, a, b);
        const float mean = half_wave_total(a + b) / (float)C;
        const float da = ok ? a - mean : 0.f, db = ok ? b - mean : 0.f;
        const float rstd = rsqrtf(half_wave_total(da * da + db * db) / (float)C + eps);
        if (ok) {
            float u = da * rstd * g0 + b0, v = db * rstd * g1 + b1;
            if (gelu) u = gelu_erf(u), v = gelu_erf(v);
            store_pair<T>(out + r * C + c, u, v);
        }
    }
}

// rows of C contiguous channels; one wave per row, grid-stride over rows
template <typename T, int NP>
__global__ __launch_bounds__(kFusedThreads) void layernorm_nhwc_kernel(
    const T *__restrict__ x, const float *__restrict__ gamma, const float *__restrict__ beta,
    T *__restrict__ out, long rows, int C, float eps, int gelu) {
    const int lane = threadIdx.x & 63;
    const long wave = (long)blockIdx.x * (kFusedThreads / 64) + (threadIdx.x >> 6);
    const long nwaves = (long)gridDim.x * (kFusedThreads / 64);
    for (long r = wave; r < rows; r += nwaves) {
        float v[2 * NP];
#pragma unroll
        for (int k = 0; k < NP; k++) {
            const int c = 2 * lane + 128 * k;
            v[2 * k] = v[2 * k + 1] = 0.f;
            if (c < C) load_pair<T>(x + r * C + c, v[2 * k], v[2 * k + 1]);
        }
        normalise_and_store<T, NP>(v, C, eps, gamma, beta, gelu != 0, out + r * C);
    }
}

// NCHW side of the transposing kernels: channel rows of P consecutive pixels <-> the LDS tile
// [C][P + 1].  With HW a multiple of four a lane moves four pixels (one 8- or 16-byte access);
// all of a thread's loads are issued before their results are consumed.
template <typename T, int VEC, class F>
__device__ __forceinline__ void for_each_row_chunk(int C, int P, int np, F &&body) {
    const int per_row = P / VEC;
    const int total = C * per_row;
    for (int i0 = threadIdx.x; i0 < total; i0 += 4 * kFusedThreads) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = i0 + u * kFusedThreads;
            const int c = i / per_row, p = VEC * (i % per_row);  // P is a power of two
            body(u, i < total && p < np, c, p, false);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int i = i0 + u * kFusedThreads;
            const int c = i / per_row, p = VEC * (i % per_row);
            body(u, i < total && p < np, c, p, true);
        }
    }
}

template <typename T, int VEC>
struct PixelVec;
template <typename T>
struct PixelVec<T, 4> : Vec4<T> {
    __device__ __forceinline__ void load(const T *p) { this->load_cached(p); }
    __device__ __forceinline__ void store(T *p) const { this->store_cached(p); }
};
template <typename T>
struct PixelVec<T, 1> {
    T v;
    __device__ __forceinline__ void load(const T *p) { v = *p; }
    __device__ __forceinline__ void store(T *p) const { *p = v; }
    __device__ __forceinline__ float get(int) const { return to_float(v); }
    __device__ __forceinline__ T elem(int) const { return v; }
    __device__ __forceinline__ void set(float a, float, float, float) { v = from_float<T>(a); }
};

// x [N,C,HW] -> out [N,HW,C], normalised over C.  Workgroup = (pixel tile, image).  The
// statistics of a pixel are gathered by kFusedThreads / P threads, each over a stride of the
// channels (mean first, then the variance around it), and combined through LDS; then a wave
// writes one pixel at a time, its lanes holding channel pairs.
template <typename T, int NP, int VEC>
__global__ __launch_bounds__(kFusedThreads) void nchw_layernorm_nhwc_kernel(
    const T *__restrict__ x, const float *__restrict__ gamma, const float *__restrict__ beta,
    T *__restrict__ out, int C, int HW, int P, float eps) {
    // partial sums [G][P], mean [P], rstd [P], then the tile [C][P + 1] in the tensor's type
    extern __shared__ float lds_fused[];
    const int G = kFusedThreads / P;
    float *part = lds_fused;
    float *mean_s = part + G * P, *rstd_s = mean_s + P;
    T *tile = reinterpret_cast<T *>(rstd_s + P);
    const int n = blockIdx.y, p0 = blockIdx.x * P;
    const int np = min(P, HW - p0);
    const T *xn = x + (size_t)n * C * HW + p0;
    PixelVec<T, VEC> in[4];
    for_each_row_chunk<T, VEC>(C, P, np, [&](int u, bool ok, int c, int p, bool second) {
        if (!ok) return;
        if (!second) {
            in[u].load(xn + (size_t)c * HW + p);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; e++) tile[c * (P + 1) + p + e] = in[u].elem(e);
        }
    });
    __syncthreads();
    // statistics: thread (g, p) over channels g, g + G, ..
    const int sp = threadIdx.x % P, sg = threadIdx.x / P;
    float s = 0.f;
    for (int c = sg; c < C; c += G) s += to_float(tile[c * (P + 1) + sp]);
    part[sg * P + sp] = s;
    __syncthreads();
    float mean = 0.f;
    for (int g = 0; g < G; g++) mean += part[g * P + sp];
    mean /= (float)C;
    float q = 0.f;
    for (int c = sg; c < C; c += G) {
        const float dlt = to_float(tile[c * (P + 1) + sp]) - mean;
        q += dlt * dlt;
    }
    __syncthreads();  // every thread has read the partial sums
    part[sg * P + sp] = q;
    __syncthreads();
    if (sg == 0) {
        float var = 0.f;
        for (int g = 0; g < G; g++) var += part[g * P + sp];
        mean_s[sp] = mean;
        rstd_s[sp] = rsqrtf(var / (float)C + eps);
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    float gm[2 * NP], bt[2 * NP];
#pragma unroll
    for (int k = 0; k < NP; k++) {
        const int c = 2 * lane + 128 * k;
        gm[2 * k] = gm[2 * k + 1] = bt[2 * k] = bt[2 * k + 1] = 0.f;
        if (c < C) gm[2 * k] = gamma[c], gm[2 * k + 1] = gamma[c + 1], bt[2 * k] = beta[c], bt[2 * k + 1] = beta[c + 1];
    }
    T *on = out + ((size_t)n * HW + p0) * C;
    for (int p = threadIdx.x >> 6; p < np; p += kFusedThreads / 64) {
        const float m = mean_s[p], r = rstd_s[p];
#pragma unroll
        for (int k = 0; k < NP; k++) {
            const int c = 2 * lane + 128 * k;
            if (c < C)
                store_pair<T>(on + (size_t)p * C + c,
                              (to_float(tile[c * (P + 1) + p]) - m) * r * gm[2 * k] + bt[2 * k],
                              (to_float(tile[(c + 1) * (P + 1) + p]) - m) * r * gm[2 * k + 1] +
                                  bt[2 * k + 1]);
        }
    }
}

// y [N,HW,C] -> out [N,C,HW] = res + scale[c] * y (res and scale optional).  Workgroup =
// (pixel tile, channel tile, image): up to kFusedChanTile channels x P pixels.
template <typename T, int VEC>
__global__ __launch_bounds__(kFusedThreads) void nhwc_scale_add_nchw_kernel(
    const T *__restrict__ y, const float *__restrict__ scale, const T *__restrict__ res,
    T *__restrict__ out, int C, int HW, int P, int ptiles) {
    extern __shared__ float tile[];  // [CT][P + 1]
    const int n = blockIdx.y, p0 = (blockIdx.x % ptiles) * P, c0 = (blockIdx.x / ptiles) * kFusedChanTile;
    const int np = min(P, HW - p0), CT = min(kFusedChanTile, C - c0);
    const T *yn = y + ((size_t)n * HW + p0) * C + c0;
    const size_t base = ((size_t)n * C + c0) * HW + p0;
    // the residual rows do not depend on the tile: their loads go out first
    PixelVec<T, VEC> rs[4];
    const bool one_round = CT * (P / VEC) <= 4 * kFusedThreads;
    if (res != nullptr && one_round)
        for_each_row_chunk<T, VEC>(CT, P, np, [&](int u, bool ok, int c, int p, bool second) {
            if (ok && !second) rs[u].load(res + base + (size_t)c * HW + p);
        });
    // pixels of CT contiguous channels, read as pairs
    const int half = CT / 2;
    for (int i = threadIdx.x; i < half * np; i += kFusedThreads) {
        const int p = i / half, c = 2 * (i % half);
        float a, b;
        load_pair<T>(yn + (size_t)p * C + c, a, b);
        tile[c * (P + 1) + p] = a;
        tile[(c + 1) * (P + 1) + p] = b;
    }
    __syncthreads();
    for_each_row_chunk<T, VEC>(CT, P, np, [&](int u, bool ok, int c, int p, bool second) {
        if (!ok) return;
        if (!second) {
            if (res != nullptr && !one_round) rs[u].load(res + base + (size_t)c * HW + p);
        } else {
            float v[4] = {0.f, 0.f, 0.f, 0.f};
            const float sc = scale != nullptr ? scale[c0 + c] : 1.f;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                v[e] = tile[c * (P + 1) + p + e] * sc;
                if (res != nullptr) v[e] += rs[u].get(e);
            }
            PixelVec<T, VEC> o;
            o.set(v[0], v[1], v[2], v[3]);
            o.store(out + base + (size_t)c * HW + p);
        }
    });
}

// pairs per lane needed for C channels: 1, 2, 4, 8 or 16
#define DWO_FUSED_NP_DISPATCH(C, CALL) \
    do {                               \
        if ((C) <= 128) {              \
            CALL(1);                   \
        } else if ((C) <= 256) {       \
            CALL(2);                   \
        } else if ((C) <= 512) {       \
            CALL(4);                   \
        } else if ((C) <= 1024) {      \
            CALL(8);                   \
        } else {                       \
            CALL(16);                  \
        }                              \
    } while (0)

template <typename T>
int launch_layernorm_nhwc(const void *x, const float *gamma, const float *beta, void *out, long rows,
                          int C, float eps, int gelu, hipStream_t st) {
    long blocks = (rows + kFusedThreads / 64 - 1) / (kFusedThreads / 64);
    if (blocks > 65536) blocks = 65536;
    if (C <= 64) {
        layernorm_nhwc_narrow_kernel<T><<<dim3((unsigned)((blocks + 1) / 2)), dim3(kFusedThreads), 0,
                                          st>>>((const T *)x, gamma, beta, (T *)out, rows, C, eps,
                                                gelu);
        const hipError_t e = hipGetLastError();
        return e == hipSuccess ? 0 : (int)e;
    }
#define DWO_CALL(NP_)                                                                        \
    layernorm_nhwc_kernel<T, NP_><<<dim3((unsigned)blocks), dim3(kFusedThreads), 0, st>>>(   \
        (const T *)x, gamma, beta, (T *)out, rows, C, eps, gelu)
    DWO_FUSED_NP_DISPATCH(C, DWO_CALL);
#undef DWO_CALL
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

template <typename T>
int launch_nchw_layernorm_nhwc(const void *x, const float *gamma, const float *beta, void *out,
                               int N, int C, int HW, float eps, hipStream_t st) {
    const int P = fused_tile_pixels(C, (int)sizeof(T));
    const size_t lds = ((size_t)kFusedThreads + 2 * P) * sizeof(float) + (size_t)C * (P + 1) * sizeof(T);
    const dim3 grid((HW + P - 1) / P, N), block(kFusedThreads);
#define DWO_CALL(NP_)                                                              \
    do {                                                                           \
        if (HW % 4 == 0)                                                           \
            nchw_layernorm_nhwc_kernel<T, NP_, 4><<<grid, block, lds, st>>>(       \
                (const T *)x, gamma, beta, (T *)out, C, HW, P, eps);               \
        else                                                                       \
            nchw_layernorm_nhwc_kernel<T, NP_, 1><<<grid, block, lds, st>>>(       \
                (const T *)x, gamma, beta, (T *)out, C, HW, P, eps);               \
    } while (0)
    DWO_FUSED_NP_DISPATCH(C, DWO_CALL);
#undef DWO_CALL
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

template <typename T>
int launch_nhwc_scale_add_nchw(const void *y, const float *scale, const void *res, void *out, int N,
                               int C, int HW, hipStream_t st) {
    constexpr int P = 64;
    const size_t lds = (size_t)kFusedChanTile * (P + 1) * sizeof(float);
    const int ptiles = (HW + P - 1) / P, ctiles = (C + kFusedChanTile - 1) / kFusedChanTile;
    const dim3 grid(ptiles * ctiles, N), block(kFusedThreads);
    if (HW % 4 == 0)
        nhwc_scale_add_nchw_kernel<T, 4><<<grid, block, lds, st>>>(
            (const T *)y, scale, (const T *)res, (T *)out, C, HW, P, ptiles);
    else
        nhwc_scale_add_nchw_kernel<T, 1><<<grid, block, lds, st>>>(
            (const T *)y, scale, (const T *)res, (T *)out, C, HW, P, ptiles);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

}  // namespace dwo

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
constexpr int kFusedMaxTileC = 1536;      // transposing kernels: 8 pixels x C floats within 64 KB
constexpr int kFusedTileFloats = 12288;   // LDS tile of the transposing kernels (48 KB)

// pixels per tile for C channels: a power of two between 8 and 64 that fits the LDS tile
inline int fused_tile_pixels(int C) {
    int p = 64;
    while (p > 8 && (long)C * (p + 1) > kFusedTileFloats) p >>= 1;
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
    *reinterpret_cast<uint32_t *>(p) =
        (uint32_t)from_float<bf16_t>(a).bits | ((uint32_t)from_float<bf16_t>(b).bits << 16);
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

// x [N,C,HW] -> out [N,HW,C], normalised over C.  Workgroup = (pixel tile, image).
template <typename T, int NP>
__global__ __launch_bounds__(kFusedThreads) void nchw_layernorm_nhwc_kernel(
    const T *__restrict__ x, const float *__restrict__ gamma, const float *__restrict__ beta,
    T *__restrict__ out, int C, int HW, int P, float eps) {
    extern __shared__ float tile[];  // [C][P + 1]
    const int n = blockIdx.y, p0 = blockIdx.x * P;
    const int np = min(P, HW - p0);
    const T *xn = x + (size_t)n * C * HW + p0;
    // channel rows of P consecutive pixels: consecutive lanes read consecutive pixels
    if (HW % 2 == 0) {  // (p0 and P are even: pairs of pixels stay aligned and inside the plane)
        const int hp = P / 2;
        for (int i = threadIdx.x; i < C * hp; i += kFusedThreads) {
            const int c = i / hp, p = 2 * (i % hp);  // P is a power of two
            if (p < np) {
                float a, b;
                load_pair<T>(xn + (size_t)c * HW + p, a, b);
                tile[c * (P + 1) + p] = a;
                tile[c * (P + 1) + p + 1] = b;
            }
        }
    } else {
        for (int i = threadIdx.x; i < C * P; i += kFusedThreads) {
            const int c = i / P, p = i % P;
            if (p < np) tile[c * (P + 1) + p] = to_float(xn[(size_t)c * HW + p]);
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    T *on = out + ((size_t)n * HW + p0) * C;
    for (int p = threadIdx.x >> 6; p < np; p += kFusedThreads / 64) {
        float v[2 * NP];
#pragma unroll
        for (int k = 0; k < NP; k++) {
            const int c = 2 * lane + 128 * k;
            v[2 * k] = v[2 * k + 1] = 0.f;
            if (c < C) v[2 * k] = tile[c * (P + 1) + p], v[2 * k + 1] = tile[(c + 1) * (P + 1) + p];
        }
        normalise_and_store<T, NP>(v, C, eps, gamma, beta, false, on + (size_t)p * C);
    }
}

// y [N,HW,C] -> out [N,C,HW] = res + scale[c] * y (res and scale optional)
template <typename T>
__global__ __launch_bounds__(kFusedThreads) void nhwc_scale_add_nchw_kernel(
    const T *__restrict__ y, const float *__restrict__ scale, const T *__restrict__ res,
    T *__restrict__ out, int C, int HW, int P) {
    extern __shared__ float tile[];  // [C][P + 1]
    const int n = blockIdx.y, p0 = blockIdx.x * P;
    const int np = min(P, HW - p0);
    const T *yn = y + ((size_t)n * HW + p0) * C;
    // pixels of C contiguous channels, read as pairs
    const int half = C / 2;
    for (int i = threadIdx.x; i < half * np; i += kFusedThreads) {
        const int p = i / half, c = 2 * (i % half);
        float a, b;
        load_pair<T>(yn + (size_t)p * C + c, a, b);
        tile[c * (P + 1) + p] = a;
        tile[(c + 1) * (P + 1) + p] = b;
    }
    __syncthreads();
    const size_t base = (size_t)n * C * HW + p0;
    if (HW % 2 == 0) {  // two pixels per lane: 4-byte (8-byte fp32) accesses on the NCHW side
        const int hp = P / 2;
        for (int i = threadIdx.x; i < C * hp; i += kFusedThreads) {
            const int c = i / hp, p = 2 * (i % hp);
            if (p < np) {
                float a = tile[c * (P + 1) + p], b = tile[c * (P + 1) + p + 1];
                if (scale != nullptr) a *= scale[c], b *= scale[c];
                if (res != nullptr) {
                    float ra, rb;
                    load_pair<T>(res + base + (size_t)c * HW + p, ra, rb);
                    a += ra, b += rb;
                }
                store_pair<T>(out + base + (size_t)c * HW + p, a, b);
            }
        }
    } else {
        for (int i = threadIdx.x; i < C * P; i += kFusedThreads) {
            const int c = i / P, p = i % P;
            if (p < np) {
                float v = tile[c * (P + 1) + p];
                if (scale != nullptr) v *= scale[c];
                if (res != nullptr) v += to_float(res[base + (size_t)c * HW + p]);
                out[base + (size_t)c * HW + p] = from_float<T>(v);
            }
        }
    }
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
    const int P = fused_tile_pixels(C);
    const size_t lds = (size_t)C * (P + 1) * sizeof(float);
    const dim3 grid((HW + P - 1) / P, N), block(kFusedThreads);
#define DWO_CALL(NP_)                                                    \
    nchw_layernorm_nhwc_kernel<T, NP_><<<grid, block, lds, st>>>(        \
        (const T *)x, gamma, beta, (T *)out, C, HW, P, eps)
    DWO_FUSED_NP_DISPATCH(C, DWO_CALL);
#undef DWO_CALL
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

template <typename T>
int launch_nhwc_scale_add_nchw(const void *y, const float *scale, const void *res, void *out, int N,
                               int C, int HW, hipStream_t st) {
    const int P = fused_tile_pixels(C);
    const size_t lds = (size_t)C * (P + 1) * sizeof(float);
    const dim3 grid((HW + P - 1) / P, N), block(kFusedThreads);
    nhwc_scale_add_nchw_kernel<T><<<grid, block, lds, st>>>((const T *)y, scale, (const T *)res,
                                                           (T *)out, C, HW, P);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

}  // namespace dwo

// Shared device/host helpers for the gfx950 depthwise oriented 1D convolution kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "dwoconv1d_hip.h"

namespace dwo {

// One 16-byte (8-byte) LDS read of four (two) adjacent words; p must be aligned to the access.
// A float4 / float2 dereference is taken apart into 4-byte reads by the passes this library
// is built with; at a lane stride of four words those hit every bank eight times.
typedef float lds_f4 __attribute__((ext_vector_type(4)));
typedef float lds_f2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ lds_f4 lds_read4(const float *p) {
    return *reinterpret_cast<const lds_f4 *>(__builtin_assume_aligned(p, 16));
}
__device__ __forceinline__ lds_f2 lds_read2(const float *p) {
    return *reinterpret_cast<const lds_f2 *>(__builtin_assume_aligned(p, 8));
}


// ---------------------------------------------------------------------------------------------
// Tap blob (private layout).  Built on the host by dwo_build_taps, copied verbatim to the device.
//   int32 header[8] : magic, version, C, K, off_dhdw, off_class, off_order, off_extent
//   int8  dhdw[C][K][2]        (dh, dw) of every tap, padded to 16 bytes
//   int32 cls[C]               canonical orientation id 0..7 of the channel's tap pattern
//                              (k * 22.5 degrees), or -1 when the pattern is not canonical;
//                              padded to 16 bytes
//   int32 order[C]             the channels in an order that cycles through the orientation
//                              classes (class 0, 1, .., 7, other, 0, 1, ..): the per-channel
//                              workgroups of fprop and dgrad take their channel from it, so that
//                              whatever way the angles are laid out over the channels,
//                              neighbouring workgroup ids (hence every XCD and CU) get a mix of
//                              orientations
//   int8  extent[C][2]         (max |dh|, max |dw|) over the channel's taps, padded to 16 bytes
//   int32 sorted[C]            the channels sorted by what their orientation class costs in the
//                              plane kernels, dearest first (non-canonical, 22.5 and 157.5
//                              degrees, 67.5 and 112.5, 0, 90, 45 and 135): wgrad deals this
//                              list to the CUs so that their loads come out even; padded to 16
//                              bytes
// ---------------------------------------------------------------------------------------------
constexpr int32_t kTapsMagic = 0x44574f31;  // "DWO1"
constexpr int32_t kTapsVersion = 6;
constexpr int kTapsHeaderInts = 8;
constexpr int kTapsHeaderBytes = kTapsHeaderInts * 4;

__host__ __device__ inline size_t taps_dhdw_bytes(int C, int K) {
    return (((size_t)C * K * 2) + 15) & ~(size_t)15;
}
__host__ __device__ inline const int8_t *taps_dhdw(const void *blob) {
    return reinterpret_cast<const int8_t *>(blob) + kTapsHeaderBytes;
}
__host__ __device__ inline size_t taps_class_bytes(int C) {
    return ((size_t)C * 4 + 15) & ~(size_t)15;
}
__host__ __device__ inline const int32_t *taps_class(const void *blob, int C, int K) {
    return reinterpret_cast<const int32_t *>(reinterpret_cast<const int8_t *>(blob) +
                                             kTapsHeaderBytes + taps_dhdw_bytes(C, K));
}
__host__ __device__ inline size_t taps_extent_bytes(int C) {
    return ((size_t)C * 2 + 15) & ~(size_t)15;
}
__host__ __device__ inline const int8_t *taps_extent(const void *blob, int C, int K) {
    return reinterpret_cast<const int8_t *>(blob) + kTapsHeaderBytes + taps_dhdw_bytes(C, K) +
           2 * taps_class_bytes(C);
}
__host__ __device__ inline const int32_t *taps_sorted(const void *blob, int C, int K) {
    return reinterpret_cast<const int32_t *>(reinterpret_cast<const int8_t *>(blob) +
                                             kTapsHeaderBytes + taps_dhdw_bytes(C, K) +
                                             2 * taps_class_bytes(C) + taps_extent_bytes(C));
}
__host__ __device__ inline const int32_t *taps_order(const void *blob, int C, int K) {
    return reinterpret_cast<const int32_t *>(reinterpret_cast<const int8_t *>(blob) +
                                             kTapsHeaderBytes + taps_dhdw_bytes(C, K) +
                                             taps_class_bytes(C));
}

// ---------------------------------------------------------------------------------------------
// Element types.  Activations are fp32, bf16 (raw uint16 bits) or fp16; arithmetic is fp32.
// ---------------------------------------------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};
typedef _Float16 f16_t;

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) {
    return __uint_as_float(static_cast<uint32_t>(v.bits) << 16);
}
__device__ __forceinline__ float to_float(f16_t v) { return static_cast<float>(v); }

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) {
    return v;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
    // round to nearest even in hardware (v_cvt_pk_bf16_f32)
    bf16_t r;
    r.bits = __builtin_bit_cast(uint16_t, (__bf16)v);
    return r;
}
// two values at once: (lo, hi) as one 32-bit word
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    bf2 v;
    v[0] = (__bf16)lo, v[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
}
template <>
__device__ __forceinline__ f16_t from_float<f16_t>(float v) {
    return static_cast<f16_t>(v);
}

// Wave64 sum via cross-lane shuffles; every lane ends with the total of lanes >= itself folded
// down, lane 0 holds the wave total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

// Dynamic LDS beyond 64 KB has to be allowed per kernel before the first launch.
template <class Kern>
void allow_large_lds(Kern kern, size_t lds) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
}

// One-time set-up of a kernel on a device (dynamic-LDS attribute, occupancy query): `make()` runs
// once per device with that device current and its non-zero result is kept in cache[device].
// Launchers called with an empty batch (N = 0) stop right after it, which is how dwo_init
// prepares every kernel ahead of a stream capture.
constexpr int kMaxDevices = 64;
template <class F>
inline int per_device_once(int *cache, F make) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return make();
    int v = __atomic_load_n(&cache[dev], __ATOMIC_ACQUIRE);
    if (v == 0) {
        v = make();  // idempotent: two threads racing here compute the same value
        __atomic_store_n(&cache[dev], v, __ATOMIC_RELEASE);
    }
    return v;
}

struct ConvDims {
    int N, C, H, W, P, Q, K, stride, shift;  // shift = log2(stride)
};

}  // namespace dwo

// Declarations of the per-(element type, plane extent) launchers defined in dwo_inst.hip, and the
// list of plane extents that have LDS-staged kernels.  Each (type, extent) pair is compiled as
// its own translation unit so the build can run them in parallel.
#pragma once

#include <hip/hip_runtime.h>

#include "dwo_common.h"
#include "dwo_plan.h"

// X(K, H, W): kernel size and plane extents with compile-time kernels (stride 1): the ConvNeXt
// stage extents at 224 x 224 input for K = 31 (1D blocks, second conv of 1D++ blocks) and K = 15
// (first conv of 1D++ blocks), and K = 7 at the three extents of the reference's own
// micro-benchmark (analysis/benchmark.py:84-104); and the stage extents of a 512 x 512 input
// that fit a workgroup's LDS (64, 32, 16 squared; NCHW only, see nhwc_plane_shape)
#ifndef DWO_PLANE_SHAPES
#define DWO_PLANE_SHAPES(X)                                   \
    X(31, 56, 56) X(31, 28, 28) X(31, 14, 14) X(31, 7, 7)     \
    X(15, 56, 56) X(15, 28, 28) X(15, 14, 14) X(15, 7, 7)     \
    X(7, 56, 56) X(7, 28, 28) X(7, 14, 14)                    \
    X(31, 64, 64) X(31, 32, 32) X(31, 16, 16)
#endif

namespace dwo {

enum { OP_FPROP = 0, OP_DGRAD = 1 };

// Image groups per channel: as many workgroups as can be resident at once (no second round),
// at most kMaxPlaneGroups and at most one staged batch per group.
constexpr int kMaxPlaneGroups = 32;
inline int plane_groups(int N, int C, int PB, int slots) {
    int g = slots / C;
    const int nbatch = (N + PB - 1) / PB;
    if (g > nbatch) g = nbatch;
    if (g > kMaxPlaneGroups) g = kMaxPlaneGroups;
    if (g < 1) g = 1;
    // A single round that would leave more than a quarter of the slots idle (512 channels on
    // 768 slots): two full rounds of smaller workgroups instead, when C divides two rounds'
    // worth of slots to within 5 %.
    if ((long)C * g * 4 < (long)slots * 3) {
        const int g2 = 2 * slots / C;
        if (g2 > g && g2 <= nbatch && g2 <= kMaxPlaneGroups && (long)C * g2 * 20 >= (long)slots * 38)
            return g2;
    }
    // prefer an even split of the batches (every workgroup the same number of images) when one
    // exists within 3/4 of the resident-slot count: the kernel ends with its slowest workgroup
    for (int d = g; d * 4 >= g * 3 && d >= 1; d--)
        if (nbatch % d == 0) return d;
    return g;
}

template <typename T, int K, int H, int W>
int launch_plane_conv(int op, const void *src, const float *w, const float *bias, const void *taps,
                      void *dst, int N, int C, hipStream_t st);
template <typename T, int K, int H, int W>
int launch_plane_wgrad(const void *x, const void *dy, const void *taps, float *part, float *dw,
                       float *db, unsigned *tickets, int N, int C, int *groups_out, hipStream_t st);

// NHWC, C a multiple of 4: channel-slice workgroups over the same LDS planes
template <typename T, int K, int H, int W>
int launch_nhwc_plane_conv(int op, const void *src, const float *w, const float *bias,
                           const void *taps, void *dst, int N, int C, hipStream_t st);

template <typename T, int K, int H, int W>
int launch_nhwc_plane_wgrad(const void *x, const void *dy, const void *taps, float *part, float *dw,
                            float *db, unsigned *tickets, int N, int C, int *groups_out,
                            hipStream_t st);

#define DWO_DECLARE(T, K, H, W)                                                                   \
    extern template int launch_plane_conv<T, K, H, W>(int, const void *, const float *,           \
                                                      const float *, const void *, void *, int,   \
                                                      int, hipStream_t);                          \
    extern template int launch_plane_wgrad<T, K, H, W>(const void *, const void *, const void *,  \
                                                       float *, float *, float *, unsigned *,     \
                                                       int, int, int *, hipStream_t);             \
    extern template int launch_nhwc_plane_conv<T, K, H, W>(int, const void *, const float *,      \
                                                           const float *, const void *, void *,   \
                                                           int, int, hipStream_t);        \
    extern template int launch_nhwc_plane_wgrad<T, K, H, W>(const void *, const void *,           \
                                                            const void *, float *, float *,       \
                                                            float *, unsigned *, int, int, int *, \
                                                            hipStream_t);
#define DWO_DECLARE_ALL(K, H, W) \
    DWO_DECLARE(float, K, H, W) DWO_DECLARE(bf16_t, K, H, W) DWO_DECLARE(f16_t, K, H, W)
DWO_PLANE_SHAPES(DWO_DECLARE_ALL)
#undef DWO_DECLARE_ALL
#undef DWO_DECLARE

}  // namespace dwo

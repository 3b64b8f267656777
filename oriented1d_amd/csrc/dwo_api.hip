// C ABI of libdwoconv1d_hip.so: argument validation, host-side tap table, kernel selection
// and launch.  No device allocation and no retained caller pointers; the only state is what
// dwo_init caches per device (occupancy figures, kernel attributes, the address of the static
// wgrad scratch).
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "dwo_common.h"
#include "dwo_generic.h"
#include "dwo_nhwc.h"
#include "dwo_dispatch.h"
#include "dwo_nhwc_tile.h"
#include "dwo_fused.h"

using namespace dwo;

namespace {

int log2_stride(int stride) { return stride == 1 ? 0 : (stride == 2 ? 1 : (stride == 4 ? 2 : -1)); }

int check_common(int N, int C, int H, int W, int K, int stride, int dtype, int layout) {
    if (N < 1 || C < 1 || H < 1 || W < 1) return DWO_ERR_BAD_SHAPE;
    if ((double)N * C * H * W >= 2147483648.0) return DWO_ERR_BAD_SHAPE;
    if (K < 1 || K > DWO_MAX_K || (K & 1) == 0) return DWO_ERR_BAD_KERNEL;
    if (log2_stride(stride) < 0) return DWO_ERR_BAD_STRIDE;
    if (dtype != DWO_F32 && dtype != DWO_BF16 && dtype != DWO_F16) return DWO_ERR_BAD_DTYPE;
    if (layout != DWO_NCHW && layout != DWO_NHWC) return DWO_ERR_BAD_LAYOUT;
    return DWO_OK;
}

ConvDims make_dims(int N, int C, int H, int W, int K, int stride) {
    ConvDims d;
    d.N = N, d.C = C, d.H = H, d.W = W, d.K = K, d.stride = stride;
    d.shift = log2_stride(stride);
    d.P = (H + stride - 1) / stride;
    d.Q = (W + stride - 1) / stride;
    return d;
}

int launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? DWO_OK : (int)e;
}

// The launchers report hipGetLastError() after their launch; an error left behind on this
// thread by unrelated earlier work must not be returned as this call's status, so every
// launching entry point starts by clearing it.
void begin_call() { (void)hipGetLastError(); }

struct WgradSplit {
    int blocks_x, G, per_slice;
};

// Slices of the N*P*Q positions per channel block for the generic wgrad: enough workgroups
// to fill 256 CUs several times over, at least 1024 positions per slice.
WgradSplit wgrad_generic_split(const ConvDims &d, int layout) {
    WgradSplit s;
    s.blocks_x = layout == DWO_NCHW ? d.C : (d.C + 63) / 64;
    const long npos = (long)d.N * d.P * d.Q;
    long G = 4096 / s.blocks_x;
    const long cap = (npos + 1023) / 1024;
    if (G > cap) G = cap;
    if (G < 1) G = 1;
    s.per_slice = (int)((npos + G - 1) / G);
    s.G = (int)((npos + s.per_slice - 1) / s.per_slice);
    return s;
}

// Plane extents with LDS-staged kernels (NCHW, stride 1).  PB = planes staged per batch.
int plane_batch(const ConvDims &d, int layout) {
    if (layout != DWO_NCHW || d.stride != 1) return 0;
#define DWO_MATCH(K_, H_, W_) \
    if (d.K == K_ && d.H == H_ && d.W == W_) return Tile<H_, W_>::PB;
    DWO_PLANE_SHAPES(DWO_MATCH)
#undef DWO_MATCH
    return 0;
}

// returns -100 when no LDS-staged kernel covers the shape
template <typename T>
int try_plane_conv(int op, const void *src, const float *w, const float *bias, const void *taps,
                   void *dst, const ConvDims &d, int layout, hipStream_t st) {
    if (plane_batch(d, layout) == 0) return -100;
#define DWO_MATCH(K_, H_, W_)                                                               \
    if (d.K == K_ && d.H == H_ && d.W == W_)                                                \
        return launch_plane_conv<T, K_, H_, W_>(op, src, w, bias, taps, dst, d.N, d.C, st);
    DWO_PLANE_SHAPES(DWO_MATCH)
#undef DWO_MATCH
    return -100;
}

template <typename T>
int try_plane_wgrad(const void *x, const void *dy, const void *taps, float *part, float *dw,
                    float *db, unsigned *tickets, int *groups, const ConvDims &d, hipStream_t st) {
#define DWO_MATCH(K_, H_, W_)                                                               \
    if (d.K == K_ && d.H == H_ && d.W == W_)                                                \
        return launch_plane_wgrad<T, K_, H_, W_>(x, dy, taps, part, dw, db, tickets, d.N, d.C, \
                                                 groups, st);
    DWO_PLANE_SHAPES(DWO_MATCH)
#undef DWO_MATCH
    return -100;
}

int nhwc_plane_batch(const ConvDims &d, int layout);

// NHWC with the channel count a multiple of 4, stride 1, at the same extents: the slice kernels
template <typename T>
int try_nhwc_plane_conv(int op, const void *src, const float *w, const float *bias,
                        const void *taps, void *dst, const ConvDims &d, int layout, hipStream_t st) {
    if (nhwc_plane_batch(d, layout) == 0) return -100;
#define DWO_MATCH(K_, H_, W_)                                                                    \
    if (d.K == K_ && d.H == H_ && d.W == W_)                                                     \
        return launch_nhwc_plane_conv<T, K_, H_, W_>(op, src, w, bias, taps, dst, d.N, d.C, st);
    DWO_PLANE_SHAPES(DWO_MATCH)
#undef DWO_MATCH
    return -100;
}

// NHWC with a kernel size that has lane-resident tap kernels; -100 otherwise
#define DWO_NHWC_KS(X) X(7) X(13) X(15) X(27) X(31)
bool nhwc_has_k(int K) {
#define DWO_MATCH(K_) if (K == K_) return true;
    DWO_NHWC_KS(DWO_MATCH)
#undef DWO_MATCH
    return false;
}

// wgrad partial-sum count per (channel, tap): an upper bound that sizes the scratch buffer
// (the staged path picks its group count from the device's occupancy at launch, never more
// than kMaxPlaneGroups nor than the number of staged batches).
// images per staged batch of the NHWC slice kernels, 0 when they do not cover the shape
int nhwc_plane_batch(const ConvDims &d, int layout) {
    if (layout != DWO_NHWC || d.stride != 1 || d.C % kSliceCh != 0) return 0;
#define DWO_MATCH(K_, H_, W_) \
    if (d.K == K_ && d.H == H_ && d.W == W_) return nhwc_plane_shape_rt(H_, W_) ? NhwcTile<H_, W_>::PBI : 0;
    DWO_PLANE_SHAPES(DWO_MATCH)
#undef DWO_MATCH
    return 0;
}

template <typename T>
int try_nhwc_plane_wgrad(const void *x, const void *dy, const void *taps, float *part, float *dw,
                         float *db, unsigned *tickets, int *groups, const ConvDims &d,
                         hipStream_t st) {
#define DWO_MATCH(K_, H_, W_)                                                                    \
    if (d.K == K_ && d.H == H_ && d.W == W_)                                                     \
        return launch_nhwc_plane_wgrad<T, K_, H_, W_>(x, dy, taps, part, dw, db, tickets, d.N, d.C, \
                                                      groups, st);
    DWO_PLANE_SHAPES(DWO_MATCH)
#undef DWO_MATCH
    return -100;
}

// shapes the tile kernels take: NCHW always, NHWC with the channel count a multiple of 4; images
// below 2 GB (32-bit offsets inside one)
bool tile_covers(const ConvDims &d, int layout, size_t esize) {
    if ((size_t)d.H * d.W * d.C * esize >= 0x80000000ull) return false;
    // the smallest sub-tile (1 x 8 outputs) of the widest possible taps must fit a channel plane
    const int plane = esize == 2 ? tile_plane_elems<bf16_t>() : tile_plane_elems<float>();
    if (d.K * ((7 * d.stride + d.K) | 1) > plane) return false;
    return layout == DWO_NCHW || d.C % kSliceCh == 0;
}

int wgrad_max_partials(const ConvDims &d, int layout, size_t esize) {
    const int PBI = nhwc_plane_batch(d, layout);
    if (PBI != 0) {
        const int nbatch = (d.N + PBI - 1) / PBI;
        return nbatch < kMaxPlaneGroups ? nbatch : kMaxPlaneGroups;
    }
    const int PB = plane_batch(d, layout);
    if (PB == 0 && tile_covers(d, layout, esize)) {
        int band_rows, nbands;
        return tile_wgrad_groups(d, &band_rows, &nbands);
    }
    if (PB == 0 && layout == DWO_NHWC && nhwc_has_k(d.K)) {
        int ppw = 0;
        return nhwc_wgrad_groups((long)d.N * d.P * d.Q, (d.C + 63) / 64, &ppw);
    }
    if (PB == 0) return wgrad_generic_split(d, layout).G;
    const int nbatch = (d.N + PB - 1) / PB;
    return nbatch < kMaxPlaneGroups ? nbatch : kMaxPlaneGroups;
}

// fprop (flip = 0) or dgrad (flip = 1) at any extent by the tile kernels: NCHW always, NHWC with
// the channel count a multiple of 4; images below 2 GB (32-bit offsets inside one)
template <typename T>
int try_tile_conv(const void *x, const float *w, const float *bias, const void *taps, void *y,
                  const ConvDims &d, int layout, int flip, hipStream_t st) {
    if (!tile_covers(d, layout, sizeof(T))) return -100;
    if (flip && d.stride != 1)
        return launch_tile_dgrad_strided<T>(x, w, taps, y, d, layout == DWO_NCHW, st);
    if (layout == DWO_NCHW) return launch_nchw_tile_fprop<T>(x, w, bias, taps, y, d, flip, st);
    return launch_nhwc_tile_fprop<T>(x, w, bias, taps, y, d, flip, st);
}

template <typename T, int MODE>
int try_nhwc_conv(const void *src, const float *w, const float *bias, const void *taps, void *dst,
                  const ConvDims &d, int layout, hipStream_t st) {
    if (layout != DWO_NHWC || !nhwc_has_k(d.K)) return -100;
    if (MODE == NHWC_DGRAD && d.stride != 1) return -100;  // strided dgrad: generic kernel
    const int slabs = (d.C + 63) / 64;
    const long per_image = MODE == NHWC_DGRAD ? (long)d.H * d.W : (long)d.P * d.Q;
    const int ppw = nhwc_pix_per_wave(d.N * per_image, slabs);
    const dim3 grid(nhwc_conv_grid(d.N, per_image, ppw, slabs)), block(kNhwcThreads);
#define DWO_MATCH(K_)                                                                         \
    if (d.K == K_)                                                                            \
        nhwc_conv_kernel<T, K_, MODE><<<grid, block, 0, st>>>((const T *)src, w, bias,        \
                                                              taps_dhdw(taps), (T *)dst, d, ppw);
    DWO_NHWC_KS(DWO_MATCH)
#undef DWO_MATCH
    return launch_status();
}

template <typename T>
int try_nhwc_wgrad(const void *dy, const void *x, const void *taps, float *part, int *groups,
                   const ConvDims &d, hipStream_t st) {
    const int slabs = (d.C + 63) / 64;
    int ppw = 0;
    const int NG = nhwc_wgrad_groups((long)d.N * d.P * d.Q, slabs, &ppw);
    *groups = NG;
    const dim3 grid(slabs, NG), block(kNhwcThreads);
#define DWO_MATCH(K_)                                                                          \
    if (d.K == K_)                                                                             \
        nhwc_wgrad_kernel<T, K_><<<grid, block, 0, st>>>((const T *)dy, (const T *)x,          \
                                                         taps_dhdw(taps), part, d, ppw, NG);
    DWO_NHWC_KS(DWO_MATCH)
#undef DWO_MATCH
    return launch_status();
}

template <typename T>
int fprop_t(const void *x, const float *w, const float *bias, const void *taps, void *y,
            const ConvDims &d, int layout, hipStream_t st) {
    const int fast = try_plane_conv<T>(OP_FPROP, x, w, bias, taps, y, d, layout, st);
    if (fast != -100) return fast;
    const int sliced = try_nhwc_plane_conv<T>(OP_FPROP, x, w, bias, taps, y, d, layout, st);
    if (sliced != -100) return sliced;
    const int tiled = try_tile_conv<T>(x, w, bias, taps, y, d, layout, 0, st);
    if (tiled != -100) return tiled;
    const int nhwc = try_nhwc_conv<T, NHWC_FPROP>(x, w, bias, taps, y, d, layout, st);
    if (nhwc != -100) return nhwc;
    const int total = d.N * d.C * d.P * d.Q;
    const dim3 grid((total + 255) / 256), block(256);
    const int8_t *tp = taps_dhdw(taps);
    if (layout == DWO_NCHW)
        gather_generic_kernel<T, DWO_NCHW, false><<<grid, block, 0, st>>>(
            (const T *)x, w, bias, tp, (T *)y, d, total);
    else
        gather_generic_kernel<T, DWO_NHWC, false><<<grid, block, 0, st>>>(
            (const T *)x, w, bias, tp, (T *)y, d, total);
    return launch_status();
}

template <typename T>
int dgrad_t(const void *dy, const float *w, const void *taps, void *dx, const ConvDims &d,
            int layout, hipStream_t st) {
    const int fast = try_plane_conv<T>(OP_DGRAD, dy, w, nullptr, taps, dx, d, layout, st);
    if (fast != -100) return fast;
    const int sliced = try_nhwc_plane_conv<T>(OP_DGRAD, dy, w, nullptr, taps, dx, d, layout, st);
    if (sliced != -100) return sliced;
    const int tiled = try_tile_conv<T>(dy, w, nullptr, taps, dx, d, layout, 1, st);
    if (tiled != -100) return tiled;
    const int nhwc = try_nhwc_conv<T, NHWC_DGRAD>(dy, w, nullptr, taps, dx, d, layout, st);
    if (nhwc != -100) return nhwc;
    const int total = d.N * d.C * d.H * d.W;
    const dim3 grid((total + 255) / 256), block(256);
    const int8_t *tp = taps_dhdw(taps);
    if (layout == DWO_NCHW)
        gather_generic_kernel<T, DWO_NCHW, true><<<grid, block, 0, st>>>(
            (const T *)dy, w, nullptr, tp, (T *)dx, d, total);
    else
        gather_generic_kernel<T, DWO_NHWC, true><<<grid, block, 0, st>>>(
            (const T *)dy, w, nullptr, tp, (T *)dx, d, total);
    return launch_status();
}

// Ticket counters of the plane wgrad kernels (wgrad_finish): one counter per channel block.  They
// live in the library's device image, zero when the library is loaded (dwo_init clears them
// again), and every launch leaves its counters at zero.  Launches that may run at the same time
// must not share counters, so a row of counters belongs to one stream: launches on a stream run
// one after the other, and the first kTicketSlots streams that call wgrad on a device each own a
// row for good.  Everything else takes the separate reduction kernel (bit-identical results):
// calls under stream capture (a graph would keep its row while eager calls go on using it, and
// two replays of one graph may overlap), the per-thread default stream (one handle, many
// streams), further streams once the rows are taken, shapes with more channel blocks than a row
// holds, and devices where the symbol cannot be resolved.
constexpr int kTicketSlots = 64, kTicketRow = 4096;
static __device__ unsigned g_tickets[kTicketSlots * kTicketRow];
struct TicketRows {
    std::mutex mu;
    unsigned *base = nullptr;
    int used = 0;
    hipStream_t owner[kTicketSlots];
};
TicketRows g_ticket_rows[kMaxDevices];
std::atomic<int> g_tickets_enabled{1};  // dwo_set_wgrad_reduction

// the device's counter array (resolved once per device), or null
unsigned *ticket_base(TicketRows &rows) {
    if (rows.base == nullptr) {
        void *sym = nullptr;
        if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_tickets)) != hipSuccess || sym == nullptr) {
            (void)hipGetLastError();
            return nullptr;
        }
        rows.base = (unsigned *)sym;
    }
    return rows.base;
}

unsigned *ticket_row(int blocks, hipStream_t st) {
    if (blocks > kTicketRow || !g_tickets_enabled.load(std::memory_order_relaxed)) return nullptr;
    if (st == hipStreamPerThread) return nullptr;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    if (cap != hipStreamCaptureStatusNone) return nullptr;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    TicketRows &rows = g_ticket_rows[dev];
    std::lock_guard<std::mutex> lock(rows.mu);
    unsigned *base = ticket_base(rows);
    if (base == nullptr) return nullptr;
    int r = 0;
    while (r < rows.used && rows.owner[r] != st) r++;
    if (r == rows.used) {
        if (rows.used == kTicketSlots) return nullptr;
        rows.owner[rows.used++] = st;
    }
    return base + (size_t)r * kTicketRow;
}

// dwo_init: the counters back to zero (they already are unless a launch was torn down half way)
int reset_tickets() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return DWO_OK;
    TicketRows &rows = g_ticket_rows[dev];
    std::lock_guard<std::mutex> lock(rows.mu);
    unsigned *base = ticket_base(rows);
    if (base == nullptr) return DWO_OK;
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipMemset(base, 0, sizeof(unsigned) * kTicketSlots * kTicketRow);
    return e == hipSuccess ? DWO_OK : (int)e;
}

template <typename T>
int wgrad_t(const void *dy, const void *x, const void *taps, float *dw, float *db, void *scratch,
            const ConvDims &d, int layout, hipStream_t st) {
    float *part = (float *)scratch;
    int rc, NG = 0;
    bool direct = false;  // stage 1 wrote dw / db itself (one group per channel, or tickets)
    if (plane_batch(d, layout) != 0) {
        unsigned *tickets = ticket_row(d.C, st);
        rc = try_plane_wgrad<T>(x, dy, taps, part, dw, db, tickets, &NG, d, st);
        direct = NG == 1 || tickets != nullptr;
    } else if (nhwc_plane_batch(d, layout) != 0) {
        unsigned *tickets = ticket_row(d.C / kSliceCh, st);
        rc = try_nhwc_plane_wgrad<T>(x, dy, taps, part, dw, db, tickets, &NG, d, st);
        direct = NG == 1 || tickets != nullptr;
    } else if (tile_covers(d, layout, sizeof(T))) {
        rc = launch_tile_wgrad<T>(x, dy, taps, part, &NG, d, layout == DWO_NCHW, st);
    } else if (layout == DWO_NHWC && nhwc_has_k(d.K)) {
        rc = try_nhwc_wgrad<T>(dy, x, taps, part, &NG, d, st);
    } else {
        const WgradSplit s = wgrad_generic_split(d, layout);
        NG = s.G;
        const dim3 grid(s.blocks_x, s.G), block(256);
        const int8_t *tp = taps_dhdw(taps);
        if (layout == DWO_NCHW)
            wgrad_generic_kernel<T, DWO_NCHW><<<grid, block, 0, st>>>(
                (const T *)dy, (const T *)x, tp, part, d, s.G, s.per_slice);
        else
            wgrad_generic_kernel<T, DWO_NHWC><<<grid, block, 0, st>>>(
                (const T *)dy, (const T *)x, tp, part, d, s.G, s.per_slice);
        rc = launch_status();
    }
    if (rc != DWO_OK || direct) return rc;
    const int cells = d.C * (d.K + 1);
    wgrad_reduce_kernel<<<dim3((cells + 255) / 256), dim3(256), 0, st>>>(part, dw, db, d.C, d.K,
                                                                        NG);
    return launch_status();
}

template <typename T>
int pointwise_fprop_t(const void *x, const float *pw_w, const float *pw_b, const float *w,
                      const float *bias, const void *taps, void *y, int Cin, const ConvDims &d,
                      hipStream_t st) {
    switch (Cin) {
        case 1: return launch_nhwc_tile_pointwise_fprop<T, 1>(x, pw_w, pw_b, w, bias, taps, y, d, st);
        case 2: return launch_nhwc_tile_pointwise_fprop<T, 2>(x, pw_w, pw_b, w, bias, taps, y, d, st);
        case 3: return launch_nhwc_tile_pointwise_fprop<T, 3>(x, pw_w, pw_b, w, bias, taps, y, d, st);
        default: return launch_nhwc_tile_pointwise_fprop<T, 4>(x, pw_w, pw_b, w, bias, taps, y, d, st);
    }
}

int wgrad_dispatch(const void *dy, const void *x, const void *taps, float *dw, float *db,
                   void *scratch, int N, int C, int H, int W, int K, int stride, int dtype,
                   int layout, hipStream_t st) {
    const ConvDims d = make_dims(N, C, H, W, K, stride);
    begin_call();
    switch (dtype) {
        case DWO_F32: return wgrad_t<float>(dy, x, taps, dw, db, scratch, d, layout, st);
        case DWO_BF16: return wgrad_t<bf16_t>(dy, x, taps, dw, db, scratch, d, layout, st);
        default: return wgrad_t<f16_t>(dy, x, taps, dw, db, scratch, d, layout, st);
    }
}

// Partial sums of dwo_wgrad_static.  One copy per GPU, held until the process ends.  The name
// is only a host-side handle: the memory's address on the current device comes from
// hipGetSymbolAddress (static_scratch below) and that pointer is what the kernels are given.
static __device__ __align__(256) unsigned char g_wgrad_scratch[DWO_STATIC_SCRATCH_BYTES];
void *g_wgrad_scratch_ptr[kMaxDevices];

int static_scratch(void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return DWO_ERR_BAD_SHAPE;
    void *p = __atomic_load_n(&g_wgrad_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (p == nullptr) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_wgrad_scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return (int)hipErrorInvalidSymbol;
        __atomic_store_n(&g_wgrad_scratch_ptr[dev], p, __ATOMIC_RELEASE);
    }
    *out = p;
    return DWO_OK;
}

// One-time set-up of every kernel on the current device (see per_device_once): the launchers
// are called with an empty batch, which stops them after their set-up.
template <typename T>
int init_type() {
    int rc = 0, ng = 0;
#define DWO_PREP(K_, H_, W_)                                                                      \
    rc |= launch_plane_conv<T, K_, H_, W_>(OP_FPROP, nullptr, nullptr, nullptr, nullptr, nullptr, \
                                           0, 1, nullptr);                                        \
    rc |= launch_plane_wgrad<T, K_, H_, W_>(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, \
                                            nullptr, 0, 1, &ng, nullptr);                         \
    rc |= launch_nhwc_plane_conv<T, K_, H_, W_>(OP_FPROP, nullptr, nullptr, nullptr, nullptr,     \
                                                nullptr, 0, kSliceCh, nullptr);                   \
    rc |= launch_nhwc_plane_wgrad<T, K_, H_, W_>(nullptr, nullptr, nullptr, nullptr, nullptr,     \
                                                 nullptr, nullptr, 0, kSliceCh, &ng, nullptr);
    DWO_PLANE_SHAPES(DWO_PREP)
#undef DWO_PREP
    ConvDims d = make_dims(1, kSliceCh, 8, 8, 7, 2);
    d.N = 0;
    rc |= launch_nchw_tile_fprop<T>(nullptr, nullptr, nullptr, nullptr, nullptr, d, 0, nullptr);
    rc |= launch_nhwc_tile_fprop<T>(nullptr, nullptr, nullptr, nullptr, nullptr, d, 0, nullptr);
    rc |= launch_tile_dgrad_strided<T>(nullptr, nullptr, nullptr, nullptr, d, true, nullptr);
    rc |= launch_tile_dgrad_strided<T>(nullptr, nullptr, nullptr, nullptr, d, false, nullptr);
    rc |= launch_tile_wgrad<T>(nullptr, nullptr, nullptr, nullptr, &ng, d, true, nullptr);
    rc |= launch_tile_wgrad<T>(nullptr, nullptr, nullptr, nullptr, &ng, d, false, nullptr);
    for (int cin = 1; cin <= 4; cin++)
        rc |= pointwise_fprop_t<T>(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                                   cin, d, nullptr);
    return rc;
}

}  // namespace

extern "C" {

int dwo_init(void) {
    begin_call();
    void *scratch = nullptr;  // the static wgrad scratch's address on this device
    const int rc = static_scratch(&scratch);
    if (rc != DWO_OK) return rc;
    const int trc = reset_tickets();  // and the ticket counters', all zero from here on
    if (trc != DWO_OK) return trc;
    // (the set-up calls leave their own failures in the runtime's last-error slot)
    (void)init_type<float>();
    (void)init_type<bf16_t>();
    (void)init_type<f16_t>();
    return launch_status();
}

int dwo_version(void) { return 300; }

int dwo_set_wgrad_reduction(int in_kernel) {
    return g_tickets_enabled.exchange(in_kernel ? 1 : 0, std::memory_order_relaxed);
}

const char *dwo_status_string(int status) {
    switch (status) {
        case DWO_OK: return "ok";
        case DWO_ERR_NULL_POINTER: return "null pointer argument";
        case DWO_ERR_BAD_SHAPE: return "invalid tensor extents (must be >= 1 and index in int32)";
        case DWO_ERR_BAD_KERNEL: return "kernel size must be odd and in [1, 63]";
        case DWO_ERR_BAD_STRIDE: return "stride must be 1, 2 or 4";
        case DWO_ERR_BAD_DTYPE: return "unsupported element type";
        case DWO_ERR_BAD_LAYOUT: return "unsupported layout";
        case DWO_ERR_SCRATCH_TOO_SMALL: return "wgrad scratch buffer too small";
        case DWO_ERR_BAD_TAPS: return "tap table does not match C and K";
        case DWO_ERR_STATIC_SCRATCH_LIMIT:
            return "wgrad partial sums exceed the static scratch (DWO_STATIC_SCRATCH_BYTES)";
        default: break;
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown status";
}

size_t dwo_taps_bytes(int C, int K) {
    if (C < 1 || K < 1 || K > DWO_MAX_K || (K & 1) == 0) return 0;
    return kTapsHeaderBytes + taps_dhdw_bytes(C, K) + 3 * taps_class_bytes(C) + taps_extent_bytes(C);
}

int dwo_build_taps(const float *theta_host, int C, int K, void *taps_host) {
    if (theta_host == nullptr || taps_host == nullptr) return DWO_ERR_NULL_POINTER;
    if (C < 1) return DWO_ERR_BAD_SHAPE;
    if (K < 1 || K > DWO_MAX_K || (K & 1) == 0) return DWO_ERR_BAD_KERNEL;
    memset(taps_host, 0, dwo_taps_bytes(C, K));
    int32_t *hdr = (int32_t *)taps_host;
    hdr[0] = kTapsMagic, hdr[1] = kTapsVersion, hdr[2] = C, hdr[3] = K;
    hdr[4] = kTapsHeaderBytes;
    hdr[5] = kTapsHeaderBytes + (int32_t)taps_dhdw_bytes(C, K);
    int8_t *dhdw = (int8_t *)taps_host + kTapsHeaderBytes;
    int32_t *cls = (int32_t *)((int8_t *)taps_host + hdr[5]);
    const int pad = K / 2;
    for (int c = 0; c < C; c++) {
        // models/dwoconv1d_reference/kernels/kernels.cpp:37,43-44: fp32 sine and cosine, a
        // float product, and a C cast to int (truncation toward zero).
        const float sin_ = sinf(theta_host[c]), cos_ = cosf(theta_host[c]);
        for (int s = 0; s < K; s++) {
            volatile float fh = -sin_ * (float)(s - pad);
            volatile float fw = cos_ * (float)(s - pad);
            dhdw[((size_t)c * K + s) * 2 + 0] = (int8_t)(int)fh;
            dhdw[((size_t)c * K + s) * 2 + 1] = (int8_t)(int)fw;
        }
        // canonical orientation: all K taps equal one of the eight compile-time patterns
        cls[c] = -1;
        for (int o = 0; o < 8 && cls[c] < 0; o++) {
            bool same = true;
            for (int s = 0; s < K && same; s++)
                same = dhdw[((size_t)c * K + s) * 2] == canon_dh(o, K, s) &&
                       dhdw[((size_t)c * K + s) * 2 + 1] == canon_dw(o, K, s);
            if (same) cls[c] = o;
        }
    }
    // channel order that cycles through the classes: 0, 1, .., 7, non-canonical, 0, 1, ..
    hdr[6] = hdr[5] + (int32_t)taps_class_bytes(C);
    int32_t *order = (int32_t *)((int8_t *)taps_host + hdr[6]);
    int next[9];  // per class: next channel of that class not yet placed
    for (int k = 0; k < 9; k++) next[k] = 0;
    for (int placed = 0; placed < C;) {
        for (int k = 0; k < 9 && placed < C; k++) {
            const int want = k < 8 ? k : -1;
            int c = next[k];
            while (c < C && cls[c] != want) c++;
            next[k] = c + 1;
            if (c < C) order[placed++] = c;
        }
    }
    // and the channels sorted by the cost of their class in the plane kernels, dearest first:
    // non-canonical (table-driven body), 22.5 and 157.5 degrees, 67.5 and 112.5, 0, 90, 45 and 135
    // (stable within a class)
    int32_t *sorted = const_cast<int32_t *>(taps_sorted(taps_host, C, K));
    static const int by_cost[9] = {-1, 1, 7, 3, 5, 0, 4, 2, 6};
    for (int k = 0, placed = 0; k < 9; k++)
        for (int c = 0; c < C; c++)
            if (cls[c] == by_cost[k]) sorted[placed++] = c;
    hdr[7] = hdr[6] + (int32_t)taps_class_bytes(C);
    int8_t *extent = (int8_t *)taps_host + hdr[7];
    for (int c = 0; c < C; c++)
        for (int s = 0; s < K; s++)
            for (int k = 0; k < 2; k++) {
                const int a = abs((int)dhdw[((size_t)c * K + s) * 2 + k]);
                if (a > extent[2 * c + k]) extent[2 * c + k] = (int8_t)a;
            }
    return DWO_OK;
}

int dwo_taps_get(const void *taps_host, int c, int s, int *dh, int *dw) {
    if (taps_host == nullptr || dh == nullptr || dw == nullptr) return DWO_ERR_NULL_POINTER;
    const int32_t *hdr = (const int32_t *)taps_host;
    if (hdr[0] != kTapsMagic || hdr[1] != kTapsVersion) return DWO_ERR_BAD_TAPS;
    if (c < 0 || c >= hdr[2] || s < 0 || s >= hdr[3]) return DWO_ERR_BAD_SHAPE;
    const int8_t *dhdw = taps_dhdw(taps_host);
    *dh = dhdw[((size_t)c * hdr[3] + s) * 2];
    *dw = dhdw[((size_t)c * hdr[3] + s) * 2 + 1];
    return DWO_OK;
}

int dwo_fprop(const void *x, const float *w, const float *bias, const void *taps, void *y, int N,
              int C, int H, int W, int K, int stride, int dtype, int layout, void *stream) {
    int rc = check_common(N, C, H, W, K, stride, dtype, layout);
    if (rc != DWO_OK) return rc;
    if (!x || !w || !taps || !y) return DWO_ERR_NULL_POINTER;
    const ConvDims d = make_dims(N, C, H, W, K, stride);
    hipStream_t st = (hipStream_t)stream;
    begin_call();
    switch (dtype) {
        case DWO_F32: return fprop_t<float>(x, w, bias, taps, y, d, layout, st);
        case DWO_BF16: return fprop_t<bf16_t>(x, w, bias, taps, y, d, layout, st);
        default: return fprop_t<f16_t>(x, w, bias, taps, y, d, layout, st);
    }
}

int dwo_dgrad(const void *dy, const float *w, const void *taps, void *dx, int N, int C, int H,
              int W, int K, int stride, int dtype, int layout, void *stream) {
    int rc = check_common(N, C, H, W, K, stride, dtype, layout);
    if (rc != DWO_OK) return rc;
    if (!dy || !w || !taps || !dx) return DWO_ERR_NULL_POINTER;
    const ConvDims d = make_dims(N, C, H, W, K, stride);
    hipStream_t st = (hipStream_t)stream;
    begin_call();
    switch (dtype) {
        case DWO_F32: return dgrad_t<float>(dy, w, taps, dx, d, layout, st);
        case DWO_BF16: return dgrad_t<bf16_t>(dy, w, taps, dx, d, layout, st);
        default: return dgrad_t<f16_t>(dy, w, taps, dx, d, layout, st);
    }
}

size_t dwo_wgrad_scratch_bytes(int N, int C, int H, int W, int K, int stride, int dtype,
                               int layout) {
    if (check_common(N, C, H, W, K, stride, dtype, layout) != DWO_OK) return 0;
    const ConvDims d = make_dims(N, C, H, W, K, stride);
    return (size_t)C * (K + 1) * wgrad_max_partials(d, layout, dtype == DWO_F32 ? 4 : 2) * sizeof(float);
}

int dwo_wgrad(const void *dy, const void *x, const void *taps, float *dw, float *db,
              void *scratch, size_t scratch_bytes, int N, int C, int H, int W, int K, int stride,
              int dtype, int layout, void *stream) {
    int rc = check_common(N, C, H, W, K, stride, dtype, layout);
    if (rc != DWO_OK) return rc;
    if (!dy || !x || !taps || !dw || !scratch) return DWO_ERR_NULL_POINTER;
    if (scratch_bytes < dwo_wgrad_scratch_bytes(N, C, H, W, K, stride, dtype, layout))
        return DWO_ERR_SCRATCH_TOO_SMALL;
    return wgrad_dispatch(dy, x, taps, dw, db, scratch, N, C, H, W, K, stride, dtype, layout,
                          (hipStream_t)stream);
}

int dwo_wgrad_static(const void *dy, const void *x, const void *taps, float *dw, float *db, int N,
                     int C, int H, int W, int K, int stride, int dtype, int layout, void *stream) {
    int rc = check_common(N, C, H, W, K, stride, dtype, layout);
    if (rc != DWO_OK) return rc;
    if (!dy || !x || !taps || !dw) return DWO_ERR_NULL_POINTER;
    if (dwo_wgrad_scratch_bytes(N, C, H, W, K, stride, dtype, layout) > DWO_STATIC_SCRATCH_BYTES)
        return DWO_ERR_STATIC_SCRATCH_LIMIT;
    void *scratch = nullptr;
    rc = static_scratch(&scratch);
    if (rc != DWO_OK) return rc;
    return wgrad_dispatch(dy, x, taps, dw, db, scratch, N, C, H, W, K, stride, dtype, layout,
                          (hipStream_t)stream);
}

int dwo_pointwise_fprop_nhwc(const void *x, const float *pw_w, const float *pw_b, const float *w,
                             const float *bias, const void *taps, void *y, int N, int Cin, int C,
                             int H, int W, int K, int stride, int dtype, void *stream) {
    int rc = check_common(N, C, H, W, K, stride, dtype, DWO_NHWC);
    if (rc != DWO_OK) return rc;
    if (!x || !pw_w || !w || !taps || !y) return DWO_ERR_NULL_POINTER;
    if (Cin < 1 || Cin > 4 || C % kSliceCh != 0) return DWO_ERR_BAD_SHAPE;
    const ConvDims d = make_dims(N, C, H, W, K, stride);
    hipStream_t st = (hipStream_t)stream;
    begin_call();
    switch (dtype) {
        case DWO_F32: return pointwise_fprop_t<float>(x, pw_w, pw_b, w, bias, taps, y, Cin, d, st);
        case DWO_BF16: return pointwise_fprop_t<bf16_t>(x, pw_w, pw_b, w, bias, taps, y, Cin, d, st);
        default: return pointwise_fprop_t<f16_t>(x, pw_w, pw_b, w, bias, taps, y, Cin, d, st);
    }
}

int dwo_layernorm_nhwc(const void *x, const float *gamma, const float *beta, void *out,
                       size_t rows, int C, float eps, int gelu, int dtype, void *stream) {
    if (!x || !gamma || !beta || !out) return DWO_ERR_NULL_POINTER;
    if (rows < 1 || C < 2 || (C & 1) || C > kFusedMaxC) return DWO_ERR_BAD_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    begin_call();
    switch (dtype) {
        case DWO_F32: return launch_layernorm_nhwc<float>(x, gamma, beta, out, (long)rows, C, eps, gelu, st);
        case DWO_BF16: return launch_layernorm_nhwc<bf16_t>(x, gamma, beta, out, (long)rows, C, eps, gelu, st);
        case DWO_F16: return launch_layernorm_nhwc<f16_t>(x, gamma, beta, out, (long)rows, C, eps, gelu, st);
        default: return DWO_ERR_BAD_DTYPE;
    }
}

int dwo_nchw_layernorm_nhwc(const void *x, const float *gamma, const float *beta, void *out, int N,
                            int C, int H, int W, float eps, int dtype, void *stream) {
    if (!x || !gamma || !beta || !out) return DWO_ERR_NULL_POINTER;
    if (N < 1 || N > 65535 || H < 1 || W < 1 || C < 2 || (C & 1) || C > kFusedMaxTileC ||
        (long)H * W > 0x7fffffffL / C)
        return DWO_ERR_BAD_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    begin_call();
    switch (dtype) {
        case DWO_F32: return launch_nchw_layernorm_nhwc<float>(x, gamma, beta, out, N, C, H * W, eps, st);
        case DWO_BF16: return launch_nchw_layernorm_nhwc<bf16_t>(x, gamma, beta, out, N, C, H * W, eps, st);
        case DWO_F16: return launch_nchw_layernorm_nhwc<f16_t>(x, gamma, beta, out, N, C, H * W, eps, st);
        default: return DWO_ERR_BAD_DTYPE;
    }
}

int dwo_nhwc_scale_add_nchw(const void *y, const float *scale, const void *res, void *out, int N,
                            int C, int H, int W, int dtype, void *stream) {
    if (!y || !out) return DWO_ERR_NULL_POINTER;
    if (N < 1 || N > 65535 || H < 1 || W < 1 || C < 2 || (C & 1) || (long)H * W > 0x7fffffffL / C)
        return DWO_ERR_BAD_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    begin_call();
    switch (dtype) {
        case DWO_F32: return launch_nhwc_scale_add_nchw<float>(y, scale, res, out, N, C, H * W, st);
        case DWO_BF16: return launch_nhwc_scale_add_nchw<bf16_t>(y, scale, res, out, N, C, H * W, st);
        case DWO_F16: return launch_nhwc_scale_add_nchw<f16_t>(y, scale, res, out, N, C, H * W, st);
        default: return DWO_ERR_BAD_DTYPE;
    }
}

}  // extern "C"

// LDS-staged NHWC kernels for stride 1 with compile-time plane extents.
//
// A workgroup owns kSliceCh consecutive channels of a run of images.  Per batch of PBI images it
// loads, for every pixel, the 16-byte (fp32) or 8-byte (16-bit) slice holding its channels, and
// scatters it into one zero-haloed LDS plane per (channel, image) laid out for that channel's
// orientation -- the same planes the NCHW kernels stage.  The workgroup's threads are split into
// kSliceCh sub-groups; sub-group k runs the straight-line body of channel k's orientation over
// that channel's planes (different sub-groups run different bodies at the same time).  Results
// go back into the interiors of the planes they came from and leave as pixel slices again.
// The other channels of a 128-byte line belong to sibling workgroups; the task order places
// them on the same XCD at the same time so the line is fetched from HBM once and merged in L2
// on the way out, hence cached (not non-temporal) global accesses here.
#pragma once

#include "dwo_static.h"

namespace dwo {


// Plane layout of one orientation class as run-time data (staging and write-out handle four
// channels with different layouts in one loop).
struct GeoRt {
    short pt, rs, pl, sub, ish;
};
template <int K, int H, int W, int O>
constexpr GeoRt geo_rt_of() {
    using G = Geo<O, K, tile_L<H, W>(O), H, W>;
    return GeoRt{(short)G::PT, (short)G::RS, (short)G::PL, (short)G::SUB, (short)(G::CLS == CLS_H)};
}
template <int K, int H, int W>
__device__ __forceinline__ GeoRt geo_rt(int o) {
    using TM = TableMap<K, H, W>;
    switch (o) {
        case 0: return geo_rt_of<K, H, W, 0>();
        case 1: return geo_rt_of<K, H, W, 1>();
        case 2: return geo_rt_of<K, H, W, 2>();
        case 3: return geo_rt_of<K, H, W, 3>();
        case 4: return geo_rt_of<K, H, W, 4>();
        case 5: return geo_rt_of<K, H, W, 5>();
        case 6: return geo_rt_of<K, H, W, 6>();
        case 7: return geo_rt_of<K, H, W, 7>();
        default: return GeoRt{(short)TM::PAD, (short)TM::RS, (short)TM::PL, 1, 0};
    }
}
template <int LH>
__device__ __forceinline__ unsigned rt_index(const GeoRt &g, unsigned r, unsigned w) {
    const unsigned u = w + g.pl;
    const unsigned col = g.ish ? (u % LH) * g.sub + u / LH : u;
    return (r + g.pt) * g.rs + col;
}

// Workgroup id -> task (image group, channel slice), slices fastest.  Hardware deals
// consecutive ids to the eight XCDs in turn; within every aligned block of 8*E tasks the order
// is permuted so that the E slices of one 128-byte line get ids that land on one XCD.
// When a pixel is not a whole number of lines (96 channels of a 16-bit type: 192 bytes) a line
// holds slices of two pixels and no split of the slices keeps it on one XCD: then whole image
// groups go to an XCD instead (group g to XCD g mod 8, all its slices with it), for as many
// rounds of eight groups as there are.  (Measured at 96 x 56 x 56, bf16: 234 MB crossed the
// fabric per fprop launch for 77 MB of tensors before this, every line fetched by three XCDs.)
__device__ __forceinline__ void nhwc_task(int nslices, int groups, int E, int &slice, int &group) {
    const int id = blockIdx.x, total = nslices * groups, B = 8 * E;
    if (nslices % E != 0) {
        const int whole = (groups / 8) * 8 * nslices;  // tasks of whole rounds of eight groups
        if (id < whole) {
            const int j = id / 8;
            group = id % 8 + 8 * (j / nslices);
            slice = j % nslices;
        } else {
            slice = id % nslices;
            group = id / nslices;
        }
        return;
    }
    const int blk = id / B;
    int tau = id;
    if (blk * B + B <= total) {
        const int r = id - blk * B;
        tau = blk * B + (r % 8) * E + r / 8;
    }
    slice = tau % nslices;
    group = tau / nslices;
}

// Shared state of the workgroup: global bases of its channel slice, the layouts of its four
// channels, and the registers holding the batch in flight.
template <typename T, int K, int H, int W>
struct NhwcCtx {
    static constexpr int NT = NhwcTile<H, W>::NT, PBI = NhwcTile<H, W>::PBI;
    static constexpr int HW = H * W, PLS = plane_floats<K, H, W>();
    static constexpr int PF = (PBI * HW + NT - 1) / NT;  // pixel slices per thread and batch
    static constexpr int LH = Tile<H, W>::LH;
    const T *src;  // + c0
    T *dst;        // + c0
    float *lds;
    unsigned C;
    int n1;
    GeoRt g[kSliceCh];
    Vec4<T> pre[PF];

    __device__ __forceinline__ void zero_fill() {
        lds_zero<NT>(lds, kSliceCh * PBI * PLS);
    }
    __device__ __forceinline__ void prefetch(int nb) {
        const T *base = src + (size_t)nb * HW * C;
#pragma unroll
        for (int k = 0; k < PF; k++) {
            const unsigned v = threadIdx.x + k * NT;
            if (v < PBI * HW && nb + (int)(v / HW) < n1) pre[k].load_cached(base + v * C);
        }
    }
    __device__ __forceinline__ void commit(int nb) {
#pragma unroll
        for (int k = 0; k < PF; k++) {
            const unsigned v = threadIdx.x + k * NT;
            if (v < PBI * HW && nb + (int)(v / HW) < n1) {
                const unsigned img = v / HW, p = v % HW, r = p / W, w = p % W;
#pragma unroll
                for (int ch = 0; ch < kSliceCh; ch++)
                    lds[(ch * PBI + img) * PLS + rt_index<LH>(g[ch], r, w)] = pre[k].get(ch);
            }
        }
    }
    // results sit where the inputs were; each thread writes out the slices it staged (and will
    // stage next), so no barrier is needed between this and the next commit
    __device__ __forceinline__ void flush(int nb) {
        T *base = dst + (size_t)nb * HW * C;
#pragma unroll
        for (int k = 0; k < PF; k++) {
            const unsigned v = threadIdx.x + k * NT;
            if (v < PBI * HW && nb + (int)(v / HW) < n1) {
                const unsigned img = v / HW, p = v % HW, r = p / W, w = p % W;
                float o[kSliceCh];
#pragma unroll
                for (int ch = 0; ch < kSliceCh; ch++)
                    o[ch] = lds[(ch * PBI + img) * PLS + rt_index<LH>(g[ch], r, w)];
                Vec4<T> out;
                out.set(o[0], o[1], o[2], o[3]);
                out.store_cached(base + v * C);
            }
        }
    }
};

// Sub-group body for a canonical orientation.  All bodies (this one for any O, and the table
// one) execute the same sequence of workgroup barriers: one after the zero fill, three per batch.
template <int O, int OP, typename T, int K, int H, int W>
__device__ __forceinline__ void nhwc_canonical(NhwcCtx<T, K, H, W> &ctx, const float *__restrict__ wt,
                                               const float *__restrict__ bias, int c, int sub,
                                               unsigned stid, int n0) {
    using Ctx = NhwcCtx<T, K, H, W>;
    constexpr int L = tile_L<H, W>(O);
    constexpr int PBI = Ctx::PBI, NTS = Ctx::NT / kSliceCh, PLS = Ctx::PLS;
    using G = Geo<O, K, L, H, W>;
    constexpr int ITERS = (PBI * G::IPP + NTS - 1) / NTS;
    ChannelTaps<G, OP, T, K, false> taps;
    taps.load(wt, bias, c);
    float *planes = ctx.lds + sub * PBI * PLS;

    ctx.zero_fill();
    ctx.prefetch(n0);
    __syncthreads();
    for (int nb = n0; nb < ctx.n1; nb += PBI) {
        const int nvalid = ctx.n1 - nb;
        ctx.commit(nb);
        __syncthreads();
        if (nb + PBI < ctx.n1) ctx.prefetch(nb + PBI);
        float acc[ITERS][L];
#pragma unroll
        for (int iter = 0; iter < ITERS; iter++) {
            const unsigned item = stid + iter * NTS;
            const unsigned pl = item / G::IPP, it = item % G::IPP;
            const unsigned rb = it / G::IPR, j = it % G::IPR;
            if (item < PBI * G::IPP && (int)pl < nvalid)
                taps.accumulate(planes + (pl * PLS + rb * (G::LR * G::RS) + j), acc[iter]);
        }
        __syncthreads();  // every read of the staged inputs is done
#pragma unroll
        for (int iter = 0; iter < ITERS; iter++) {
            const unsigned item = stid + iter * NTS;
            const unsigned pl = item / G::IPP, it = item % G::IPP;
            const unsigned rb = it / G::IPR, j = it % G::IPR;
            if (item < PBI * G::IPP && (int)pl < nvalid) {
                float *plane = planes + pl * PLS;
#pragma unroll
                for (int l = 0; l < L; l++) {
                    if constexpr (G::CLS == CLS_H) {
                        plane[GeoMap<G>::index(rb, j * L + l)] = acc[iter][l];
                    } else if constexpr (G::CLS == CLS_V) {
                        if (H % L == 0 || rb * L + l < H)
                            plane[GeoMap<G>::index(rb * L + l, j)] = acc[iter][l];
                    } else {
                        const unsigned q = j + (unsigned)(l - G::Q0);  // wraps when negative
                        const unsigned row = rb * L + G::P0 + l * G::EH;
                        if (q < W && (H % L == 0 || row < H))
                            plane[GeoMap<G>::index(row, q)] = acc[iter][l];
                    }
                }
            }
        }
        __syncthreads();
        ctx.flush(nb);
    }
}

// Sub-group body for a channel with arbitrary taps (offsets and weights of the live taps are kept
// in LDS behind the planes).
template <int OP, typename T, int K, int H, int W>
__device__ __forceinline__ void nhwc_table(NhwcCtx<T, K, H, W> &ctx, const float *__restrict__ wt,
                                           const float *__restrict__ bias,
                                           const int8_t *__restrict__ dhdw, int c, int sub,
                                           unsigned stid, int n0) {
    using Ctx = NhwcCtx<T, K, H, W>;
    using Map = TableMap<K, H, W>;
    constexpr int PBI = Ctx::PBI, NTS = Ctx::NT / kSliceCh, PLS = Ctx::PLS, HW = Ctx::HW;
    constexpr int PER = (PBI * HW + NTS - 1) / NTS;
    static_assert((H + 2 * Map::PAD) * Map::RS <= PLS, "table body staging must fit the plane stride");
    float *planes = ctx.lds + sub * PBI * PLS;
    int *toff = reinterpret_cast<int *>(ctx.lds + kSliceCh * PBI * PLS + sub * (2 * K + 1));
    float *twt = reinterpret_cast<float *>(toff + K);
    int *nlive_p = toff + 2 * K;
    if (stid == 0) {
        int nl = 0;
        for (int s = 0; s < K; s++) {
            const int dh = dhdw[((size_t)c * K + s) * 2], dw = dhdw[((size_t)c * K + s) * 2 + 1];
            if (dh >= H || dh <= -H || dw >= W || dw <= -W) continue;
            toff[nl] = (OP == OP_DGRAD ? -1 : 1) * (dh * Map::RS + dw);
            twt[nl] = wt[(size_t)c * K + s];
            nl++;
        }
        *nlive_p = nl;
    }
    const float bv = (OP == OP_FPROP && bias != nullptr) ? bias[c] : 0.f;
    ctx.zero_fill();
    ctx.prefetch(n0);
    __syncthreads();
    for (int nb = n0; nb < ctx.n1; nb += PBI) {
        const int nvalid = ctx.n1 - nb;
        ctx.commit(nb);
        __syncthreads();
        if (nb + PBI < ctx.n1) ctx.prefetch(nb + PBI);
        const int nlive = *nlive_p;
        float acc[PER];
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const unsigned f = stid + i * NTS;
            const unsigned pl = f / HW, p = f % HW;
            acc[i] = bv;
            if (f < PBI * HW && (int)pl < nvalid) {
                const float *base = planes + pl * PLS + Map::index(p / W, p % W);
                for (int s = 0; s < nlive; s++) acc[i] = __builtin_fmaf(base[toff[s]], twt[s], acc[i]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const unsigned f = stid + i * NTS;
            const unsigned pl = f / HW, p = f % HW;
            if (f < PBI * HW && (int)pl < nvalid) planes[pl * PLS + Map::index(p / W, p % W)] = acc[i];
        }
        __syncthreads();
        ctx.flush(nb);
    }
}

template <int K, int H, int W>
constexpr size_t nhwc_plane_lds_bytes() {
    return ((size_t)kSliceCh * NhwcTile<H, W>::PBI * plane_floats<K, H, W>() +
            kSliceCh * (2 * K + 1)) * sizeof(float);
}

template <int OP, typename T, int K, int H, int W>
__global__ __launch_bounds__((NhwcTile<H, W>::NT)) void nhwc_plane_kernel(
    const T *__restrict__ src, const float *__restrict__ wt, const float *__restrict__ bias,
    const void *__restrict__ blob, T *__restrict__ dst, int N, int C, int groups) {
    extern __shared__ float lds[];
    using Ctx = NhwcCtx<T, K, H, W>;
    constexpr int NTS = Ctx::NT / kSliceCh;
    static_assert(NTS % 64 == 0, "sub-groups are whole waves");
    int slice, group;
    nhwc_task(C / kSliceCh, groups, 128 / (kSliceCh * (int)sizeof(T)), slice, group);
    int n0, n1;
    group_range<Ctx::PBI>(N, groups, group, n0, n1);
    const int c0 = slice * kSliceCh;
    Ctx ctx;
    ctx.src = src + c0;
    ctx.dst = dst + c0;
    ctx.lds = lds;
    ctx.C = (unsigned)C;
    ctx.n1 = n1;
    const int32_t *cls = taps_class(blob, C, K) + c0;
#pragma unroll
    for (int ch = 0; ch < kSliceCh; ch++) {
        ctx.g[ch] = geo_rt<K, H, W>(cls[ch]);
    }
    const int sub = __builtin_amdgcn_readfirstlane(threadIdx.x / NTS);
    const unsigned stid = threadIdx.x % NTS;
    const int c = c0 + sub;
    const int mine = cls[sub];
#define DWO_CASE(O)                                                             \
    case O:                                                                     \
        nhwc_canonical<O, OP, T, K, H, W>(ctx, wt, bias, c, sub, stid, n0);      \
        break;
    switch (mine) {
        DWO_CASE(0)
        DWO_CASE(1)
        DWO_CASE(2)
        DWO_CASE(3)
        DWO_CASE(4)
        DWO_CASE(5)
        DWO_CASE(6)
        DWO_CASE(7)
        default:
            nhwc_table<OP, T, K, H, W>(ctx, wt, bias, taps_dhdw(blob), c, sub, stid, n0);
    }
#undef DWO_CASE
}

// register-plane kernels (dwo_regplane.h) take fprop and dgrad of planes of at most 16 x 16 when
// the channel count is a multiple of their 32-channel blocks
template <typename T, int K, int H, int W>
int launch_regplane_nhwc_conv(int op, const void *src, const float *w, const float *bias,
                              const void *taps, void *dst, int N, int C, hipStream_t st);

// C must be a multiple of kSliceCh (the caller checks).
template <typename T, int K, int H, int W>
int launch_nhwc_plane_conv(int op, const void *src, const float *w, const float *bias,
                           const void *taps, void *dst, int N, int C, hipStream_t st) {
    if constexpr (!nhwc_plane_shape<H, W>()) {
        return N == 0 ? 0 : -100;  // not built for this extent
    } else {
    if constexpr (reg_plane_shape<H, W>()) {
        if (N > 0 && N <= 65535 && C % 32 == 0)
            return launch_regplane_nhwc_conv<T, K, H, W>(op, src, w, bias, taps, dst, N, C, st);
    }
    constexpr int NT = NhwcTile<H, W>::NT, PBI = NhwcTile<H, W>::PBI;
    const size_t lds = nhwc_plane_lds_bytes<K, H, W>();
    static int cache[kMaxDevices];
    const int slots = per_device_once(cache, [&] {
        allow_large_lds(nhwc_plane_kernel<OP_FPROP, T, K, H, W>, lds);
        allow_large_lds(nhwc_plane_kernel<OP_DGRAD, T, K, H, W>, lds);
        return resident_slots(nhwc_plane_kernel<OP_FPROP, T, K, H, W>, NT, lds) & 0xffff;
    });
    if (N == 0) return 0;  // set-up only
    const int nslices = C / kSliceCh;
    const int groups = plane_groups(N, nslices, PBI, slots);
    const dim3 grid(nslices * groups), block(NT);
    if (op == OP_FPROP)
        nhwc_plane_kernel<OP_FPROP, T, K, H, W><<<grid, block, lds, st>>>(
            (const T *)src, w, bias, taps, (T *)dst, N, C, groups);
    else
        nhwc_plane_kernel<OP_DGRAD, T, K, H, W><<<grid, block, lds, st>>>(
            (const T *)src, w, bias, taps, (T *)dst, N, C, groups);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
    }
}

// ---------------------------------------------------------------------------------------------
// wgrad
// ---------------------------------------------------------------------------------------------
// x goes into the padded planes as above; dy is staged unpadded behind them.  Where four padded
// and four unpadded planes do not fit in LDS together (56 x 56) the dy planes are staged in two
// phases of about half the rows each, cut at a row-block boundary of the channel's class, and a
// sub-group works through the row-blocks of one phase at a time.
template <int H, int W>
constexpr int nhwc_wgrad_phases() {
    return H * W >= 56 * 56 ? 2 : 1;
}
// row-blocks in phase 0 for an orientation with RB row-blocks
template <int H, int W>
constexpr int phase0_blocks(int RB) {
    return nhwc_wgrad_phases<H, W>() == 1 ? RB : (RB + 1) / 2;
}
template <int K, int H, int W, int O>
constexpr int split_row_of() {
    using G = Geo<O, K, tile_L<H, W>(O), H, W>;
    return cmin(H, phase0_blocks<H, W>(G::RB) * G::LR);
}
template <int K, int H, int W>
__device__ __forceinline__ int split_row(int o) {
    switch (o) {
        case 0: return split_row_of<K, H, W, 0>();
        case 1: return split_row_of<K, H, W, 1>();
        case 2: return split_row_of<K, H, W, 2>();
        case 3: return split_row_of<K, H, W, 3>();
        case 4: return split_row_of<K, H, W, 4>();
        case 5: return split_row_of<K, H, W, 5>();
        case 6: return split_row_of<K, H, W, 6>();
        case 7: return split_row_of<K, H, W, 7>();
        default: return phase0_blocks<H, W>(H);
    }
}
template <int K, int H, int W, int... Os>
constexpr int max_dy_rows(std::integer_sequence<int, Os...>) {
    int m = cmax(phase0_blocks<H, W>(H), H - phase0_blocks<H, W>(H));
    ((m = cmax(m, cmax(split_row_of<K, H, W, Os>(), H - split_row_of<K, H, W, Os>()))), ...);
    return m;
}
// floats per staged dy plane
template <int K, int H, int W>
constexpr int dy_plane_floats() {
    return max_dy_rows<K, H, W>(std::make_integer_sequence<int, 8>{}) * W;
}
template <int K, int H, int W>
constexpr int nhwc_dy_offset() {
    return (kSliceCh * NhwcTile<H, W>::PBI * plane_floats<K, H, W>() + kSliceCh * (2 * K + 1) + 3) & ~3;
}
template <int K, int H, int W>
constexpr size_t nhwc_plane_wgrad_lds_bytes() {
    return ((size_t)nhwc_dy_offset<K, H, W>() +
            kSliceCh * NhwcTile<H, W>::PBI * dy_plane_floats<K, H, W>()) * sizeof(float);
}

template <typename T, int K, int H, int W>
struct NhwcWgradCtx : NhwcCtx<T, K, H, W> {
    using Base = NhwcCtx<T, K, H, W>;
    static constexpr int DYP = dy_plane_floats<K, H, W>();
    const T *dy;  // + c0
    short split[kSliceCh];
    Vec4<T> gpre[Base::PF];

    __device__ __forceinline__ float *dy_planes() const { return this->lds + nhwc_dy_offset<K, H, W>(); }
    __device__ __forceinline__ void prefetch_dy(int nb) {
        const T *base = dy + (size_t)nb * Base::HW * this->C;
#pragma unroll
        for (int k = 0; k < Base::PF; k++) {
            const unsigned v = threadIdx.x + k * Base::NT;
            if (v < Base::PBI * Base::HW && nb + (int)(v / Base::HW) < this->n1)
                gpre[k].load_cached(base + v * this->C);
        }
    }
    // rows [0, split) of channel ch in phase 0, [split, H) in phase 1
    __device__ __forceinline__ void commit_dy(int nb, int phase) {
        float *ldy = dy_planes();
#pragma unroll
        for (int k = 0; k < Base::PF; k++) {
            const unsigned v = threadIdx.x + k * Base::NT;
            if (v < Base::PBI * Base::HW && nb + (int)(v / Base::HW) < this->n1) {
                const unsigned img = v / Base::HW, p = v % Base::HW;
                const int r = p / W, w = p % W;
#pragma unroll
                for (int ch = 0; ch < kSliceCh; ch++) {
                    const int lo = phase == 0 ? 0 : split[ch];
                    const int hi = phase == 0 ? split[ch] : H;
                    if (r >= lo && r < hi)
                        ldy[(ch * Base::PBI + img) * DYP + (r - lo) * W + w] = gpre[k].get(ch);
                }
            }
        }
    }
};

// Sub-group epilogue: per-thread accumulators -> wave totals (DPP) -> LDS -> one value per tap
// handed to WgradOut.
template <int K, int NT, int NTS, class SlotOf>
__device__ __forceinline__ void wgrad_epilogue_sub(float (&acc)[K + 1], float *lds,
                                                   const WgradOut &out, int c, int sub,
                                                   unsigned stid, int group, SlotOf slot_of) {
    constexpr int NWS = NTS / 64;
    __syncthreads();  // staged planes are dead from here on
    // every lane leaves the half-wave sum of one accumulator in its wave's row of 64 words
    lds[threadIdx.x] = wave_reduce32(acc);
    __syncthreads();
    if (stid <= K) {
        const int slot = stid == K ? K : slot_of(stid);
        float t = 0.f;
        if (slot >= 0) {
            const unsigned l = reduce32_lane(slot);
            for (int w = 0; w < NWS; w++)
                t += lds[(sub * NWS + w) * 64 + l] + lds[(sub * NWS + w) * 64 + 32 + l];
        }
        out.put(c, (int)stid, group, K, t);
    }
    wgrad_finish<K>(out, lds, (c - sub) / kSliceCh, c - sub, kSliceCh);
}

// Barriers per batch are the same in every body: two per phase.
template <int O, typename T, int K, int H, int W>
__device__ __forceinline__ void nhwc_canonical_wgrad(NhwcWgradCtx<T, K, H, W> &ctx,
                                                     const WgradOut &out, int c, int sub,
                                                     unsigned stid, int n0, int group) {
    using Ctx = NhwcWgradCtx<T, K, H, W>;
    constexpr int L = tile_L<H, W>(O);
    constexpr int PBI = Ctx::PBI, NT = Ctx::NT, NTS = NT / kSliceCh, PLS = Ctx::PLS, DYP = Ctx::DYP;
    constexpr int NPH = nhwc_wgrad_phases<H, W>();
    using G = Geo<O, K, L, H, W>;
    constexpr int RB0 = phase0_blocks<H, W>(G::RB);
    const float *planes = ctx.lds + sub * PBI * PLS;
    const float *ldy = ctx.dy_planes() + sub * PBI * DYP;

    float acc[K + 1];  // acc[s] for representative taps s, acc[K] = sum of dy (bias gradient)
#pragma unroll
    for (int s = 0; s <= K; s++) acc[s] = 0.f;

    ctx.zero_fill();
    ctx.prefetch(n0);
    ctx.prefetch_dy(n0);
    __syncthreads();
    for (int nb = n0; nb < ctx.n1; nb += PBI) {
        const int nvalid = ctx.n1 - nb;
        static_for<NPH>([&](auto ph) {
            constexpr int rb0 = ph == 0 ? 0 : RB0, rb1 = (ph == 0 && NPH == 2) ? RB0 : G::RB;
            constexpr int NRB = rb1 - rb0, ROW0 = rb0 * G::LR;
            constexpr int ITERS = (PBI * NRB * G::IPR + NTS - 1) / NTS;
            if constexpr (ph == 0) ctx.commit(nb);
            ctx.commit_dy(nb, ph);
            __syncthreads();
            if (nb + PBI < ctx.n1) {
                if constexpr (ph == 0) ctx.prefetch(nb + PBI);
                if constexpr (ph == NPH - 1) ctx.prefetch_dy(nb + PBI);
            }
#pragma unroll
            for (int it = 0; it < ITERS; it++) {
                const unsigned item = stid + it * NTS;
                const unsigned pl = item / (NRB * G::IPR), ii = item % (NRB * G::IPR);
                const unsigned rb = rb0 + ii / G::IPR, j = ii % G::IPR;
                if (item < PBI * NRB * G::IPR && (int)pl < nvalid) {
                    // dy of the item's L outputs (zero where the output does not exist)
                    float d[L];
                    const float *g = ldy + pl * DYP - ROW0 * W;
                    if constexpr (G::CLS == CLS_H) {
                        // one wide read: L separate reads at a lane stride of L words conflict L ways
                        if constexpr (L == 4 && W % 4 == 0) {
                            const lds_f4 dv = lds_read4(g + rb * W + j * 4);
                            d[0] = dv[0], d[1] = dv[1], d[2] = dv[2], d[3] = dv[3];
                        } else if constexpr (L == 2 && W % 2 == 0) {
                            const lds_f2 dv = lds_read2(g + rb * W + j * 2);
                            d[0] = dv[0], d[1] = dv[1];
                        } else {
#pragma unroll
                            for (int l = 0; l < L; l++) d[l] = g[rb * W + j * L + l];
                        }
                    } else if constexpr (G::CLS == CLS_V) {
#pragma unroll
                        for (int l = 0; l < L; l++)
                            d[l] = (H % L == 0 || rb * L + l < H) ? g[(rb * L + l) * W + j] : 0.f;
                    } else {
#pragma unroll
                        for (int l = 0; l < L; l++) {
                            const unsigned q = j + (unsigned)(l - G::Q0);
                            const bool ok = q < W && (H % L == 0 || rb * L + G::P0 + l * G::EH < H);
                            d[l] = ok ? g[(int)(rb * (L * W) + j) + (G::P0 + l * G::EH) * W + l - G::Q0]
                                      : 0.f;
                        }
                    }
                    const float *base = planes + (pl * PLS + rb * (G::LR * G::RS) + j);
                    static_for<G::plan.nsrc>([&](auto m) {
                        constexpr int off = G::imm(G::plan.sh[m], G::plan.sw[m]);
                        const float v = base[off];
                        static_for<L>([&](auto l) {
                            constexpr int t = G::plan.user[m][l];
                            if constexpr (t >= 0) acc[t] = __builtin_fmaf(v, d[l], acc[t]);
                        });
                    });
                    pipeline_reads_and_fmas<G::plan.nsrc, plan_fma_count(G::plan, L)>();
#pragma unroll
                    for (int l = 0; l < L; l++) acc[K] += d[l];
                }
            }
            __syncthreads();  // staged x and dy of this phase are consumed
        });
    }
    wgrad_epilogue_sub<K, NT, NTS>(acc, ctx.lds, out, c, sub, stid, group,
                                   [](int s) { return (int)G::plan.rep[s]; });
}

template <typename T, int K, int H, int W>
__device__ __forceinline__ void nhwc_table_wgrad(NhwcWgradCtx<T, K, H, W> &ctx,
                                                 const int8_t *__restrict__ dhdw,
                                                 const WgradOut &out, int c, int sub,
                                                 unsigned stid, int n0, int group) {
    using Ctx = NhwcWgradCtx<T, K, H, W>;
    using Map = TableMap<K, H, W>;
    constexpr int PBI = Ctx::PBI, NT = Ctx::NT, NTS = NT / kSliceCh, PLS = Ctx::PLS, DYP = Ctx::DYP;
    constexpr int NPH = nhwc_wgrad_phases<H, W>();
    constexpr int R0 = phase0_blocks<H, W>(H);  // rows in phase 0
    const float *planes = ctx.lds + sub * PBI * PLS;
    const float *ldy = ctx.dy_planes() + sub * PBI * DYP;
    int *toff = reinterpret_cast<int *>(ctx.lds + kSliceCh * PBI * PLS + sub * (2 * K + 1));
    int *tlive = toff + K;  // dead taps read the centre and are zeroed at the end
    if (stid < K) {
        const int dh = dhdw[((size_t)c * K + stid) * 2], dw = dhdw[((size_t)c * K + stid) * 2 + 1];
        const bool dead = dh >= H || dh <= -H || dw >= W || dw <= -W;
        toff[stid] = dead ? 0 : dh * Map::RS + dw;
        tlive[stid] = dead ? -1 : (int)stid;
    }
    float acc[K + 1];
#pragma unroll
    for (int s = 0; s <= K; s++) acc[s] = 0.f;
    ctx.zero_fill();
    ctx.prefetch(n0);
    ctx.prefetch_dy(n0);
    __syncthreads();
    for (int nb = n0; nb < ctx.n1; nb += PBI) {
        const int nvalid = ctx.n1 - nb;
        static_for<NPH>([&](auto ph) {
            constexpr int row0 = ph == 0 ? 0 : R0, row1 = (ph == 0 && NPH == 2) ? R0 : H;
            constexpr int NPIX = (row1 - row0) * W;
            if constexpr (ph == 0) ctx.commit(nb);
            ctx.commit_dy(nb, ph);
            __syncthreads();
            if (nb + PBI < ctx.n1) {
                if constexpr (ph == 0) ctx.prefetch(nb + PBI);
                if constexpr (ph == NPH - 1) ctx.prefetch_dy(nb + PBI);
            }
            for (unsigned f = stid; f < PBI * NPIX; f += NTS) {
                const unsigned pl = f / NPIX, p = f % NPIX;
                if ((int)pl >= nvalid) break;
                const float gy = ldy[pl * DYP + p];
                const float *base = planes + pl * PLS + Map::index(row0 + p / W, p % W);
#pragma unroll
                for (int s = 0; s < K; s++)
                    acc[s] = __builtin_fmaf(base[*(volatile int *)&toff[s]], gy, acc[s]);
                acc[K] += gy;
            }
            __syncthreads();
        });
    }
    wgrad_epilogue_sub<K, NT, NTS>(acc, ctx.lds, out, c, sub, stid, group,
                                   [&](int s) { return tlive[s]; });
}

template <typename T, int K, int H, int W>
__global__ __launch_bounds__((NhwcTile<H, W>::NT)) void nhwc_plane_wgrad_kernel(
    const T *__restrict__ x, const T *__restrict__ dy, const void *__restrict__ blob,
    WgradOut out, int N, int C) {
    extern __shared__ float lds[];
    using Ctx = NhwcWgradCtx<T, K, H, W>;
    const int NG = out.NG;
    constexpr int NTS = Ctx::NT / kSliceCh;
    int slice, group;
    nhwc_task(C / kSliceCh, NG, 128 / (kSliceCh * (int)sizeof(T)), slice, group);
    int n0, n1;
    group_range<Ctx::PBI>(N, NG, group, n0, n1);
    const int c0 = slice * kSliceCh;
    Ctx ctx;
    ctx.src = x + c0;
    ctx.dst = nullptr;
    ctx.dy = dy + c0;
    ctx.lds = lds;
    ctx.C = (unsigned)C;
    ctx.n1 = n1;
    const int32_t *cls = taps_class(blob, C, K) + c0;
#pragma unroll
    for (int ch = 0; ch < kSliceCh; ch++) {
        ctx.g[ch] = geo_rt<K, H, W>(cls[ch]);
        ctx.split[ch] = (short)split_row<K, H, W>(cls[ch]);
    }
    const int sub = __builtin_amdgcn_readfirstlane(threadIdx.x / NTS);
    const unsigned stid = threadIdx.x % NTS;
    const int c = c0 + sub;
    const int mine = cls[sub];
#define DWO_CASE(O)                                                                     \
    case O:                                                                             \
        nhwc_canonical_wgrad<O, T, K, H, W>(ctx, out, c, sub, stid, n0, group);          \
        break;
    switch (mine) {
        DWO_CASE(0)
        DWO_CASE(1)
        DWO_CASE(2)
        DWO_CASE(3)
        DWO_CASE(4)
        DWO_CASE(5)
        DWO_CASE(6)
        DWO_CASE(7)
        default:
            nhwc_table_wgrad<T, K, H, W>(ctx, taps_dhdw(blob), out, c, sub, stid, n0, group);
    }
#undef DWO_CASE
}

// Same contract as launch_plane_wgrad.
template <typename T, int K, int H, int W>
int launch_nhwc_plane_wgrad(const void *x, const void *dy, const void *taps, float *part, float *dw,
                            float *db, unsigned *tickets, int N, int C, int *groups_out,
                            hipStream_t st) {
    if constexpr (!nhwc_plane_shape<H, W>()) {
        return N == 0 ? 0 : -100;  // not built for this extent
    } else {
    constexpr int NT = NhwcTile<H, W>::NT, PBI = NhwcTile<H, W>::PBI;
    const size_t lds = nhwc_plane_wgrad_lds_bytes<K, H, W>();
    static int cache[kMaxDevices];
    const int slots = per_device_once(cache, [&] {
        allow_large_lds(nhwc_plane_wgrad_kernel<T, K, H, W>, lds);
        return resident_slots(nhwc_plane_wgrad_kernel<T, K, H, W>, NT, lds) & 0xffff;
    });
    if (N == 0) return 0;  // set-up only
    const int nslices = C / kSliceCh;
    const int groups = plane_groups(N, nslices, PBI, slots);
    *groups_out = groups;
    nhwc_plane_wgrad_kernel<T, K, H, W><<<dim3(nslices * groups), dim3(NT), lds, st>>>(
        (const T *)x, (const T *)dy, taps, WgradOut{part, dw, db, groups, tickets}, N, C);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
    }
}

}  // namespace dwo

// LDS-staged NCHW kernels for stride 1 with compile-time plane extents.
//
// Workgroup (c, group): channel c, a run of G consecutive images.  PB planes (n, c) are staged
// at a time into LDS with a zero halo (zeroed once: only plane interiors are rewritten), so no
// tap needs a bounds test.  While a batch is being computed the next batch is already in
// flight from HBM into registers.  Channels whose taps match one of the eight canonical
// orientations run the straight-line body generated from dwo_plan.h; any other channel takes
// the table-driven body at the bottom (same staging, dynamic taps).
#pragma once

// Register budget of the plane kernels: at least six waves per SIMD, i.e. three 448-thread
// workgroups per CU (seven would need 72 registers and spill).
#define DWO_WPE 6
#ifndef DWO_WPE_WGRAD
#define DWO_WPE_WGRAD 6
#endif
// batches in flight from HBM per tensor in the wgrad kernels (register sets per tensor)
#ifndef DWO_WGRAD_DEPTH
#define DWO_WGRAD_DEPTH 1
#endif
// the same for planes of at most 16 x 16, whose register sets are one chunk per thread
// (measured at batch 64: depth 1 / 2 / 4 = 18.8 / 21.0 / 30.8 us at 14 x 14, 11.8 / 11.5 / 11.3 us
// at 7 x 7: these launches are not waiting for HBM)
#ifndef DWO_WGRAD_DEPTH_SMALL
#define DWO_WGRAD_DEPTH_SMALL 1
#endif

#include "dwo_common.h"
#include "dwo_dispatch.h"
#include "dwo_plan.h"

namespace dwo {

template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}



// All of the wave's outstanding global loads and stores have completed.  The kernels call this
// once per staged batch, unconditionally, right before the staged registers are written to LDS
// (which has to wait for them anyway).  Stated in straight-line code it also tells the compiler
// that nothing is pending when the next prefetch is issued: left to itself it places a full wait
// inside every conditionally executed load and LDS write of the batch loop (a load's address
// is computed in the registers the load will fill, which on some path still look busy), so
// that the second load of a batch was only issued after the first had come back from HBM.
__device__ __forceinline__ void wait_vmem_done() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), expcnt and lgkmcnt untouched
}

// Issue priority of the calling wave for its next staged batch, from the share of its batches it
// has finished: 3 at the start, falling to 0 in the last quarter.  The CU's instruction arbiter
// serves waves of equal priority oldest first, so of the workgroups that share a CU the one
// dispatched first ran at close to full speed and the last one crawled until the others had
// left: at 96 x 56 x 56 the workgroups of an fprop launch ended between 17 and 35 us after its
// start, and a CU spent the last third of the launch with one or two workgroups.  With the
// priority tied to progress a workgroup that is ahead yields to the ones behind it, whatever the
// dispatch order was: the same launch's workgroups end between 25.5 and 32.6 us, the launch
// 11 % earlier.
__device__ __forceinline__ void set_progress_priority(int done, int total) {
    const int p = 3 - min(3, done * 4 / total);
    if (p == 0) __builtin_amdgcn_s_setprio(0);
    else if (p == 1) __builtin_amdgcn_s_setprio(1);
    else if (p == 2) __builtin_amdgcn_s_setprio(2);
    else __builtin_amdgcn_s_setprio(3);
}
// (planes below 10 x 10: the eight-plane batches of the 7 x 7 wgrad measured 7 % slower with it)
template <int H, int W>
constexpr bool use_progress_priority() {
    return H * W >= 100;
}

// Four consecutive activations of type T as floats (one 16-byte or 8-byte global access).
// Activations are touched exactly once per pass, so all global accesses are non-temporal:
// outputs stream to HBM while the kernel runs instead of sitting dirty in L2 until the
// end-of-kernel write-back, and inputs do not displace them.
template <typename T>
struct Vec4;
// (native vector types: each load/store below is a single 16- or 8-byte memory instruction)
template <>
struct Vec4<float> {
    typedef float f4 __attribute__((ext_vector_type(4)));
    f4 v;
    __device__ __forceinline__ void load(const float *p) {
        v = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(p));
    }
    __device__ __forceinline__ void store(float *p) const {
        __builtin_nontemporal_store(v, reinterpret_cast<f4 *>(p));
    }
    // through the caches: for lines that other workgroups touch at about the same time
    __device__ __forceinline__ void load_cached(const float *p) { v = *reinterpret_cast<const f4 *>(p); }
    __device__ __forceinline__ void store_cached(float *p) const { *reinterpret_cast<f4 *>(p) = v; }
    __device__ __forceinline__ float get(int i) const { return v[i]; }
    __device__ __forceinline__ float elem(int i) const { return v[i]; }
    __device__ __forceinline__ void clear() { v = f4{0.f, 0.f, 0.f, 0.f}; }
    __device__ __forceinline__ uint16_t bits(int) const { return 0; }
    __device__ __forceinline__ void set(float a, float b, float c, float d) {
        v[0] = a, v[1] = b, v[2] = c, v[3] = d;
    }
};
template <>
struct Vec4<bf16_t> {
    typedef uint32_t u2 __attribute__((ext_vector_type(2)));
    u2 v;
    __device__ __forceinline__ void load(const bf16_t *p) {
        v = __builtin_nontemporal_load(reinterpret_cast<const u2 *>(p));
    }
    __device__ __forceinline__ void store(bf16_t *p) const {
        __builtin_nontemporal_store(v, reinterpret_cast<u2 *>(p));
    }
    __device__ __forceinline__ void load_cached(const bf16_t *p) { v = *reinterpret_cast<const u2 *>(p); }
    __device__ __forceinline__ void store_cached(bf16_t *p) const { *reinterpret_cast<u2 *>(p) = v; }
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = i < 2 ? v.x : v.y;
        return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    __device__ __forceinline__ uint16_t bits(int i) const {
        return (uint16_t)((i < 2 ? v.x : v.y) >> (16 * (i & 1)));
    }
    __device__ __forceinline__ bf16_t elem(int i) const { return bf16_t{bits(i)}; }
    __device__ __forceinline__ void clear() { v = u2{0u, 0u}; }
    __device__ __forceinline__ void set(float a, float b, float c, float d) {
        v.x = pack_bf16(a, b);
        v.y = pack_bf16(c, d);
    }
};
template <>
struct Vec4<f16_t> {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    h4 v;
    __device__ __forceinline__ void load(const f16_t *p) {
        v = __builtin_nontemporal_load(reinterpret_cast<const h4 *>(p));
    }
    __device__ __forceinline__ void store(f16_t *p) const {
        __builtin_nontemporal_store(v, reinterpret_cast<h4 *>(p));
    }
    __device__ __forceinline__ void load_cached(const f16_t *p) { v = *reinterpret_cast<const h4 *>(p); }
    __device__ __forceinline__ void store_cached(f16_t *p) const { *reinterpret_cast<h4 *>(p) = v; }
    __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
    __device__ __forceinline__ f16_t elem(int i) const { return v[i]; }
    __device__ __forceinline__ void clear() { v = h4{0, 0, 0, 0}; }
    __device__ __forceinline__ uint16_t bits(int i) const {
        return __builtin_bit_cast(uint16_t, (_Float16)v[i]);
    }
    __device__ __forceinline__ void set(float a, float b, float c, float d) {
        v[0] = (_Float16)a, v[1] = (_Float16)b, v[2] = (_Float16)c, v[3] = (_Float16)d;
    }
};

// The unrolled table bodies run all K taps of any angle, lanes along consecutive outputs.  The
// staged plane then has a halo of K / 2 on every side, so that a tap that misses the plane
// (|dh| >= H or |dw| >= W: small planes only) reads zeros like any tap that leaves it.  Used
// where a batch of such planes stays within 40 KB of LDS (every plane extent of the build but
// 7 x 7 at K = 31); elsewhere the halo stops at what a live tap can reach and the bodies loop
// over the live taps.
template <int K, int H, int W>
constexpr bool table_unrolled() {
    constexpr int PAD = K / 2, PL = (PAD + 3) & ~3;
    return Tile<H, W>::PB * (H + 2 * PAD) * (W + (PL + PAD + 31) / 32 * 32) * 4 <= 40 * 1024;
}
template <int K, int H, int W>
constexpr int table_pad() {
    return table_unrolled<K, H, W>() || K / 2 < cmax(H, W) - 1 ? K / 2 : cmax(H, W) - 1;
}
// Row stride of the table bodies' staged plane: left margin (a multiple of four words), row,
// right margin.  The unrolled bodies read one word per lane from consecutive outputs, which
// wrap from one row to the next inside a wave: with a stride that equals W modulo the 32 banks
// the wrapped lanes continue on the banks where the row left off (no conflicts at any offset).
template <int K, int H, int W>
constexpr int table_row_stride() {
    constexpr int PAD = table_pad<K, H, W>(), PL = (PAD + 3) & ~3;
    return table_unrolled<K, H, W>() ? W + (PL + PAD + 31) / 32 * 32 : W + PL + PAD;
}

// orientation classes with a pair form (16-bit activations)
constexpr bool pair_class(int cls) { return cls == CLS_H || cls == CLS_V; }

template <int K, int H, int W, int... Os>
constexpr int max_plane_floats(std::integer_sequence<int, Os...>) {
    constexpr int PAD = table_pad<K, H, W>();
    int m = (H + 2 * PAD) * cmax(W + 2 * PAD + 3, table_row_stride<K, H, W>());  // table-driven body
    ((m = cmax(m, Geo<Os, K, tile_L<H, W>(Os), H, W>::PLANE)), ...);
    ((m = cmax(m, Geo<Os, K, wgrad_L<H, W>(Os), H, W>::PLANE)), ...);
    // (pair geometries of the classes that have a pair form, see use_pairs)
    ((m = cmax(m, pair_class(orient_class(Os)) ? Geo<Os, K, tile_L<H, W>(Os), H, W, true>::PLANE : 0)), ...);
    return m;
}
// (a multiple of four words: planes keep the 16-byte alignment that wide LDS writes need)
template <int K, int H, int W>
constexpr int plane_floats() {
    return (max_plane_floats<K, H, W>(std::make_integer_sequence<int, 8>{}) + 3) & ~3;
}

// Zero `words` floats of LDS (a multiple of four, 16-byte aligned) with 16-byte writes.
template <int NT>
__device__ __forceinline__ void lds_zero(float *lds, unsigned words) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    for (unsigned i = threadIdx.x * 4; i < words; i += NT * 4)
        *reinterpret_cast<f4 *>(__builtin_assume_aligned(lds + i, 16)) = f4{0.f, 0.f, 0.f, 0.f};
}

// scalar stores of single results (4-byte ones non-temporal, like the vector stores)
__device__ __forceinline__ void st_out(float *p, float v) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ void st_out(f16_t *p, f16_t v) { *p = v; }
__device__ __forceinline__ void st_out(bf16_t *p, bf16_t v) { *p = v; }

// 16-bit patterns of the 16-bit element types, and the two-element dot product with fp32
// accumulation they feed (a and b each hold two elements; c + a.lo*b.lo + a.hi*b.hi).
__device__ __forceinline__ uint16_t raw16(bf16_t v) { return v.bits; }
__device__ __forceinline__ uint16_t raw16(f16_t v) { return __builtin_bit_cast(uint16_t, v); }
__device__ __forceinline__ uint16_t raw16(float) { return 0; }
__device__ __forceinline__ float dot2_acc(unsigned a, unsigned b, float c, bf16_t) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, a), __builtin_bit_cast(bf2, b), c,
                                           false);
}
__device__ __forceinline__ float dot2_acc(unsigned a, unsigned b, float c, f16_t) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, a), __builtin_bit_cast(h2, b), c, false);
}
__device__ __forceinline__ float dot2_acc(unsigned, unsigned, float c, float) { return c; }

// VL consecutive activations of a plane held in registers between the global load and the LDS
// write (VL = 4: one 16/8-byte access; VL = 1: planes whose size is not a multiple of four).
template <typename T, int VL>
struct Chunk;
template <typename T>
struct Chunk<T, 4> : Vec4<T> {};
template <typename T>
struct Chunk<T, 1> {
    T v;
    __device__ __forceinline__ void load(const T *p) { v = *p; }
    __device__ __forceinline__ float get(int) const { return to_float(v); }
    __device__ __forceinline__ uint16_t bits(int) const { return raw16(v); }
};

// Staging of PB planes (n, c), n = nb .. nb+PB-1, through registers into LDS.  `Map` gives the
// LDS index of interior element (r, w) relative to the plane's LDS origin, PLS the LDS distance
// between planes.  Global addresses are a uniform 64-bit base (plane (nb, c)) plus an unsigned
// 32-bit per-lane element offset.  Loads do not depend on the channel's orientation, so the
// kernels issue the first ones before they know which body will run.
template <typename T, int H, int W, int PB, int NT>
struct Stager {
    static constexpr int VL = (H * W) % 4 == 0 ? 4 : 1;
    static constexpr int FP = H * W / VL;              // chunks per plane
    static constexpr int PF = (PB * FP + NT - 1) / NT; // chunks per thread
    Chunk<T, VL> pre[PF];
    Chunk<T, VL> below[PF];  // the same columns one row further down (pair staging of the
                             // stacked class only; unused, it costs no registers)

    // base = first plane of the batch; `nvalid` planes of the batch exist
    __device__ __forceinline__ void prefetch(const T *__restrict__ base, unsigned plane_stride,
                                             int nvalid) {
#pragma unroll
        for (int k = 0; k < PF; k++) {
            const unsigned f = threadIdx.x + k * NT;
            const unsigned pl = f / FP, g = f % FP;
            if (f < PB * FP && (int)pl < nvalid) pre[k].load(base + (pl * plane_stride + g * VL));
        }
    }
    // the chunks one row below the ones prefetch() fetched (zeros below the last row)
    __device__ __forceinline__ void prefetch_below(const T *__restrict__ base,
                                                   unsigned plane_stride, int nvalid) {
        static_assert(VL == 1 || W % VL == 0, "rows must split into whole chunks");
#pragma unroll
        for (int k = 0; k < PF; k++) {
            const unsigned f = threadIdx.x + k * NT;
            const unsigned pl = f / FP, g = f % FP;
            if (f < PB * FP && (int)pl < nvalid) {
                if (g + W / VL < FP) below[k].load(base + (pl * plane_stride + g * VL + W));
                else below[k].clear();
            }
        }
    }
    template <class Map, int PLS>
    __device__ __forceinline__ void commit(float *lds, int nvalid) const {
#pragma unroll
        for (int k = 0; k < PF; k++) {
            const unsigned f = threadIdx.x + k * NT;
            const unsigned pl = f / FP, g = f % FP;
            if (f < PB * FP && (int)pl < nvalid) {
                float *plane = lds + pl * PLS;
                if constexpr (W % VL == 0 && Map::kChunked) {
                    const unsigned r = g / (W / VL), w0 = (g % (W / VL)) * VL;
                    float *q = plane + Map::index(r, w0);
                    if constexpr (VL == 4 && Map::kWide && PLS % 4 == 0) {
                        // the chunk's four words are adjacent and 16-byte aligned in LDS: one
                        // wide write (four 4-byte writes at a lane stride of four words would
                        // hit every bank four times)
                        typedef float f4 __attribute__((ext_vector_type(4)));
                        *reinterpret_cast<f4 *>(__builtin_assume_aligned(q, 16)) =
                            f4{pre[k].get(0), pre[k].get(1), pre[k].get(2), pre[k].get(3)};
                    } else {
#pragma unroll
                        for (int e = 0; e < VL; e++) q[Map::step(e)] = pre[k].get(e);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < VL; e++) {
                        const unsigned i = g * VL + e;
                        plane[Map::index(i / W, i % W)] = pre[k].get(e);
                    }
                }
            }
        }
    }
    // Pair staging for 16-bit activations: element (r, w) becomes the low half of the word at
    // (r, w) and the high half of the word at (r - EH, w - EW), so that every word holds an
    // element and its neighbour along the step direction (EH, EW).
    template <class Map, int PLS, int EH, int EW>
    __device__ __forceinline__ void commit_pairs(float *lds, int nvalid) const {
        uint16_t *half = reinterpret_cast<uint16_t *>(lds);
#pragma unroll
        for (int k = 0; k < PF; k++) {
            const unsigned f = threadIdx.x + k * NT;
            const unsigned pl = f / FP, g = f % FP;
            if (f < PB * FP && (int)pl < nvalid) {
                if constexpr (W % VL == 0) {
                    // one address per chunk; every half-word sits at a constant distance from it
                    const unsigned r = g / (W / VL), w0 = (g % (W / VL)) * VL;
                    uint16_t *q = half + 2 * (pl * PLS + Map::index((int)r, (int)w0));
                    if constexpr (EH == 0 && EW == 1 && VL == 4) {
                        // a chunk holds both halves of its first three words
                        unsigned *q32 = reinterpret_cast<unsigned *>(q);
#pragma unroll
                        for (int e = 0; e < 3; e++)
                            q32[Map::step(e)] =
                                (unsigned)pre[k].bits(e) | (unsigned)pre[k].bits(e + 1) << 16;
                        q[2 * Map::step(3)] = pre[k].bits(3);
                        q[2 * Map::pair_step(0) + 1] = pre[k].bits(0);
                    } else if constexpr (EH == 1 && EW == 0 && VL == 4) {
                        // both halves of the chunk's four words are in registers (own row and
                        // the row below): whole words, adjacent in LDS
                        unsigned *q32 = reinterpret_cast<unsigned *>(q);
                        typedef unsigned u4 __attribute__((ext_vector_type(4)));
                        u4 v;
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            v[e] = (unsigned)pre[k].bits(e) | (unsigned)below[k].bits(e) << 16;
                        if constexpr (Map::kWide && PLS % 4 == 0) {
                            *reinterpret_cast<u4 *>(__builtin_assume_aligned(q32, 16)) = v;
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++) q32[e] = v[e];
                        }
                        // the words above the first row hold (0, x[0][w])
                        if (r == 0) {
                            unsigned *up = q32 + ((int)Map::index(-1, 0) - (int)Map::index(0, 0));
#pragma unroll
                            for (int e = 0; e < 4; e++) up[e] = (unsigned)pre[k].bits(e) << 16;
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < VL; e++) {
                            const uint16_t v = pre[k].bits(e);
                            q[2 * Map::step(e)] = v;
                            q[2 * Map::pair_step(e) + 1] = v;
                        }
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < VL; e++) {
                        const unsigned i = g * VL + e;
                        const unsigned r = i / W, w = i % W;
                        const uint16_t v = pre[k].bits(e);
                        half[2 * (pl * PLS + Map::index((int)r, (int)w))] = v;
                        half[2 * (pl * PLS + Map::index((int)r - EH, (int)w - EW)) + 1] = v;
                    }
                }
            }
        }
    }
};

// Interior-element map of a canonical geometry.  step(e) is the LDS distance from element
// (r, w0) to (r, w0 + e) when w0 is a multiple of four and the row is at least four wide.
template <class G>
struct GeoMap {
    // rows whose four-element chunks land on 16-byte boundaries of adjacent words
    static constexpr bool kWide = G::CLS != CLS_H && G::RS % 4 == 0 && G::PL % 4 == 0;
    // step() below holds: a four-element chunk starts at a multiple of the interleave factor
    static constexpr bool kChunked = G::CLS != CLS_H || G::L_ < 4 || 4 % G::L_ == 0 || G::L_ % 4 == 0;
    static __device__ __forceinline__ unsigned index(int r, int w) {
        return G::interior_row(r) + G::col(w + G::PL);
    }
    static constexpr int step(int e) {
        return G::CLS == CLS_H ? (G::L_ >= 4 ? (e % G::L_) * G::SUB + e / G::L_
                                             : G::col(e + G::PL) - G::col(G::PL))
                               : e;
    }
    // distance from (r, w0) to the position one step (EH, EW) before (r, w0 + e)
    static constexpr int pair_step(int e) {
        return G::CLS == CLS_H ? (e > 0 ? step(e - 1) : (G::L_ - 1) * G::SUB - 1)
                               : e - G::EH * G::RS - G::EW;
    }
};

// Instruction-order hint for one unrolled item body of NSRC LDS reads feeding NFMA FMAs: reads
// are issued in chunks of CH, and the FMAs that consume chunk k are placed after the reads of
// chunk k+1, so a wave's LDS latency overlaps its own arithmetic instead of being waited out
// chunk by chunk.
template <int NSRC, int NFMA, int CH = 8>
__device__ __forceinline__ void pipeline_reads_and_fmas() {
    constexpr int NC = (NSRC + CH - 1) / CH;
    constexpr int PER = (NFMA + NC - 1) / NC;
    __builtin_amdgcn_sched_group_barrier(0x100, CH, 0);  // DS read
    static_for<NC>([&](auto) {
        __builtin_amdgcn_sched_group_barrier(0x100, CH, 0);  // next chunk's reads
        __builtin_amdgcn_sched_group_barrier(0x002, PER, 0); // FMAs of the previous chunk
    });
}

template <class P>
constexpr int plan_fma_count(const P &p, int L) {
    int n = 0;
    for (int m = 0; m < p.nsrc; m++)
        for (int l = 0; l < L; l++) n += p.user[m][l] >= 0 ? 1 : 0;
    return n;
}

// Workgroup -> (channel, image group) of fprop and dgrad.  Hardware hands consecutive workgroup
// ids to the eight XCDs round-robin and fills the CUs of an XCD in order.  Channels are taken
// from the tap table's class-cycling order (position p holds a channel of class p mod 8 while
// all classes last), and the task id is rotated inside every aligned block of eight ids by
// (block + block/32), so every XCD and every CU gets a mix of orientations (hence of costs).
__device__ __forceinline__ void plane_task(const void *blob, int C, int K, int groups, int &c,
                                           int &group) {
    const int i = blockIdx.x, total = C * groups;
    const int j = i >> 3;
    int t = i;
    if (j * 8 + 8 <= total) t = (j << 3) + ((i + j + (j >> 5)) & 7);
    c = taps_order(blob, C, K)[t % C];
    group = t / C;
}
// Workgroup -> (channel, image group) of wgrad.  Tasks are numbered channel-major over the tap
// table's cost-sorted channel list (most expensive orientation class first, a channel's image
// groups adjacent).  Workgroup ids b, b + cus, b + 2 cus, .. meet on one CU (see above) and a
// launch lasts as long as its most loaded CU, so the list is dealt to the CUs in rows of `cus`
// tasks, every second row backwards: the CUs that got the dearest tasks of one row get the
// cheapest of the next, and the sums per CU come out close to each other (class costs differ by
// a quarter at 56 x 56).  The host pads grids above `cus` to a multiple of it; returns false for
// a padding workgroup.
__device__ __forceinline__ bool wgrad_task(const void *blob, int C, int K, int groups, int cus,
                                           int &c, int &group) {
    const int b = blockIdx.x, total = C * groups;
    int tau = b;
    if ((int)gridDim.x > cus) {
        const int row = b / cus, cu = b - row * cus;
        // (backwards in blocks of eight: a task keeps its place modulo 8, i.e. its XCD, in every
        // row, so channels that are neighbours in memory and share cache lines on the small
        // planes still meet in one L2 when the class sizes are multiples of eight)
        const int back = (cus & 7) == 0 ? cus - 8 - (cu & ~7) + (cu & 7) : cus - 1 - cu;
        tau = row * cus + ((row & 1) ? back : cu);
    }
    if (tau >= total) return false;
    c = taps_sorted(blob, C, K)[tau / groups];
    group = tau % groups;
    return true;
}
// Images [n0, n1) of group g: the ceil(N/PB) staged batches are split as evenly as possible.
template <int PB>
__device__ __forceinline__ void group_range(int N, int groups, int g, int &n0, int &n1) {
    const int nbatch = (N + PB - 1) / PB;
    n0 = (int)(((long)g * nbatch) / groups) * PB;
    n1 = min((int)(((long)(g + 1) * nbatch) / groups) * PB, N);
}

// V and D class items produce one element per lane and row.  As 2-byte stores these run far
// below the rate of wider ones, so for 16-bit activations their results go through an unpadded fp32 out-tile in LDS (behind the
// planes and the tap tables) and leave as 16/8-byte non-temporal stores one batch later.
template <int K, int H, int W>
constexpr int out_tile_offset() {
    return (Tile<H, W>::PB * plane_floats<K, H, W>() + 2 * K + 3) & ~3;
}
template <typename T, int H, int W>
constexpr bool use_out_tile() {
    return (H * W) % 4 == 0;
}
// Which classes go through the out-tile.  16-bit activations: the stacked and the diagonal class
// (2-byte stores run far below the rate of wider ones).  fp32: the diagonal class (its
// row-shifted 4-byte stores measured 10 % slower than the tile's 16-byte ones) and, on planes
// staged one per batch, the stacked class (96 x 56 x 56, all channels at 90 degrees: fprop 42.1 ->
// 35.1 us, dgrad 39.3 -> 37.5; at 28 x 28 it measured 3-5 % slower).  The row-direction class
// stores 16 bytes per lane from registers and measured 5-10 % slower through the tile.
template <typename T, int CLS, int H, int W>
constexpr bool out_tile_class() {
    return CLS == CLS_D || (CLS == CLS_V && (sizeof(T) < 4 || Tile<H, W>::PB == 1));
}
template <typename T, int H, int W, int PB, int NT>
__device__ __forceinline__ void flush_out_tile(const float *lout, T *__restrict__ obase,
                                               unsigned pstride, int nvalid) {
    constexpr int FP = H * W / 4;
    for (unsigned f = threadIdx.x; f < PB * FP; f += NT) {
        const unsigned pl = f / FP, g = f % FP;
        if ((int)pl < nvalid) {
            const lds_f4 v = lds_read4(lout + f * 4);
            Vec4<T> r;
            r.set(v[0], v[1], v[2], v[3]);
            r.store(obase + (pl * pstride + g * 4));
        }
    }
}


// The two register sets of the fprop/dgrad pipeline; start() issues the loads of the first two
// batches of images [n0, n1) of channel c.
template <typename T, int H, int W>
struct ConvStagers {
    Stager<T, H, W, Tile<H, W>::PB, Tile<H, W>::NT> a, b;
    __device__ __forceinline__ void start(const T *__restrict__ src, int c, int C, int n0, int n1) {
        constexpr int PB = Tile<H, W>::PB;
        const unsigned pstride = (unsigned)C * (H * W);
        const T *sbase = src + (size_t)c * (H * W);
        a.prefetch(sbase + (size_t)n0 * pstride, pstride, n1 - n0);
        if (n0 + PB < n1) b.prefetch(sbase + (size_t)(n0 + PB) * pstride, pstride, n1 - n0 - PB);
    }
};

// Weights of one channel for a canonical geometry G, duplicates folded into their
// representative tap (and packed two taps to a word when PAIR), plus the bias; accumulate()
// is the straight-line body of one item: G::plan.nsrc LDS reads feeding L accumulators.
template <class G, int OP, typename T, int K, bool PAIR>
struct ChannelTaps {
    static constexpr int L = G::L_;
    static constexpr int NPAIR = [] {
        if constexpr (PAIR) return cmax((int)G::plan.npair, 1);
        else return 1;
    }();
    float wv[K];
    unsigned wp[NPAIR];
    float bv;

    __device__ __forceinline__ void load(const float *__restrict__ wt, const float *__restrict__ bias,
                                         int c) {
        const float *wc = wt + (size_t)c * K;
#pragma unroll
        for (int s = 0; s < K; s++) wv[s] = wc[OP == OP_DGRAD ? K - 1 - s : s];
        static_for<K>([&](auto s) {
            constexpr int r = G::plan.rep[s];
            if constexpr (r >= 0 && r != s) wv[r] += wv[s];
        });
        // folded sums are uniform: move them back to scalar registers
        static_for<K>([&](auto s) {
            if constexpr (s > 0 && G::plan.rep[s] >= 0 && G::plan.rep[s] != s) {
                constexpr int r = G::plan.rep[s];
                wv[r] = __builtin_bit_cast(
                    float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, wv[r])));
            }
        });
        bv = (OP == OP_FPROP && bias != nullptr) ? bias[c] : 0.f;
        // pair form: (tap, next tap along the run) as two 16-bit weights per uniform word
        if constexpr (PAIR) {
            static_for<NPAIR>([&](auto q) {
                constexpr int lo = G::plan.pair_lo[q], hi = G::plan.pair_hi[q];
                unsigned v = raw16(from_float<T>(wv[lo]));
                if constexpr (hi >= 0) v |= (unsigned)raw16(from_float<T>(wv[hi])) << 16;
                wp[q] = __builtin_amdgcn_readfirstlane(v);
            });
        }
    }

    __device__ __forceinline__ void accumulate(const float *base, float (&acc)[L]) const {
#pragma unroll
        for (int l = 0; l < L; l++) acc[l] = bv;
        static_for<G::plan.nsrc>([&](auto m) {
            constexpr int off = G::imm(G::plan.sh[m], G::plan.sw[m]);
            if constexpr (PAIR) {
                const unsigned v = reinterpret_cast<const unsigned *>(base)[off];
                static_for<L>([&](auto l) {
                    constexpr int q = G::plan.user[m][l];
                    if constexpr (q >= 0) acc[l] = dot2_acc(v, wp[q], acc[l], T{});
                });
            } else {
                const float v = base[off];
                static_for<L>([&](auto l) {
                    constexpr int t = G::plan.user[m][l];
                    if constexpr (t >= 0) acc[l] = __builtin_fmaf(v, wv[t], acc[l]);
                });
            }
        });
        pipeline_reads_and_fmas<G::plan.nsrc, plan_fma_count(G::plan, L)>();
    }
};

// ---------------------------------------------------------------------------------------------
// canonical body
// ---------------------------------------------------------------------------------------------
// 16-bit activations take the pair form: LDS words hold (x[pos], x[pos + e]) in the activation's
// own format, weights are rounded to that format and packed two taps to a word, and one dot2
// replaces two FMAs (accumulation stays fp32).
// Used where it measures faster: orientations whose step runs along a row (there most staged
// words leave a thread as whole 32-bit writes) on planes whose rows split into 4-element chunks.
template <typename T, int O, int W>
constexpr bool use_pairs() {
    return sizeof(T) == 2 && pair_class(orient_class(O)) && W % 4 == 0;
}
template <int O, int OP, typename T, int K, int H, int W>
__device__ __forceinline__ void run_canonical(const T *__restrict__ src, const float *__restrict__ wt,
                                              const float *__restrict__ bias, T *__restrict__ dst,
                                              float *lds, int c, int C, int n0, int n1,
                                              ConvStagers<T, H, W> &sg) {
    constexpr int L = tile_L<H, W>(O);
    constexpr int PB = Tile<H, W>::PB, NT = Tile<H, W>::NT;
    constexpr bool PAIR = use_pairs<T, O, W>();
    using G = Geo<O, K, L, H, W, PAIR>;
    constexpr int PLS = plane_floats<K, H, W>();  // LDS plane stride (same for all orientations)
    constexpr int ITERS = (PB * G::IPP + NT - 1) / NT;
    const unsigned tid = threadIdx.x;
    const unsigned pstride = (unsigned)C * (H * W);  // elements between images of one channel

    ChannelTaps<G, OP, T, K, PAIR> taps;
    taps.load(wt, bias, c);

    // zero the staging area once; interiors are overwritten per batch, halos stay zero
    lds_zero<NT>(lds, PB * PLS);

    const T *sbase = src + (size_t)c * (H * W);
    T *dbase = dst + (size_t)c * (H * W);
    // pair staging of the stacked class also needs every chunk's lower neighbour
    constexpr bool BELOW = PAIR && G::CLS == CLS_V;
    if constexpr (BELOW) {
        sg.a.prefetch_below(sbase + (size_t)n0 * pstride, pstride, n1 - n0);
        if (n0 + PB < n1) sg.b.prefetch_below(sbase + (size_t)(n0 + PB) * pstride, pstride, n1 - n0 - PB);
    }

    constexpr bool TILE = out_tile_class<T, G::CLS, H, W>() && use_out_tile<T, H, W>();
    float *lout = lds + out_tile_offset<K, H, W>();

    // results of item (pl, rb, j) of the batch that starts at obase -> global memory or out-tile
    auto emit = [&](T *obase, unsigned pl, unsigned rb, unsigned j, const float (&acc)[L]) {
        if constexpr (G::CLS == CLS_H) {
            T *o = obase + (pl * pstride + rb * W + j * L);
            if constexpr (L % 4 == 0) {
#pragma unroll
                for (int l = 0; l < L; l += 4) {
                    Vec4<T> r;
                    r.set(acc[l], acc[l + 1], acc[l + 2], acc[l + 3]);
                    r.store(o + l);
                }
            } else {
#pragma unroll
                for (int l = 0; l < L; l++) st_out(o + l, from_float<T>(acc[l]));
            }
        } else if constexpr (G::CLS == CLS_V) {
            // output l sits at row rb*L + l, column j
#pragma unroll
            for (int l = 0; l < L; l++)
                if (H % L == 0 || rb * L + l < H) {
                    if constexpr (TILE)
                        lout[pl * (H * W) + rb * (L * W) + j + l * W] = acc[l];
                    else
                        st_out(obase + (pl * pstride + rb * (L * W) + j) + l * W, from_float<T>(acc[l]));
                }
        } else {
            // output l sits at row rb*L + P0 + l*EH, column j - Q0 + l
#pragma unroll
            for (int l = 0; l < L; l++) {
                const unsigned q = j + (unsigned)(l - G::Q0);  // wraps when negative
                const int doff = (G::P0 + l * G::EH) * W + l - G::Q0;
                if (q < W && (H % L == 0 || rb * L + G::P0 + l * G::EH < H)) {
                    if constexpr (TILE)
                        lout[(int)(pl * (H * W) + rb * (L * W) + j) + doff] = acc[l];
                    else
                        st_out(obase + (pl * pstride + rb * (L * W) + j) + doff, from_float<T>(acc[l]));
                }
            }
        }
    };
    // Two register sets keep two batches in flight from HBM while a third is being computed.
    auto process = [&](auto &stg, int nb) {
        const int nvalid = n1 - nb;
        if constexpr (use_progress_priority<H, W>())
            set_progress_priority((nb - n0) / PB, (n1 - n0 + PB - 1) / PB);
        __syncthreads();  // previous batch fully consumed (first pass: zero fill done)
        wait_vmem_done();
        if constexpr (PAIR)
            stg.template commit_pairs<GeoMap<G>, PLS, G::EH, G::EW>(lds, nvalid);
        else
            stg.template commit<GeoMap<G>, PLS>(lds, nvalid);
        // The previous batch's results leave after the commit: the commit waits for every
        // outstanding global access of the wave, and stores issued just before it would make
        // it wait for their acknowledgement too.
        if constexpr (TILE) {
            if (nb > n0)
                flush_out_tile<T, H, W, PB, NT>(lout, dbase + (size_t)(nb - PB) * pstride, pstride, PB);
        }
        __syncthreads();
        if (nb + 2 * PB < n1) {
            stg.prefetch(sbase + (size_t)(nb + 2 * PB) * pstride, pstride, n1 - nb - 2 * PB);
            if constexpr (BELOW)
                stg.prefetch_below(sbase + (size_t)(nb + 2 * PB) * pstride, pstride, n1 - nb - 2 * PB);
        }
        T *obase = dbase + (size_t)nb * pstride;  // uniform
#pragma unroll
        for (int iter = 0; iter < ITERS; iter++) {
            const unsigned item = tid + iter * NT;
            const unsigned pl = item / G::IPP, it = item % G::IPP;
            const unsigned rb = it / G::IPR, j = it % G::IPR;
            if (item < PB * G::IPP && (int)pl < nvalid) {
                const float *base = lds + (pl * PLS + rb * (G::LR * G::RS) + j);
                float acc[L];
                taps.accumulate(base, acc);
                emit(obase, pl, rb, j, acc);
            }
        }
    };
    int nb = n0;
    for (; nb < n1; nb += 2 * PB) {
        process(sg.a, nb);
        if (nb + PB < n1) process(sg.b, nb + PB);
    }
    if constexpr (TILE) {
        const int last = n0 + ((n1 - n0 - 1) / PB) * PB;  // first image of the final batch
        __syncthreads();
        flush_out_tile<T, H, W, PB, NT>(lout, dbase + (size_t)last * pstride, pstride, n1 - last);
    }
}

// ---------------------------------------------------------------------------------------------
// table-driven body (any angle): same staging with a square halo, taps from the device table
// ---------------------------------------------------------------------------------------------
template <int K, int H, int W>
struct TableMap {
    static constexpr int PAD = table_pad<K, H, W>();
    static constexpr int PL = (PAD + 3) & ~3;
    static constexpr int RS = table_row_stride<K, H, W>();
    static constexpr bool kWide = RS % 4 == 0, kChunked = true;
    static __device__ __forceinline__ unsigned index(unsigned r, unsigned w) {
        return (r + PAD) * RS + w + PL;
    }
    static constexpr int step(int e) { return e; }
};
// In the unrolled table bodies (table_unrolled) a tap's LDS offset (and, for fprop and dgrad,
// weight) is a scalar (TableTaps below), and a thread evaluates table_rows outputs of one
// column, H / table_rows rows apart, so one address per tap serves that many multiply-adds
// while consecutive lanes still read consecutive words.
template <int H, int W>
constexpr int table_rows() {
    // the divisor of H up to 8 that keeps most threads busy (the largest one among equals)
    constexpr int PB = Tile<H, W>::PB, NT = Tile<H, W>::NT;
    int best = 1;
    long num = 0, den = 1;  // busy share of the best so far = num / den
    for (int r = 1; r <= 8; r++) {
        if (H % r != 0) continue;
        const int items = PB * (H / r) * W, slots = (items + NT - 1) / NT * NT;
        if ((long)items * den >= num * slots) best = r, num = items, den = slots;
    }
    return best;
}
// Taps of channel c for the unrolled table bodies: lane s of every wave holds tap s (LDS offset
// and weight bits), and the bodies fetch tap s into scalar registers with a lane read when they
// get to it.  (All K offsets and weights held in scalar registers for the whole body ran out of
// them, and the few the compiler then parks in a vector register cost the canonical bodies
// their last one.)
template <class Map, int K, int H, int W>
struct TableTaps {
    static_assert(K <= 64, "one lane per tap");
    int off, wbits;
    // does tap s of channel c miss an H x W plane altogether?
    static __device__ __forceinline__ bool dead(const int8_t *__restrict__ dhdw, int c, int s) {
        const int dh = dhdw[((size_t)c * K + s) * 2], dw = dhdw[((size_t)c * K + s) * 2 + 1];
        return dh >= H || dh <= -H || dw >= W || dw <= -W;
    }
    // (a tap that misses the plane reads the halo's zeros; its weight is zeroed as well, so that
    // it adds nothing whatever the weight holds)
    __device__ __forceinline__ void load(const int8_t *__restrict__ dhdw, const float *__restrict__ wt,
                                         int c, int sign) {
        const int s = min((int)(threadIdx.x & 63), K - 1);
        const int dh = dhdw[((size_t)c * K + s) * 2], dw = dhdw[((size_t)c * K + s) * 2 + 1];
        off = sign * (dh * Map::RS + dw);
        wbits = wt != nullptr && !dead(dhdw, c, s) ? __builtin_bit_cast(int, wt[(size_t)c * K + s]) : 0;
    }
    // (opaque to the optimiser: called once per batch, so that the lane reads stay inside the
    // batch instead of being hoisted into 2 K scalar registers for the whole loop)
    __device__ __forceinline__ void touch() { asm volatile("" : "+v"(off), "+v"(wbits)); }
    __device__ __forceinline__ int offset(int s) const { return __builtin_amdgcn_readlane(off, s); }
    __device__ __forceinline__ float weight(int s) const {
        return __builtin_bit_cast(float, __builtin_amdgcn_readlane(wbits, s));
    }
};

template <int OP, typename T, int K, int H, int W>
__device__ __forceinline__ void run_table(const T *__restrict__ src, const float *__restrict__ wt,
                                          const float *__restrict__ bias,
                                          const int8_t *__restrict__ dhdw, T *__restrict__ dst,
                                          float *lds, int c, int C, int n0, int n1,
                                          ConvStagers<T, H, W> &sg) {
    constexpr int PB = Tile<H, W>::PB, NT = Tile<H, W>::NT;
    using Map = TableMap<K, H, W>;
    constexpr int PLS = plane_floats<K, H, W>();
    static_assert((H + 2 * Map::PAD) * Map::RS <= PLS, "table body staging must fit the plane stride");
    const unsigned tid = threadIdx.x;
    const unsigned pstride = (unsigned)C * (H * W);
    if constexpr (table_unrolled<K, H, W>()) {
        TableTaps<Map, K, H, W> taps;
        taps.load(dhdw, wt, c, OP == OP_DGRAD ? -1 : 1);
        const float bv = (OP == OP_FPROP && bias != nullptr) ? bias[c] : 0.f;
        lds_zero<NT>(lds, PB * PLS);
        const T *sbase = src + (size_t)c * (H * W);
        T *dbase = dst + (size_t)c * (H * W);
        constexpr int R = table_rows<H, W>(), HR = H / R;
        constexpr int ITEMS = PB * HR * W, ITERS = (ITEMS + NT - 1) / NT;
        auto process = [&](auto &stg, int nb) {
            const int nvalid = n1 - nb;
            taps.touch();
            if constexpr (use_progress_priority<H, W>())
                set_progress_priority((nb - n0) / PB, (n1 - n0 + PB - 1) / PB);
            __syncthreads();
            wait_vmem_done();
            stg.template commit<Map, PLS>(lds, nvalid);
            __syncthreads();
            if (nb + 2 * PB < n1)
                stg.prefetch(sbase + (size_t)(nb + 2 * PB) * pstride, pstride, nvalid - 2 * PB);
            T *obase = dbase + (size_t)nb * pstride;
#pragma unroll
            for (int iter = 0; iter < ITERS; iter++) {
                const unsigned f = tid + iter * NT;
                const unsigned pl = f / (HR * W), g = f % (HR * W);
                if (f < ITEMS && (int)pl < nvalid) {
                    // (opaque: the K addresses base + offset are the same in every batch and
                    // would otherwise be kept in K registers across the batch loop)
                    unsigned at = pl * PLS + Map::index(g / W, g % W);
                    asm volatile("" : "+v"(at));
                    const float *base = lds + at;
                    float acc[R];
#pragma unroll
                    for (int k = 0; k < R; k++) acc[k] = bv;
                    // the reads of tap s + D are issued before the multiply-adds of tap s
                    constexpr int D = R <= 4 ? 2 : 1;
                    float v[D + 1][R];
                    auto read_tap = [&](int s) {
                        const float *q = base + taps.offset(s);
#pragma unroll
                        for (int k = 0; k < R; k++) v[s % (D + 1)][k] = q[k * (HR * Map::RS)];
                    };
#pragma unroll
                    for (int s = 0; s < D && s < K; s++) read_tap(s);
#pragma unroll
                    for (int s = 0; s < K; s++) {
                        if (s + D < K) read_tap(s + D);
                        const float ws = taps.weight(s);
#pragma unroll
                        for (int k = 0; k < R; k++)
                            acc[k] = __builtin_fmaf(v[s % (D + 1)][k], ws, acc[k]);
                    }
                    // (opaque to the optimiser: R store addresses kept as batch-loop invariants
                    // would not fit the register budget next to the canonical bodies')
                    unsigned o = pl * pstride + g;
                    asm volatile("" : "+v"(o));
#pragma unroll
                    for (int k = 0; k < R; k++)
                        st_out(obase + (o + k * (HR * W)), from_float<T>(acc[k]));
                }
            }
        };
        for (int nb = n0; nb < n1; nb += 2 * PB) {
            process(sg.a, nb);
            if (nb + PB < n1) process(sg.b, nb + PB);
        }
        return;
    }
    // live taps of this channel as (LDS offset, weight) pairs (dead taps never reach the plane
    // and are skipped); kept in LDS behind the planes, read as one 8-byte broadcast per tap
    typedef int i2 __attribute__((ext_vector_type(2)));
    int *tapw = reinterpret_cast<int *>(lds + PB * PLS);
    __shared__ int nlive_s;
    if (tid == 0) {
        int nl = 0;
        for (int s = 0; s < K; s++) {
            const int dh = dhdw[((size_t)c * K + s) * 2], dw = dhdw[((size_t)c * K + s) * 2 + 1];
            if (dh >= H || dh <= -H || dw >= W || dw <= -W) continue;
            tapw[2 * nl] = (OP == OP_DGRAD ? -1 : 1) * (dh * Map::RS + dw);
            tapw[2 * nl + 1] = __builtin_bit_cast(int, wt[(size_t)c * K + s]);
            nl++;
        }
        nlive_s = nl;
    }
    const float bv = (OP == OP_FPROP && bias != nullptr) ? bias[c] : 0.f;
    lds_zero<NT>(lds, PB * PLS);
    const T *sbase = src + (size_t)c * (H * W);
    T *dbase = dst + (size_t)c * (H * W);
    // A thread evaluates R outputs of one column, H / R rows apart: one tap read and one address
    // serve R multiply-adds, and consecutive lanes still read consecutive words.
    constexpr int R = H % 4 == 0 ? 4 : (H % 2 == 0 ? 2 : 1), HR = H / R;
    auto process = [&](auto &stg, int nb) {
        const int nvalid = n1 - nb;
        if constexpr (use_progress_priority<H, W>())
            set_progress_priority((nb - n0) / PB, (n1 - n0 + PB - 1) / PB);
        __syncthreads();
        wait_vmem_done();
        stg.template commit<Map, PLS>(lds, nvalid);
        __syncthreads();
        if (nb + 2 * PB < n1)
            stg.prefetch(sbase + (size_t)(nb + 2 * PB) * pstride, pstride, nvalid - 2 * PB);
        const int nlive = nlive_s;
        T *obase = dbase + (size_t)nb * pstride;
        for (unsigned f = tid; f < PB * HR * W; f += NT) {
            const unsigned pl = f / (HR * W), g = f % (HR * W);
            if ((int)pl >= nvalid) break;
            const float *base = lds + pl * PLS + Map::index(g / W, g % W);
            float acc[R];
#pragma unroll
            for (int k = 0; k < R; k++) acc[k] = bv;
            for (int s = 0; s < nlive; s++) {
                const i2 t = *reinterpret_cast<const i2 *>(__builtin_assume_aligned(tapw + 2 * s, 8));
                // (copies first: a bit cast applied to a vector element reads element 0)
                const int off = t[0], wbits = t[1];
                const float *q = base + off;
                const float ws = __builtin_bit_cast(float, wbits);
#pragma unroll
                for (int k = 0; k < R; k++) acc[k] = __builtin_fmaf(q[k * (HR * Map::RS)], ws, acc[k]);
            }
#pragma unroll
            for (int k = 0; k < R; k++)
                st_out(obase + (pl * pstride + g + k * (HR * W)), from_float<T>(acc[k]));
        }
    };
    for (int nb = n0; nb < n1; nb += 2 * PB) {
        process(sg.a, nb);
        if (nb + PB < n1) process(sg.b, nb + PB);
    }
}

// ---------------------------------------------------------------------------------------------
// wgrad: dw[c,s] = sum over n,p,q of x[n,c,p+dh(s),q+dw(s)] * dy[n,c,p,q]
// ---------------------------------------------------------------------------------------------
// Wave64 sum with DPP row shifts and row broadcasts (no LDS traffic); the total lands in lane 63.
__device__ __forceinline__ float wave_sum_dpp(float v) {
#define DWO_DPP_ADD(ctrl, row_mask)                                                              \
    v += __builtin_bit_cast(                                                                     \
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, row_mask, 0xf, true))
    DWO_DPP_ADD(0x111, 0xf);  // row_shr:1
    DWO_DPP_ADD(0x112, 0xf);  // row_shr:2
    DWO_DPP_ADD(0x114, 0xf);  // row_shr:4
    DWO_DPP_ADD(0x118, 0xf);  // row_shr:8  -> lane 15 of each row holds the row total
    DWO_DPP_ADD(0x142, 0xa);  // row_bcast:15 into rows 1 and 3
    DWO_DPP_ADD(0x143, 0xc);  // row_bcast:31 into rows 2 and 3
#undef DWO_DPP_ADD
    return v;
}

// Half-wave sums of up to 32 per-lane values, all at once.  A stage pairs every lane with a
// partner; of two values a lane keeps one and hands the other to its partner, which kept that
// one, so the number of values halves while the number of lanes summed doubles.  After five
// stages (partners 7-i within eight lanes, then i^1, i^2, i^8, i^16) a lane holds the sum over
// the 32 lanes of its half wave of value number reduce32_index(lane): about 100 vector
// instructions for 32 values, where 32 separate wave sums take about 200 and 32 single-lane
// stores.
template <int CTRL>
__device__ __forceinline__ float lane_exchange(float v) {
    if constexpr (CTRL == 0x401F) {  // ds_swizzle, bit-mask mode (and 0x1f, or 0, xor 0x10): lane ^ 16
        return __builtin_bit_cast(float,
                                  __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
    } else {
        return __builtin_bit_cast(
            float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
    }
}
template <int CTRL, int N>
__device__ __forceinline__ void reduce_stage(const float (&in)[2 * N], float (&out)[N], bool sel) {
#pragma unroll
    for (int m = 0; m < N; m++) {
        const float keep = sel ? in[2 * m + 1] : in[2 * m];
        const float send = sel ? in[2 * m] : in[2 * m + 1];
        out[m] = keep + lane_exchange<CTRL>(send);
    }
}
// number of the value whose half-wave sum wave_reduce32 leaves in `lane`, and the lane (of the
// first half wave) that holds value number idx
__device__ __forceinline__ unsigned reduce32_index(unsigned lane) {
    return ((lane >> 2) & 1) | (lane & 1) << 1 | ((lane >> 1) & 1) << 2 | (lane & 0x18);
}
__device__ __forceinline__ unsigned reduce32_lane(unsigned idx) {
    return ((idx >> 1) & 1) | ((idx >> 2) & 1) << 1 | (idx & 1) << 2 | (idx & 0x18);
}
template <int NV>
__device__ __forceinline__ float wave_reduce32(const float (&a)[NV]) {
    static_assert(NV <= 32, "at most 32 values");
    const unsigned lane = threadIdx.x & 63;
    float r32[32], r16[16], r8[8], r4[4], r2[2], r1[1];
#pragma unroll
    for (int s = 0; s < 32; s++) r32[s] = s < NV ? a[s] : 0.f;
    reduce_stage<0x141, 16>(r32, r16, (lane & 4) != 0);  // row_half_mirror
    reduce_stage<0x0B1, 8>(r16, r8, (lane & 1) != 0);    // quad_perm [1,0,3,2]
    reduce_stage<0x04E, 4>(r8, r4, (lane & 2) != 0);     // quad_perm [2,3,0,1]
    reduce_stage<0x128, 2>(r4, r2, (lane & 8) != 0);     // row_ror:8
    reduce_stage<0x401F, 1>(r2, r1, (lane & 16) != 0);   // lane ^ 16
    return r1[0];
}

// Workgroup epilogue: per-thread accumulators acc[0..NV) -> wave totals (DPP) -> LDS -> one
// value per tap handed to WgradOut.  `slot_of(s)` maps tap s to the
// accumulator that holds its sum (-1: the tap never reaches the plane, its gradient is zero).
// Where a workgroup's sums go: one partial per (channel, tap, group) in scratch for the stage-2
// reduction, or, when a channel has a single group, straight into dw / db.
struct WgradOut {
    float *part, *dw, *db;
    int NG;
    unsigned *tickets;  // one zeroed counter per channel block, or null: separate reduction pass
    __device__ __forceinline__ void put(int c, int s, int group, int K, float t) const {
        if (NG > 1 && tickets != nullptr)  // read by another workgroup of this launch: see wgrad_finish
            __hip_atomic_store(part + ((size_t)c * (K + 1) + s) * NG + group, t, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        else if (NG > 1)
            part[((size_t)c * (K + 1) + s) * NG + group] = t;
        else if (s < K)
            dw[(size_t)c * K + s] = t;
        else if (db != nullptr)
            db[c] = t;
    }
};

// The single cross-workgroup reduction, folded into stage 1: the workgroups of a channel block
// (channels [c_first, c_first + nch)) each take a ticket after their partials are visible
// device-wide; the one that draws the last ticket adds the NG partials of every (channel, tap)
// in index order -- the same fixed order whichever workgroup happens to be last, so the result
// is bit-reproducible -- writes dw / db and puts the counter back to zero for the next launch.
// All threads of the workgroup call this (it contains barriers).
template <int K>
__device__ __forceinline__ void wgrad_finish(const WgradOut &out, float *lds, int ticket,
                                             int c_first, int nch) {
    if (out.NG <= 1 || out.tickets == nullptr) return;  // uniform
    // Partial sums are written and read with device-scope (cache-bypassing) accesses and the
    // ticket is a device-scope atomic, all relaxed: a fence pair at device scope would write
    // back and invalidate the XCD's whole L2 once per workgroup (measured: +20 to +70 % kernel
    // time).  Order is kept by completion instead: every thread waits until its stores are
    // acknowledged before the barrier that precedes the ticket, and the last workgroup's loads
    // are issued only after its ticket value has come back.
    // (That argument rests on how gfx942 / gfx950 complete device-scope accesses -- stores
    // written through and counted by vmcnt, loads served past the L2 of another XCD.  Any other
    // target takes the ticket with release-acquire ordering, which the memory model itself
    // guarantees.)
#if defined(__gfx942__) || defined(__gfx950__)
    constexpr int kTicketOrder = __ATOMIC_RELAXED;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#else
    constexpr int kTicketOrder = __ATOMIC_ACQ_REL;
#endif
    __syncthreads();
    unsigned *flag = reinterpret_cast<unsigned *>(lds);
    if (threadIdx.x == 0)
        *flag = __hip_atomic_fetch_add(out.tickets + ticket, 1u, kTicketOrder,
                                       __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*flag != (unsigned)out.NG - 1) return;
    const int NG = out.NG;
    for (int i = threadIdx.x; i < nch * (K + 1); i += blockDim.x) {
        const int c = c_first + i / (K + 1), s = i % (K + 1);
        if (s == K && out.db == nullptr) continue;
        // (device-scope loads: the other workgroups ran on other XCDs, behind other L2s)
        const float *p = out.part + ((size_t)c * (K + 1) + s) * NG;
        auto ld = [&](int g) {
            return __hip_atomic_load(p + g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        };
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        int g = 0;
        for (; g + 4 <= NG; g += 4) a0 += ld(g), a1 += ld(g + 1), a2 += ld(g + 2), a3 += ld(g + 3);
        for (; g < NG; g++) a0 += ld(g);
        const float total = (a0 + a1) + (a2 + a3);
        if (s == K)
            out.db[c] = total;
        else
            out.dw[(size_t)c * K + s] = total;
    }
    if (threadIdx.x == 0)
        __hip_atomic_store(out.tickets + ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int K, int NT, class SlotOf>
__device__ __forceinline__ void wgrad_epilogue(float (&acc)[K + 1], float *lds, const WgradOut &out,
                                               int c, int group, SlotOf slot_of) {
    constexpr int NW = NT / 64;
    __syncthreads();  // staged planes are dead from here on
    // every lane leaves the half-wave sum of one accumulator in its wave's row of 64 words
    lds[threadIdx.x] = wave_reduce32(acc);
    __syncthreads();
    if (threadIdx.x <= K) {
        const int slot = threadIdx.x == K ? K : slot_of(threadIdx.x);
        float t = 0.f;
        if (slot >= 0) {
            const unsigned l = reduce32_lane(slot);
            for (int w = 0; w < NW; w++) t += lds[w * 64 + l] + lds[w * 64 + 32 + l];
        }
        out.put(c, threadIdx.x, group, K, t);
    }
    wgrad_finish<K>(out, lds, c, c, 1);
}

// dy planes are staged without a halo right behind the x planes and the tap tables, rows DRS
// words apart.  An item reads the dy of its L outputs; for the stacked and diagonal classes
// that is one word per lane and row, lanes along j, and DRS is chosen like the x rows' stride so
// that stepping to the next row-block continues the same line modulo the 32 banks.  The
// row-direction classes read their L adjacent outputs as one wide word: rows stay W apart.
template <int W, int DRS>
struct DyMap {
    static constexpr bool kWide = DRS % 4 == 0, kChunked = true;
    static __device__ __forceinline__ unsigned index(unsigned r, unsigned w) { return r * DRS + w; }
    static constexpr int step(int e) { return e; }
};
template <class G, int W>
constexpr int dy_row_stride() {
    return G::CLS == CLS_H ? W : bank_stride(W, G::LR, G::IPR);
}
template <int K, int H, int W, int... Os>
constexpr int max_dy_plane(std::integer_sequence<int, Os...>) {
    int m = H * W;  // table-driven body and row-direction classes
    ((m = cmax(m, H * dy_row_stride<Geo<Os, K, wgrad_L<H, W>(Os), H, W>, W>())), ...);
    return (m + 3) & ~3;
}
template <int K, int H, int W>
constexpr int wgrad_dy_plane() {
    return max_dy_plane<K, H, W>(std::make_integer_sequence<int, 8>{});
}
template <int K, int H, int W>
constexpr int wgrad_dy_offset() {
    return (Tile<H, W>::PB * plane_floats<K, H, W>() + 2 * K + 3) & ~3;
}

template <int O, typename T, int K, int H, int W>
__device__ __forceinline__ void run_canonical_wgrad(const T *__restrict__ x, const T *__restrict__ dy,
                                                    const WgradOut &out, float *lds, int c,
                                                    int C, int n0, int n1, int group) {
    constexpr int L = wgrad_L<H, W>(O);
    constexpr int PB = Tile<H, W>::PB, NT = Tile<H, W>::NT;
    using G = Geo<O, K, L, H, W>;
    constexpr int PLS = plane_floats<K, H, W>();
    static_assert(G::PLANE <= PLS, "wgrad geometry must fit the plane stride");
    constexpr int ITERS = (PB * G::IPP + NT - 1) / NT;
    const unsigned tid = threadIdx.x;
    const unsigned pstride = (unsigned)C * (H * W);
    const T *xbase = x + (size_t)c * (H * W);
    const T *gbase = dy + (size_t)c * (H * W);
    float *ldy = lds + wgrad_dy_offset<K, H, W>();
    constexpr int DRS = dy_row_stride<G, W>(), DYP = wgrad_dy_plane<K, H, W>();

    // DEPTH register sets per tensor keep that many batches in flight while another is summed.
    constexpr int DEPTH = H * W <= 256 ? DWO_WGRAD_DEPTH_SMALL : DWO_WGRAD_DEPTH;
    Stager<T, H, W, PB, NT> sx[DEPTH], sg[DEPTH];
#pragma unroll
    for (int k = 0; k < DEPTH; k++)
        if (n0 + k * PB < n1) {
            sx[k].prefetch(xbase + (size_t)(n0 + k * PB) * pstride, pstride, n1 - n0 - k * PB);
            sg[k].prefetch(gbase + (size_t)(n0 + k * PB) * pstride, pstride, n1 - n0 - k * PB);
        }
    // (after the first loads are on their way: the zero fill runs under their latency)
    lds_zero<NT>(lds, PB * PLS);

    float acc[K + 1];  // acc[s] for representative taps s, acc[K] = sum of dy (bias gradient)
#pragma unroll
    for (int s = 0; s <= K; s++) acc[s] = 0.f;
    auto process = [&](auto &stx, auto &stg, int nb) {
        const int nvalid = n1 - nb;
        if constexpr (use_progress_priority<H, W>())
            set_progress_priority((nb - n0) / PB, (n1 - n0 + PB - 1) / PB);
        __syncthreads();
        wait_vmem_done();
        stx.template commit<GeoMap<G>, PLS>(lds, nvalid);
        stg.template commit<DyMap<W, DRS>, DYP>(ldy, nvalid);
        __syncthreads();
        if (nb + DEPTH * PB < n1) {
            stx.prefetch(xbase + (size_t)(nb + DEPTH * PB) * pstride, pstride, nvalid - DEPTH * PB);
            stg.prefetch(gbase + (size_t)(nb + DEPTH * PB) * pstride, pstride, nvalid - DEPTH * PB);
        }
#pragma unroll
        for (int it = 0; it < ITERS; it++) {
            const unsigned item = tid + it * NT;
            const unsigned pl = item / G::IPP, ii = item % G::IPP;
            const unsigned rb = ii / G::IPR, j = ii % G::IPR;
            if (item < PB * G::IPP && (int)pl < nvalid) {
                // dy of the item's L outputs (zero where the output does not exist)
                float d[L];
                const float *g = ldy + pl * DYP;
                if constexpr (G::CLS == CLS_H) {
                    // one wide read: L separate reads at a lane stride of L words conflict L ways
                    if constexpr (L == 4 && W % 4 == 0 && (H * W) % 4 == 0) {
                        const lds_f4 dv = lds_read4(g + rb * W + j * 4);
                        d[0] = dv[0], d[1] = dv[1], d[2] = dv[2], d[3] = dv[3];
                    } else if constexpr (L == 2 && W % 2 == 0 && (H * W) % 2 == 0) {
                        const lds_f2 dv = lds_read2(g + rb * W + j * 2);
                        d[0] = dv[0], d[1] = dv[1];
                    } else {
#pragma unroll
                        for (int l = 0; l < L; l++) d[l] = g[rb * W + j * L + l];
                    }
                } else if constexpr (G::CLS == CLS_V) {
#pragma unroll
                    for (int l = 0; l < L; l++)
                        d[l] = (H % L == 0 || rb * L + l < H) ? g[(rb * L + l) * DRS + j] : 0.f;
                } else {
#pragma unroll
                    for (int l = 0; l < L; l++) {
                        const unsigned q = j + (unsigned)(l - G::Q0);
                        const bool ok = q < W && (H % L == 0 || rb * L + G::P0 + l * G::EH < H);
                        d[l] = ok ? g[(int)(rb * (L * DRS) + j) + (G::P0 + l * G::EH) * DRS + l - G::Q0] : 0.f;
                    }
                }
                const float *base = lds + (pl * PLS + rb * (G::LR * G::RS) + j);
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
    };
    for (int nb = n0; nb < n1; nb += DEPTH * PB) {
        static_for<DEPTH>([&](auto k) {
            if (nb + k * PB < n1) process(sx[k], sg[k], nb + k * PB);
        });
    }
    wgrad_epilogue<K, NT>(acc, lds, out, c, group, [](int s) { return (int)G::plan.rep[s]; });
}

// table-driven wgrad body (any angle)
template <typename T, int K, int H, int W>
__device__ __forceinline__ void run_table_wgrad(const T *__restrict__ x, const T *__restrict__ dy,
                                                const int8_t *__restrict__ dhdw,
                                                const WgradOut &out, float *lds, int c, int C,
                                                int n0, int n1, int group) {
    constexpr int PB = Tile<H, W>::PB, NT = Tile<H, W>::NT;
    using Map = TableMap<K, H, W>;
    constexpr int PLS = plane_floats<K, H, W>();
    const unsigned tid = threadIdx.x;
    const unsigned pstride = (unsigned)C * (H * W);
    if constexpr (table_unrolled<K, H, W>()) {
        TableTaps<Map, K, H, W> taps;
        taps.load(dhdw, nullptr, c, 1);
        lds_zero<NT>(lds, PB * PLS);
        float acc[K + 1];
#pragma unroll
        for (int s = 0; s <= K; s++) acc[s] = 0.f;
        const T *xbase = x + (size_t)c * (H * W);
        const T *gbase = dy + (size_t)c * (H * W);
        constexpr int R = table_rows<H, W>(), HR = H / R;
        constexpr int ITEMS = PB * HR * W, ITERS = (ITEMS + NT - 1) / NT;
        Stager<T, H, W, PB, NT> st;
        st.prefetch(xbase + (size_t)n0 * pstride, pstride, n1 - n0);
        // dy of a batch goes straight from HBM to the registers of the lanes that use it, issued
        // before the batch's x planes are written to LDS (a batch ahead, as for x, they would not
        // fit next to the K + 1 sums)
        for (int nb = n0; nb < n1; nb += PB) {
            const int nvalid = n1 - nb;
            taps.touch();
            if constexpr (use_progress_priority<H, W>())
                set_progress_priority((nb - n0) / PB, (n1 - n0 + PB - 1) / PB);
            __syncthreads();
            wait_vmem_done();
            const T *gb = gbase + (size_t)nb * pstride;
            T gy[ITERS][R];
#pragma unroll
            for (int iter = 0; iter < ITERS; iter++) {
                const unsigned f = tid + iter * NT;
                const unsigned pl = f / (HR * W), g = f % (HR * W);
                const bool on = f < ITEMS && (int)pl < nvalid;
                unsigned o = pl * pstride + g;  // (opaque: see the stores of run_table)
                asm volatile("" : "+v"(o));
#pragma unroll
                for (int k = 0; k < R; k++)
                    gy[iter][k] = on ? gb[o + k * (HR * W)] : from_float<T>(0.f);
            }
            st.template commit<Map, PLS>(lds, nvalid);
            __syncthreads();
            if (nb + PB < n1) st.prefetch(xbase + (size_t)(nb + PB) * pstride, pstride, nvalid - PB);
#pragma unroll
            for (int iter = 0; iter < ITERS; iter++) {
                const unsigned f = tid + iter * NT;
                const unsigned pl = f / (HR * W), g = f % (HR * W);
                if (f < ITEMS && (int)pl < nvalid) {
                    unsigned at = pl * PLS + Map::index(g / W, g % W);
                    asm volatile("" : "+v"(at));  // (opaque: see run_table)
                    const float *base = lds + at;
                    float gf[R];
#pragma unroll
                    for (int k = 0; k < R; k++) gf[k] = to_float(gy[iter][k]);
                    // the reads of tap s + D are issued before the multiply-adds of tap s
                    constexpr int D = R <= 4 ? 2 : 1;
                    float v[D + 1][R];
                    auto read_tap = [&](int s) {
                        const float *q = base + taps.offset(s);
#pragma unroll
                        for (int k = 0; k < R; k++) v[s % (D + 1)][k] = q[k * (HR * Map::RS)];
                    };
#pragma unroll
                    for (int s = 0; s < D && s < K; s++) read_tap(s);
#pragma unroll
                    for (int s = 0; s < K; s++) {
                        if (s + D < K) read_tap(s + D);
#pragma unroll
                        for (int k = 0; k < R; k++)
                            acc[s] = __builtin_fmaf(v[s % (D + 1)][k], gf[k], acc[s]);
                    }
#pragma unroll
                    for (int k = 0; k < R; k++) acc[K] += gf[k];
                }
            }
        }
        // (taps that miss the plane have summed halo zeros times dy: their gradient is zero by
        // definition, whatever dy holds)
        wgrad_epilogue<K, NT>(acc, lds, out, c, group, [&](int s) {
            return TableTaps<Map, K, H, W>::dead(dhdw, c, s) ? -1 : s;
        });
        return;
    }
    int *toff = reinterpret_cast<int *>(lds + PB * PLS);  // LDS offset per tap; dead taps read the
    int *tlive = toff + K;                                 // centre and are zeroed at the end
    if (tid < K) {
        const int dh = dhdw[((size_t)c * K + tid) * 2], dw = dhdw[((size_t)c * K + tid) * 2 + 1];
        const bool dead = dh >= H || dh <= -H || dw >= W || dw <= -W;
        toff[tid] = dead ? 0 : dh * Map::RS + dw;
        tlive[tid] = dead ? -1 : (int)tid;
    }
    lds_zero<NT>(lds, PB * PLS);
    float acc[K + 1];
#pragma unroll
    for (int s = 0; s <= K; s++) acc[s] = 0.f;
    const T *xbase = x + (size_t)c * (H * W);
    const T *gbase = dy + (size_t)c * (H * W);
    Stager<T, H, W, PB, NT> st;
    st.prefetch(xbase + (size_t)n0 * pstride, pstride, n1 - n0);
    for (int nb = n0; nb < n1; nb += PB) {
        const int nvalid = n1 - nb;
        if constexpr (use_progress_priority<H, W>())
            set_progress_priority((nb - n0) / PB, (n1 - n0 + PB - 1) / PB);
        __syncthreads();
        wait_vmem_done();
        st.template commit<Map, PLS>(lds, nvalid);
        __syncthreads();
        if (nb + PB < n1) st.prefetch(xbase + (size_t)(nb + PB) * pstride, pstride, nvalid - PB);
        const T *gb = gbase + (size_t)nb * pstride;
        for (unsigned f = tid; f < PB * H * W; f += NT) {
            const unsigned pl = f / (H * W), g = f % (H * W);
            if ((int)pl >= nvalid) break;
            const float gy = to_float(gb[pl * pstride + g]);
            const float *base = lds + pl * PLS + Map::index(g / W, g % W);
#pragma unroll
            // (offsets are re-read from LDS per tap: keeping all K of them in registers next to
            // the K accumulators would cost occupancy for every channel, canonical ones included)
            for (int s = 0; s < K; s++)
                acc[s] = __builtin_fmaf(base[*(volatile int *)&toff[s]], gy, acc[s]);
            acc[K] += gy;
        }
    }
    wgrad_epilogue<K, NT>(acc, lds, out, c, group, [&](int s) { return tlive[s]; });
}

template <typename T, int K, int H, int W>
__global__ __launch_bounds__((Tile<H, W>::NT)) __attribute__((amdgpu_waves_per_eu(DWO_WPE_WGRAD, 8))) void plane_wgrad_kernel(
    const T *__restrict__ x, const T *__restrict__ dy, const void *__restrict__ blob,
    WgradOut out, int N, int C, int cus) {
    extern __shared__ __align__(16) float lds[];
    const int NG = out.NG;
    int c, group;
    if (!wgrad_task(blob, C, K, NG, cus, c, group)) return;
    int n0, n1;
    group_range<Tile<H, W>::PB>(N, NG, group, n0, n1);
    const int cls = taps_class(blob, C, K)[c];
#define DWO_CASE(O)                                                                      \
    case O:                                                                              \
        run_canonical_wgrad<O, T, K, H, W>(x, dy, out, lds, c, C, n0, n1, group);         \
        break;
    switch (cls) {
        DWO_CASE(0)
        DWO_CASE(1)
        DWO_CASE(2)
        DWO_CASE(3)
        DWO_CASE(4)
        DWO_CASE(5)
        DWO_CASE(6)
        DWO_CASE(7)
        default:
            run_table_wgrad<T, K, H, W>(x, dy, taps_dhdw(blob), out, lds, c, C, n0, n1, group);
    }
#undef DWO_CASE
}

// LDS bytes a launch of plane_kernel / plane_wgrad_kernel<.., K, H, W> needs
template <typename T, int K, int H, int W>
constexpr size_t plane_kernel_lds_bytes() {
    return ((size_t)out_tile_offset<K, H, W>() +
            (use_out_tile<T, H, W>() ? Tile<H, W>::PB * H * W : 0)) * sizeof(float);
}
template <int K, int H, int W>
constexpr size_t plane_wgrad_lds_bytes() {
    return ((size_t)wgrad_dy_offset<K, H, W>() + Tile<H, W>::PB * wgrad_dy_plane<K, H, W>()) * sizeof(float);
}

template <int OP, typename T, int K, int H, int W>
__global__ __launch_bounds__((Tile<H, W>::NT)) __attribute__((amdgpu_waves_per_eu(DWO_WPE, 8))) void plane_kernel(
    const T *__restrict__ src, const float *__restrict__ wt, const float *__restrict__ bias,
    const void *__restrict__ blob, T *__restrict__ dst, int N, int C, int groups) {
    extern __shared__ __align__(16) float lds[];
    int c, group;
    plane_task(blob, C, K, groups, c, group);
    int n0, n1;
    group_range<Tile<H, W>::PB>(N, groups, group, n0, n1);
    ConvStagers<T, H, W> sg;
    sg.start(src, c, C, n0, n1);  // HBM latency overlaps the class lookup, weights and zero fill
    const int cls = taps_class(blob, C, K)[c];
#define DWO_CASE(O)                                                                  \
    case O:                                                                          \
        run_canonical<O, OP, T, K, H, W>(src, wt, bias, dst, lds, c, C, n0, n1, sg);  \
        break;
    switch (cls) {
        DWO_CASE(0)
        DWO_CASE(1)
        DWO_CASE(2)
        DWO_CASE(3)
        DWO_CASE(4)
        DWO_CASE(5)
        DWO_CASE(6)
        DWO_CASE(7)
        default:
            run_table<OP, T, K, H, W>(src, wt, bias, taps_dhdw(blob), dst, lds, c, C, n0, n1, sg);
    }
#undef DWO_CASE
}

// ---------------------------------------------------------------------------------------------
// host launchers (instantiated per element type and plane extent in dwo_inst.hip)
// ---------------------------------------------------------------------------------------------
// Workgroups that can be resident at once on the current device for a kernel, and the device's
// CU count, packed as slots | cus << 16.
template <class Kern>
int resident_slots(Kern kern, int block, size_t lds) {
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, block, lds) != hipSuccess ||
        cus < 1 || per_cu < 1 || cus > 4096 || cus * per_cu > 65535)
        return 1024 | (256 << 16);
    return (cus * per_cu) | (cus << 16);
}
// grid of C * groups tasks, padded to a multiple of the CU count once it exceeds it (wgrad_task)
inline unsigned plane_grid(int C, int groups, int cus) {
    const long total = (long)C * groups;
    return (unsigned)(total > cus ? (total + cus - 1) / cus * cus : total);
}

// register-plane kernels (dwo_regplane.h) take fprop and dgrad of planes of at most 16 x 16
template <typename T, int K, int H, int W>
int launch_regplane_conv(int op, const void *src, const float *w, const float *bias,
                         const void *taps, void *dst, int N, int C, hipStream_t st);
template <typename T, int K, int H, int W>
int launch_plane_conv(int op, const void *src, const float *w, const float *bias, const void *taps,
                      void *dst, int N, int C, hipStream_t st) {
    if constexpr (reg_plane_shape<H, W>()) {
        return launch_regplane_conv<T, K, H, W>(op, src, w, bias, taps, dst, N, C, st);
    } else {
    constexpr int NT = Tile<H, W>::NT;
    const size_t lds = plane_kernel_lds_bytes<T, K, H, W>();
    static int cache[kMaxDevices];
    const int packed = per_device_once(
        cache, [&] { return resident_slots(plane_kernel<OP_FPROP, T, K, H, W>, NT, lds); });
    if (N == 0) return 0;  // set-up only
    const int slots_f = packed & 0xffff;
    const int groups = plane_groups(N, C, Tile<H, W>::PB, slots_f);
    const dim3 grid(C * groups), block(NT);
    if (op == OP_FPROP)
        plane_kernel<OP_FPROP, T, K, H, W><<<grid, block, lds, st>>>((const T *)src, w, bias, taps,
                                                                   (T *)dst, N, C, groups);
    else
        plane_kernel<OP_DGRAD, T, K, H, W><<<grid, block, lds, st>>>((const T *)src, w, bias, taps,
                                                                   (T *)dst, N, C, groups);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
    }
}

// Writes NG = *groups_out partials per (channel, tap) into part[(c*(K+1)+s)*NG + g]; with
// NG = 1 the sums go straight to dw / db (db may be null) and no reduction is needed, and with
// `tickets` (C zeroed counters) the last workgroup of each channel reduces them itself.
template <typename T, int K, int H, int W>
int launch_plane_wgrad(const void *x, const void *dy, const void *taps, float *part, float *dw,
                       float *db, unsigned *tickets, int N, int C, int *groups_out, hipStream_t st) {
    constexpr int NT = Tile<H, W>::NT;
    const size_t lds = plane_wgrad_lds_bytes<K, H, W>();
    static int cache[kMaxDevices];
    const int packed = per_device_once(
        cache, [&] { return resident_slots(plane_wgrad_kernel<T, K, H, W>, NT, lds); });
    if (N == 0) return 0;  // set-up only
    const int slots = packed & 0xffff, cus = packed >> 16;
    const int groups = plane_groups(N, C, Tile<H, W>::PB, slots);
    *groups_out = groups;
    plane_wgrad_kernel<T, K, H, W><<<dim3(plane_grid(C, groups, cus)), dim3(NT), lds, st>>>(
        (const T *)x, (const T *)dy, taps, WgradOut{part, dw, db, groups, tickets}, N, C, cus);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

}  // namespace dwo

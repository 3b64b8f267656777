// LDS-staged NCHW kernels for stride 1 with compile-time plane extents.
//
// Workgroup (c, group): channel c, a run of G consecutive images.  PB planes (n, c) are staged
// at a time into LDS with a zero halo (zeroed once: only plane interiors are rewritten), so no
// tap needs a bounds test.  While a batch is being computed the next batch is already in
// flight from HBM into registers.  Channels whose taps match one of the eight canonical
// orientations run the straight-line body generated from dwo_plan.h; any other channel takes
// the table-driven body at the bottom (same staging, dynamic taps).
#pragma once

#include "dwo_common.h"
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

enum { OP_FPROP = 0, OP_DGRAD = 1 };

// Four consecutive activations of type T as floats (one 16-byte or 8-byte global access).
template <typename T>
struct Vec4;
template <>
struct Vec4<float> {
    float4 v;
    __device__ __forceinline__ void load(const float *p) { v = *reinterpret_cast<const float4 *>(p); }
    __device__ __forceinline__ void store(float *p) const { *reinterpret_cast<float4 *>(p) = v; }
    __device__ __forceinline__ float get(int i) const { return i == 0 ? v.x : (i == 1 ? v.y : (i == 2 ? v.z : v.w)); }
    __device__ __forceinline__ void set(float a, float b, float c, float d) { v = make_float4(a, b, c, d); }
};
template <>
struct Vec4<bf16_t> {
    uint2 v;
    __device__ __forceinline__ void load(const bf16_t *p) { v = *reinterpret_cast<const uint2 *>(p); }
    __device__ __forceinline__ void store(bf16_t *p) const { *reinterpret_cast<uint2 *>(p) = v; }
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = i < 2 ? v.x : v.y;
        return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    __device__ __forceinline__ void set(float a, float b, float c, float d) {
        v.x = (uint32_t)from_float<bf16_t>(a).bits | ((uint32_t)from_float<bf16_t>(b).bits << 16);
        v.y = (uint32_t)from_float<bf16_t>(c).bits | ((uint32_t)from_float<bf16_t>(d).bits << 16);
    }
};
template <>
struct Vec4<f16_t> {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    h4 v;
    __device__ __forceinline__ void load(const f16_t *p) { v = *reinterpret_cast<const h4 *>(p); }
    __device__ __forceinline__ void store(f16_t *p) const { *reinterpret_cast<h4 *>(p) = v; }
    __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
    __device__ __forceinline__ void set(float a, float b, float c, float d) {
        v[0] = (_Float16)a, v[1] = (_Float16)b, v[2] = (_Float16)c, v[3] = (_Float16)d;
    }
};

// Work decomposition per plane extent: outputs per lane (L) for each orientation class, planes
// staged per batch (PB) and threads per workgroup (NT), chosen so that one batch yields close
// to NT items for every class (items per plane: H class H*W/LH, V class ceil(H/LV)*W, D class
// ceil(H/LD)*round_up(W+LD-1, 8)).
template <int H, int W>
struct Tile {
    static constexpr int LH = W % 4 == 0 ? 4 : (W % 2 == 0 ? 2 : 1);
    static constexpr int LV = LH, LD = LH;
    static constexpr int PB = 1, NT = 256;
};
template <>
struct Tile<56, 56> {  // 784 / 448 / 448 items per plane
    static constexpr int LH = 4, LV = 7, LD = 8, PB = 1, NT = 448;
};
template <>
struct Tile<28, 28> {  // 196 / 196 / 224
    static constexpr int LH = 4, LV = 4, LD = 4, PB = 2, NT = 448;
};
template <>
struct Tile<14, 14> {  // 98 / 98 / 112
    static constexpr int LH = 2, LV = 2, LD = 2, PB = 4, NT = 448;
};
template <>
struct Tile<7, 7> {  // 49 / 49 / 56
    static constexpr int LH = 1, LV = 1, LD = 1, PB = 8, NT = 448;
};
template <int H, int W>
constexpr int tile_L(int o) {
    return orient_class(o) == CLS_H ? Tile<H, W>::LH
                                    : (orient_class(o) == CLS_V ? Tile<H, W>::LV : Tile<H, W>::LD);
}

// halo of the table-driven body: no live tap reaches further than this
template <int K, int H, int W>
constexpr int table_pad() {
    return K / 2 < cmax(H, W) - 1 ? K / 2 : cmax(H, W) - 1;
}

template <int K, int H, int W, int... Os>
constexpr int max_plane_floats(std::integer_sequence<int, Os...>) {
    constexpr int PAD = table_pad<K, H, W>();
    int m = (H + 2 * PAD) * (W + 2 * PAD + 3);  // table-driven body
    ((m = cmax(m, Geo<Os, K, tile_L<H, W>(Os), H, W>::PLANE)), ...);
    return m;
}
template <int K, int H, int W>
constexpr int plane_floats() {
    return max_plane_floats<K, H, W>(std::make_integer_sequence<int, 8>{});
}

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
};

// Staging of PB planes (n, c), n = nb .. nb+PB-1, through registers into LDS.  `Map` gives the
// LDS index of interior element (r, w) relative to the plane's LDS origin.
template <typename T, int H, int W, int PB, int NT, int PLS, class Map>
struct Stager {
    static constexpr int VL = (H * W) % 4 == 0 ? 4 : 1;
    static constexpr int FP = H * W / VL;              // chunks per plane
    static constexpr int PF = (PB * FP + NT - 1) / NT; // chunks per thread
    Chunk<T, VL> pre[PF];

    __device__ __forceinline__ void prefetch(const T *__restrict__ src, int c, int C, int nb, int n1) {
#pragma unroll
        for (int k = 0; k < PF; k++) {
            const int f = threadIdx.x + k * NT;
            const int pl = f / FP, g = f % FP;
            if (f < PB * FP && nb + pl < n1)
                pre[k].load(src + ((size_t)(nb + pl) * C + c) * (H * W) + g * VL);
        }
    }
    __device__ __forceinline__ void commit(float *lds, int nb, int n1) const {
#pragma unroll
        for (int k = 0; k < PF; k++) {
            const int f = threadIdx.x + k * NT;
            const int pl = f / FP, g = f % FP;
            if (f < PB * FP && nb + pl < n1) {
                float *plane = lds + pl * PLS;
                if constexpr (W % VL == 0) {
                    const int r = g / (W / VL), w0 = (g % (W / VL)) * VL;
#pragma unroll
                    for (int e = 0; e < VL; e++) plane[Map::index(r, w0 + e)] = pre[k].get(e);
                } else {
#pragma unroll
                    for (int e = 0; e < VL; e++) {
                        const int i = g * VL + e;
                        plane[Map::index(i / W, i % W)] = pre[k].get(e);
                    }
                }
            }
        }
    }
};

// ---------------------------------------------------------------------------------------------
// canonical body
// ---------------------------------------------------------------------------------------------
template <int O, int OP, typename T, int K, int H, int W>
__device__ __forceinline__ void run_canonical(const T *__restrict__ src, const float *__restrict__ wt,
                                              const float *__restrict__ bias, T *__restrict__ dst,
                                              float *lds, int c, int C, int n0, int n1) {
    constexpr int L = tile_L<H, W>(O);
    constexpr int PB = Tile<H, W>::PB, NT = Tile<H, W>::NT;
    using G = Geo<O, K, L, H, W>;
    constexpr int PLS = plane_floats<K, H, W>();  // LDS plane stride (same for all orientations)
    struct Map {
        static __device__ __forceinline__ int index(int r, int w) {
            return G::interior_row(r) + G::col(w + G::PL);
        }
    };
    const int tid = threadIdx.x;

    // weights of this channel, duplicates folded into their representative tap
    float wv[K];
    const float *wc = wt + (size_t)c * K;
#pragma unroll
    for (int s = 0; s < K; s++) wv[s] = wc[OP == OP_DGRAD ? K - 1 - s : s];
    static_for<K>([&](auto s) {
        constexpr int r = G::plan.rep[s];
        if constexpr (r >= 0 && r != s) wv[r] += wv[s];
    });
    const float bv = (OP == OP_FPROP && bias != nullptr) ? bias[c] : 0.f;

    // zero the staging area once; interiors are overwritten per batch, halos stay zero
    for (int i = tid; i < PB * PLS; i += NT) lds[i] = 0.f;

    Stager<T, H, W, PB, NT, PLS, Map> st;
    st.prefetch(src, c, C, n0, n1);
    for (int nb = n0; nb < n1; nb += PB) {
        __syncthreads();  // previous batch fully consumed (first pass: zero fill done)
        st.commit(lds, nb, n1);
        __syncthreads();
        if (nb + PB < n1) st.prefetch(src, c, C, nb + PB, n1);

        for (int item = tid; item < PB * G::IPP; item += NT) {
            const int pl = item / G::IPP, it = item % G::IPP;
            const int rb = it / G::IPR, j = it % G::IPR;
            if (nb + pl >= n1) break;
            const float *base = lds + pl * PLS + rb * (G::LR * G::RS) + j;
            float acc[L];
#pragma unroll
            for (int l = 0; l < L; l++) acc[l] = bv;
            static_for<G::plan.nsrc>([&](auto m) {
                constexpr int off = G::imm(G::plan.sh[m], G::plan.sw[m]);
                const float v = base[off];
                static_for<L>([&](auto l) {
                    constexpr int t = G::plan.user[m][l];
                    if constexpr (t >= 0) acc[l] = __builtin_fmaf(v, wv[t], acc[l]);
                });
            });
            T *out = dst + ((size_t)(nb + pl) * C + c) * (H * W);
            if constexpr (G::CLS == CLS_H) {
                T *o = out + rb * W + j * L;
                if constexpr (L == 4) {
                    Vec4<T> r;
                    r.set(acc[0], acc[1], acc[2], acc[3]);
                    r.store(o);
                } else {
#pragma unroll
                    for (int l = 0; l < L; l++) o[l] = from_float<T>(acc[l]);
                }
            } else if constexpr (G::CLS == CLS_V) {
#pragma unroll
                for (int l = 0; l < L; l++)
                    if (H % L == 0 || rb * L + l < H) out[(rb * L + l) * W + j] = from_float<T>(acc[l]);
            } else {
                const int p0 = rb * L + G::P0, q0 = j - G::Q0;
#pragma unroll
                for (int l = 0; l < L; l++) {
                    const int p = p0 + l * G::EH, q = q0 + l;
                    if (q >= 0 && q < W && (H % L == 0 || p < H)) out[p * W + q] = from_float<T>(acc[l]);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// table-driven body (any angle): same staging with a square halo, taps from the device table
// ---------------------------------------------------------------------------------------------
template <int OP, typename T, int K, int H, int W>
__device__ __forceinline__ void run_table(const T *__restrict__ src, const float *__restrict__ wt,
                                          const float *__restrict__ bias,
                                          const int8_t *__restrict__ dhdw, T *__restrict__ dst,
                                          float *lds, int c, int C, int n0, int n1) {
    constexpr int PB = Tile<H, W>::PB, NT = Tile<H, W>::NT;
    constexpr int PAD = table_pad<K, H, W>();
    constexpr int PL = (PAD + 3) & ~3;
    constexpr int RS = W + PL + PAD;
    constexpr int PLS = plane_floats<K, H, W>();
    static_assert((H + 2 * PAD) * RS <= PLS, "table body staging must fit the plane stride");
    struct Map {
        static __device__ __forceinline__ int index(int r, int w) { return (r + PAD) * RS + w + PL; }
    };
    const int tid = threadIdx.x;
    // live taps of this channel as LDS offsets, with their weights (dead taps never reach the
    // plane and are skipped); kept in LDS behind the planes
    int *toff = reinterpret_cast<int *>(lds + PB * PLS);
    float *twt = lds + PB * PLS + K;
    __shared__ int nlive_s;
    if (tid == 0) {
        int nl = 0;
        for (int s = 0; s < K; s++) {
            const int dh = dhdw[((size_t)c * K + s) * 2], dw = dhdw[((size_t)c * K + s) * 2 + 1];
            if (dh >= H || dh <= -H || dw >= W || dw <= -W) continue;
            toff[nl] = (OP == OP_DGRAD ? -1 : 1) * (dh * RS + dw);
            twt[nl] = wt[(size_t)c * K + s];
            nl++;
        }
        nlive_s = nl;
    }
    const float bv = (OP == OP_FPROP && bias != nullptr) ? bias[c] : 0.f;
    for (int i = tid; i < PB * PLS; i += NT) lds[i] = 0.f;
    Stager<T, H, W, PB, NT, PLS, Map> st;
    st.prefetch(src, c, C, n0, n1);
    for (int nb = n0; nb < n1; nb += PB) {
        __syncthreads();
        st.commit(lds, nb, n1);
        __syncthreads();
        if (nb + PB < n1) st.prefetch(src, c, C, nb + PB, n1);
        const int nlive = nlive_s;
        for (int f = tid; f < PB * H * W; f += NT) {
            const int pl = f / (H * W), g = f % (H * W);
            if (nb + pl >= n1) break;
            const float *base = lds + pl * PLS + Map::index(g / W, g % W);
            float acc = bv;
            for (int s = 0; s < nlive; s++) acc = __builtin_fmaf(base[toff[s]], twt[s], acc);
            dst[((size_t)(nb + pl) * C + c) * (H * W) + g] = from_float<T>(acc);
        }
    }
}

// LDS bytes a launch of plane_kernel<.., K, H, W> needs
template <int K, int H, int W>
constexpr size_t plane_kernel_lds_bytes() {
    return ((size_t)Tile<H, W>::PB * plane_floats<K, H, W>() + 2 * K) * sizeof(float);
}

template <int OP, typename T, int K, int H, int W>
__global__ __launch_bounds__((Tile<H, W>::NT)) void plane_kernel(
    const T *__restrict__ src, const float *__restrict__ wt, const float *__restrict__ bias,
    const void *__restrict__ blob, T *__restrict__ dst, int N, int C, int G) {
    extern __shared__ float lds[];
    const int c = blockIdx.x % C;
    const int n0 = (blockIdx.x / C) * G;
    const int n1 = min(n0 + G, N);
    const int cls = taps_class(blob, C, K)[c];
#define DWO_CASE(O)                                                                  \
    case O:                                                                          \
        run_canonical<O, OP, T, K, H, W>(src, wt, bias, dst, lds, c, C, n0, n1);      \
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
            run_table<OP, T, K, H, W>(src, wt, bias, taps_dhdw(blob), dst, lds, c, C, n0, n1);
    }
#undef DWO_CASE
}

}  // namespace dwo

// Stage pipeline and output addressing shared by the three forward kernels
// (L_inf with argmax, interval bound, p-norm).
#pragma once
#include "kernels.hpp"
#include "tile.hpp"

#include <type_traits>

namespace ldist {

// Global -> register -> LDS staging of one pipeline stage: NX input panels
// (x, or lower and upper) followed by the weight panel.  IMG: the input is the image of a convolution-shaped
// layer and the panel is gathered from it (set `win` before init); the output keeps the conv layout.
template <class GEO, bool CONV, int VEC, int NX, bool IMG = false>
struct Stager {
    static_assert(!IMG || CONV, "an image has positions");
    static constexpr int STAGE = NX * GEO::XS + GEO::WS;  // floats per stage
    // Two LDS buffers (one barrier per stage) when that still lets a CU hold two waves
    // per SIMD, i.e. one 512-lane or two 256-lane workgroups in 160 KB; else one buffer.
    static constexpr int NBUF = (2 * STAGE * 4 * (GEO::KS == 1 ? 2 : 1) <= 160 * 1024) ? 2 : 1;
    static constexpr size_t LDS_BYTES = (size_t)NBUF * STAGE * sizeof(float);
    using WLoad = RowsK<GEO::BN, GEO::SN, GEO::NT, GEO::KK, VEC>;
    using XLoadK = RowsK<GEO::BM, GEO::SM, GEO::NT, GEO::KK, VEC>;
    using XLoadM = RowsM<GEO::BM, GEO::SM, GEO::NT, GEO::KK, VEC>;
    WLoad wl;
    XLoadK xlk[NX];
    XLoadM xlm[NX];
    using XLoadI = RowsImg<GEO::BM, GEO::SM, GEO::NT, GEO::KK>;
    XLoadI xli[IMG ? NX : 1];
    ImgWin win;
    int grp_;
    int off_m[XLoadM::N];
    const float* wbase;
    const float* in[NX];
    int K, ld_x, rows_x, rows_w, kstride, tid;

    __device__ __forceinline__ void init(const float* const (&input)[NX], const float* weight, const Dims& d, int m0,
                                         int n0, int g, int tid_) {
        tid = tid_;
        K = d.K;
        wbase = weight + ((size_t)g * d.NG + n0) * K;
        rows_w = d.NG - n0;
        rows_x = d.M - m0;
        kstride = d.HW;
        ld_x = d.G * K;
#pragma unroll
        for (int q = 0; q < NX; q++)
            in[q] = CONV ? input[q] : input[q] + ((size_t)m0 * d.G + g) * K;  // fc: row m is image b
        grp_ = g;
        if constexpr (CLAMPED) {
            wl.init_clamped(wbase, K, rows_w, tid);
#pragma unroll
            for (int q = 0; q < NX; q++) xlk[q].init_clamped(in[q], ld_x, rows_x, tid);
        }
        if constexpr (IMG) {
#pragma unroll
            for (int q = 0; q < NX; q++) xli[q].init(win, m0, d.M, tid);
        } else if constexpr (CONV) {
            XLoadM::offsets(off_m, m0, d.M, d.HW, d.G, g, K, tid);
        }
    }
    static constexpr bool CLAMPED = !CONV && VEC == 4;   // fc layout with 128-bit loads: buffer loads (RowsK::load_clamped)
    __device__ __forceinline__ void load(int k0) {
        if constexpr (CLAMPED) {
            if (k0 + GEO::KK <= K) {         // a whole stage: no predicates at all
                asm volatile("" ::: "memory");   // keeps this branch from being folded into the predicated one
                wl.template load_clamped<true>(k0, K, tid);
#pragma unroll
                for (int q = 0; q < NX; q++) xlk[q].template load_clamped<true>(k0, K, tid);
            } else {
                wl.template load_clamped<false>(k0, K, tid);
#pragma unroll
                for (int q = 0; q < NX; q++) xlk[q].template load_clamped<false>(k0, K, tid);
            }
            return;
        }
        wl.load(wbase, K, rows_w, k0, K, tid);
#pragma unroll
        for (int q = 0; q < NX; q++) {
            if constexpr (IMG) xli[q].load(in[q], win, grp_, k0, K, tid);
            else if constexpr (CONV) xlm[q].load(in[q], off_m, kstride, k0, K, tid);
            else xlk[q].load(in[q], ld_x, rows_x, k0, K, tid);
        }
    }
    // For the interval kernels (the last two panels are lower, upper): true when some value this lane
    // just loaded breaks lower <= upper, or is NaN or infinite (weights included).
    __device__ __forceinline__ bool interval_is_irregular() const {
        bool bad = false;
        if constexpr (NX >= 2) {
            constexpr float INF = __builtin_inff();
            constexpr int LO = NX - 2, UP = NX - 1;
            if constexpr (CONV) {
#pragma unroll
                for (int i = 0; i < XLoadM::N; i++)
#pragma unroll
                    for (int e = 0; e < VEC; e++) {
                        const float l = xlm[LO].v[i][e], u = xlm[UP].v[i][e];
                        bad |= !(l <= u && __builtin_fabsf(l) < INF && __builtin_fabsf(u) < INF);
                    }
            } else {
#pragma unroll
                for (int i = 0; i < XLoadK::N; i++)
#pragma unroll
                    for (int e = 0; e < VEC; e++) {
                        const float l = xlk[LO].v[i][e], u = xlk[UP].v[i][e];
                        bad |= !(l <= u && __builtin_fabsf(l) < INF && __builtin_fabsf(u) < INF);
                    }
            }
#pragma unroll
            for (int i = 0; i < WLoad::N; i++)
#pragma unroll
                for (int e = 0; e < VEC; e++) bad |= !(__builtin_fabsf(wl.v[i][e]) < INF);
        }
        return bad;
    }
    // Visits every value this lane holds of the stage it has loaded (weights and the input panels).
    template <class F>
    __device__ __forceinline__ void for_each_parked(F&& f) {
#pragma unroll
        for (int i = 0; i < WLoad::N; i++)
#pragma unroll
            for (int e = 0; e < VEC; e++) f(wl.v[i][e]);
#pragma unroll
        for (int q = 0; q < NX; q++) {
            if constexpr (IMG) {
#pragma unroll
                for (int i = 0; i < XLoadI::N; i++) f(xli[q].v[i]);
            } else if constexpr (CONV) {
#pragma unroll
                for (int i = 0; i < XLoadM::N; i++)
#pragma unroll
                    for (int e = 0; e < VEC; e++) f(xlm[q].v[i][e]);
            } else {
#pragma unroll
                for (int i = 0; i < XLoadK::N; i++)
#pragma unroll
                    for (int e = 0; e < VEC; e++) f(xlk[q].v[i][e]);
            }
        }
    }
    __device__ __forceinline__ void store(float* stage) const {
#pragma unroll
        for (int q = 0; q < NX; q++) {
            if constexpr (IMG) xli[q].store(stage + q * GEO::XS, tid);
            else if constexpr (CONV) xlm[q].store(stage + q * GEO::XS, tid);
            else xlk[q].store(stage + q * GEO::XS, tid);
        }
        wl.store(stage + NX * GEO::XS, tid);
    }
};

// Element offsets of row m of the input (k = 0) and of the output (n = 0), and
// the element strides of k and n, for either layout.
template <bool CONV>
struct RowAddr {
    size_t x, o;
    int xk, on;
    __device__ __forceinline__ RowAddr(const Dims& d, int m, int g) {
        if constexpr (CONV) {
            const int b = m / d.HW, hw = m % d.HW;
            x = ((size_t)(b * d.G + g) * d.K) * d.HW + hw;
            o = ((size_t)(b * d.G + g) * d.NG) * d.HW + hw;
            xk = d.HW;
            on = d.HW;
        } else {
            x = ((size_t)m * d.G + g) * d.K;
            o = ((size_t)m * d.G + g) * d.NG;
            xk = 1;
            on = 1;
        }
    }
};

// Writes one run of four consecutive rows (global rows m_first .. m_first+3) times the
// lane's TN columns of a result tensor.  When `vec` is set (base pointer 16-byte aligned,
// NG % 4 == 0 in the fc layout, HW % 4 == 0 in the conv layout) every group of four values
// along the contiguous axis (n for fc, the row index for conv) that lies fully inside the
// tensor goes out as one 128-bit store; everything else falls back to single stores.
template <class GEO, bool CONV, class T>
__device__ __forceinline__ void store_run(T* __restrict__ dst, const T (&val)[4][GEO::TN], const Dims& d, int m_first,
                                          int n0, int g, int tx, bool vec) {
    constexpr int TN = GEO::TN;
    using V4 = typename std::conditional<std::is_same<T, float>::value, float4, int4>::type;
    if constexpr (!CONV) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int m = m_first + e;
            if (m >= d.M) continue;
            T* row = dst + ((size_t)m * d.G + g) * d.NG;
#pragma unroll
            for (int r = 0; r < TN / 4; r++) {  // the lane's columns come in groups of four
                const int j = 4 * r;
                const int n = n0 + GEO::col(tx, j);
                if (vec && n + 3 < d.NG) {
                    V4 q;
                    q.x = val[e][j]; q.y = val[e][j + 1]; q.z = val[e][j + 2]; q.w = val[e][j + 3];
                    *reinterpret_cast<V4*>(row + n) = q;
                } else {
#pragma unroll
                    for (int c = 0; c < 4; c++)
                        if (n + c < d.NG) row[n + c] = val[e][j + c];
                }
            }
#pragma unroll
            for (int j = TN / 4 * 4; j < TN; j++) {
                const int n = n0 + GEO::col(tx, j);
                if (n < d.NG) row[n] = val[e][j];
            }
        }
    } else {
        if (m_first >= d.M) return;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + GEO::col(tx, j);
            if (n >= d.NG) continue;
            if (vec && m_first + 3 < d.M) {  // HW % 4 == 0 keeps the four rows inside one image
                const int b = m_first / d.HW, hw = m_first % d.HW;
                V4 q;
                q.x = val[0][j]; q.y = val[1][j]; q.z = val[2][j]; q.w = val[3][j];
                *reinterpret_cast<V4*>(dst + ((size_t)(b * d.G + g) * d.NG + n) * d.HW + hw) = q;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int me = m_first + e;
                    if (me < d.M) {
                        const int b = me / d.HW, hw = me % d.HW;
                        dst[((size_t)(b * d.G + g) * d.NG + n) * d.HW + hw] = val[e][j];
                    }
                }
            }
        }
    }
}

// Writes a lane's whole TM x TN patch (its rows come in runs of four, see Geo::row).
template <class GEO, bool CONV, class T>
__device__ __forceinline__ void store_patch(T* __restrict__ dst, const T (&val)[GEO::TM][GEO::TN], const Dims& d,
                                            int m0, int n0, int g, int tx, int ty, bool vec) {
#pragma unroll
    for (int r = 0; r < GEO::TM / 4; r++) {
        T run[4][GEO::TN];
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int j = 0; j < GEO::TN; j++) run[e][j] = val[4 * r + e][j];
        store_run<GEO, CONV>(dst, run, d, m0 + GEO::row(ty, 4 * r), n0, g, tx, vec);
    }
}

inline bool can_vec4_out(const Problem& pr, const void* a, const void* b = nullptr) {
    return aligned16(a) && aligned16(b) && (pr.HW == 1 ? pr.NG % 4 == 0 : pr.HW % 4 == 0);
}

inline Dims make_dims(const Problem& pr) { return Dims{pr.B, pr.G, pr.K, pr.NG, pr.HW, pr.B * pr.HW, 0, 0, 0, g_xcd_remap, 0}; }

// Dims::m_block for a kernel whose workgroup reads x_rows rows of the input panels (BM times the number of panels)
// and w_rows rows of weights per stage: `resident` workgroups share an L2 at a time (workgroups per CU times the CUs
// of an XCD); among the divisors mb of tiles_m, the piece mb x (resident / mb) with the fewest rows to stream wins.
// 0 (walk all row tiles) when that is the best there is.
inline int choose_m_block(int tiles_m, int x_rows, int w_rows, int resident) {
    int best = tiles_m;
    long best_cost = -1;
    for (int mb = 1; mb <= tiles_m && mb <= resident; mb++) {
        if (tiles_m % mb) continue;
        const long cost = (long)mb * x_rows + (long)((resident + mb - 1) / mb) * w_rows;
        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = mb; }
    }
    return best >= tiles_m ? 0 : best;
}
// workgroups of nt lanes and lds bytes that a CU holds (two waves per SIMD: these kernels use up to 256 registers)
inline int resident_per_xcd(int nt, size_t lds, int num_cu) {
    const int by_lds = (int)((size_t)160 * 1024 / (lds ? lds : 1)), by_waves = 512 / nt;
    const int per_cu = by_lds < by_waves ? by_lds : by_waves;
    return (per_cu > 0 ? per_cu : 1) * (num_cu / 8 > 0 ? num_cu / 8 : 1);
}

// 128-bit loads of the inputs and weights.  In the fc layout a lane addresses its vectors by 32-bit byte offsets
// from its tile's first row that must stay below 2 GB (RowsK::init_clamped): at most 256 rows of G * K elements.
inline bool can_vec4(const Problem& pr, const void* a, const void* b, const void* c = nullptr) {
    if (pr.HW == 1 && 4LL * 258 * pr.G * pr.K >= (1LL << 31)) return false;
    return pr.K % 4 == 0 && (pr.HW == 1 || pr.HW % 4 == 0) && aligned16(a) && aligned16(b) && aligned16(c);
}

// Input panels per stage of a kernel wrapper (its X_PANELS member; one when it has none).
template <class T, class = void> struct XPanels { static constexpr int value = 1; };
template <class T> struct XPanels<T, std::void_t<decltype(T::X_PANELS)>> { static constexpr int value = T::X_PANELS; };

// Launches KERNEL<GEO, CONV, VEC>::run for the layout and vector width of the
// problem.  KERNEL is a class template wrapping the __global__ function so that
// one dispatcher serves all forward kernels.
template <template <class, bool, int> class KERNEL, class GEO, class... Args>
hipError_t launch_forward(const Problem& pr, bool vec4, bool ovec, hipStream_t stream, Args... args) {
    Dims d = make_dims(pr);
    d.ovec = ovec;
    d.tiles_m = (d.M + GEO::BM - 1) / GEO::BM;
    d.tiles_n = (d.NG + GEO::BN - 1) / GEO::BN;
    const unsigned grid = (unsigned)d.tiles_m * d.tiles_n * d.G;
    if (pr.HW == 1) {
        constexpr int NX = XPanels<KERNEL<GEO, false, 4>>::value;
        d.m_block = choose_m_block(d.tiles_m, GEO::BM * NX, GEO::BN,
                                   resident_per_xcd(GEO::NT, Stager<GEO, false, 4, NX>::LDS_BYTES, pr.num_cu));
    }
    if (pr.HW == 1)
        return vec4 ? KERNEL<GEO, false, 4>::launch(grid, d, pr.device, stream, args...)
                    : KERNEL<GEO, false, 1>::launch(grid, d, pr.device, stream, args...);
    return vec4 ? KERNEL<GEO, true, 4>::launch(grid, d, pr.device, stream, args...)
                : KERNEL<GEO, true, 1>::launch(grid, d, pr.device, stream, args...);
}

template <template <class, bool, int> class KERNEL, class... Args>
hipError_t dispatch_forward(const Problem& pr, bool vec4, bool ovec, hipStream_t stream, Args... args) {
    switch (choose_tile(pr.B * pr.HW, pr.NG, pr.G, pr.num_cu)) {
        case TileChoice::M128N80K2:
            return launch_forward<KERNEL, Geo<128, 80, 8, 5, 2>>(pr, vec4, ovec, stream, args...);
        case TileChoice::M256N32K1:
            return launch_forward<KERNEL, Geo<256, 32, 8, 4, 1>>(pr, vec4, ovec, stream, args...);
        case TileChoice::M32N32K8:
            return launch_forward<KERNEL, Geo<32, 32, 4, 4, 8>>(pr, vec4, ovec, stream, args...);
        default:
            return launch_forward<KERNEL, Geo<128, 64, 8, 4, 1>>(pr, vec4, ovec, stream, args...);
    }
}

}  // namespace ldist

// Shared building blocks of the "tropical GEMM" forward kernels (gfx950, wave64).
//
// A workgroup owns a BM x BN tile of the (row m, output n) plane of one group
// and walks the reduction axis k in stages of KS*32 values.  The x and w panels
// of a stage sit in LDS as P[kk][m] (k-major, m contiguous) so that a lane reads
// the TM row values / TN column values it needs for one k with 128-bit LDS
// loads, and every value fetched from LDS is reused TN (resp. TM) times from
// registers.  The KS "k-groups" of a workgroup (each (BM/TM)*(BN/TN) lanes)
// share the panels and take alternate 32-wide chunks of k; their partial
// results are merged through LDS at the end.  This keeps two waves per SIMD
// busy on shapes whose m x n plane alone is too small to fill 256 CUs.
//
// Tensor layout (reference model/inf_dist_cuda.cu:29-33,65-66):
//   input (B, CI, HW): ((b*G + g)*K + k)*HW + hw     weight (CO, K): (g*NG + n)*K + k
//   output (B, CO, HW): ((b*G + g)*NG + n)*HW + hw
// "fc" kernels are the HW == 1 case (k contiguous in x), "conv" kernels the
// HW > 1 case (the row index hw is contiguous in x and in the output).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "conv_window.hpp"

namespace ldist {

constexpr int kChunk = 32;  // k values between two "did the maximum move" checks

struct Dims {
    int B, G, K, NG, HW;  // K = CI/G, NG = CO/G
    int M;                // B*HW rows
    int tiles_m, tiles_n;
    int ovec;             // outputs may be written with 128-bit stores
    int xcd_remap;        // 1: hand each XCD a contiguous run of tiles
    int m_block;          // > 0: row tiles are walked in blocks of this many (tile_of_block); 0: all of them
};

// XOR applied to the m (or n) coordinate of LDS row kk.  It permutes aligned
// groups of four floats inside aligned blocks of 32, so 128-bit accesses stay
// contiguous, panel rows need no padding, and the transposing 32-bit stores of
// the fc loader (16 lanes along k, 4 along m) hit 32 distinct banks.
__device__ __forceinline__ constexpr int swz(int kk) { return ((kk >> 2) & 7) << 2; }

template <int BM_, int BN_, int TM_, int TN_, int KS_>
struct Geo {
    static constexpr int BM = BM_, BN = BN_, TM = TM_, TN = TN_, KS = KS_;
    static constexpr int KK = KS * kChunk;       // k values per stage
    static constexpr int TX = BN / TN;           // lanes along n
    static constexpr int TY = BM / TM;           // lanes along m
    static constexpr int NGRP = TX * TY;         // lanes per k-group
    static constexpr int NT = NGRP * KS;         // workgroup size
    static constexpr int SM = (BM + 31) / 32 * 32;  // LDS row lengths
    static constexpr int SN = (BN + 31) / 32 * 32;
    static constexpr int XS = KK * SM;           // floats of one x panel
    static constexpr int WS = KK * SN;
    static_assert(TM == 4 || TM == 8, "TM");
    static_assert(TN == 3 || TN == 4 || TN == 5 || TN == 8, "TN");   // 3: columns tx*3 + j of the tile, kept at a pitch of four in the w panel
    static_assert(BM % TM == 0 && BN % TN == 0, "tile");
    static_assert(NT % 64 == 0, "whole waves");

    // Tile-local row of the i-th value a lane owns.  Eight values are two runs
    // of four, BM/2 apart, so that neighbouring lanes read neighbouring 16 bytes.
    __device__ static constexpr int row(int ty, int i) {
        return TM == 8 ? (i < 4 ? ty * 4 + i : BM / 2 + ty * 4 + (i - 4)) : ty * 4 + i;
    }
    __device__ static constexpr int col(int tx, int j) {
        return TN == 8 ? (j < 4 ? tx * 4 + j : BN / 2 + tx * 4 + (j - 4))
             : TN == 5 ? (j < 4 ? tx * 4 + j : TX * 4 + tx)
             : TN == 3 ? tx * 3 + j
                       : tx * 4 + j;
    }
};

// LDS address of the first value a lane reads in row kk (kk a multiple of 4: the
// swizzle is constant over an aligned run of four rows, so rows kk+1..kk+3 are
// plain row strides away).  BM/2 and BN/2 are multiples of 32, which the XOR
// never touches, so the second run of four sits at a fixed distance as well.
template <class GEO>
struct LanePtr {
    const float* x;   // x panel, row kk, this lane's first run of four rows
    const float* w;   // w panel, row kk, this lane's first run of four columns
    const float* w5;  // w panel, row kk, the lane's fifth column (TN == 5 only)
    __device__ __forceinline__ void set(const float* xp, const float* wp, int kk, int tx, int ty) {
        const int s = swz(kk);
        x = xp + kk * GEO::SM + ((ty * 4) ^ s);
        w = wp + kk * GEO::SN + ((tx * 4) ^ s);
        if constexpr (GEO::TN == 5) w5 = wp + kk * GEO::SN + ((GEO::TX * 4 + tx) ^ s);
    }
};

template <class GEO>
__device__ __forceinline__ void read_x(const float* __restrict__ p, int r, float (&xf)[GEO::TM]) {
    float4 a = *reinterpret_cast<const float4*>(p + r * GEO::SM);
    xf[0] = a.x; xf[1] = a.y; xf[2] = a.z; xf[3] = a.w;
    if constexpr (GEO::TM == 8) {
        float4 b = *reinterpret_cast<const float4*>(p + r * GEO::SM + GEO::BM / 2);
        xf[4] = b.x; xf[5] = b.y; xf[6] = b.z; xf[7] = b.w;
    }
}

template <class GEO>
__device__ __forceinline__ void read_w(const LanePtr<GEO>& lp, int r, float (&wf)[GEO::TN]) {
    float4 a = *reinterpret_cast<const float4*>(lp.w + r * GEO::SN);
    wf[0] = a.x; wf[1] = a.y; wf[2] = a.z;
    if constexpr (GEO::TN > 3) wf[3] = a.w;   // TN == 3: the fourth word of the lane's pitch is not a column
    if constexpr (GEO::TN == 8) {
        float4 b = *reinterpret_cast<const float4*>(lp.w + r * GEO::SN + GEO::BN / 2);
        wf[4] = b.x; wf[5] = b.y; wf[6] = b.z; wf[7] = b.w;
    }
    if constexpr (GEO::TN == 5) wf[4] = lp.w5[r * GEO::SN];
}

// Operand registers of KP consecutive k rows (1 or 2): NX x-like panels (1, or 2
// for the lower/upper interval ends) and the w panel.
template <class GEO, int NX, int KP>
struct Frag {
    float x[NX][KP][GEO::TM];
    float w[KP][GEO::TN];
    // rows r .. r+KP-1 relative to lp's row; xstride = floats between the x panels
    __device__ __forceinline__ void read(const LanePtr<GEO>& lp, int r, int xstride) {
#pragma unroll
        for (int q = 0; q < NX; q++)
#pragma unroll
            for (int e = 0; e < KP; e++) read_x<GEO>(lp.x + q * xstride, r + e, x[q][e]);
#pragma unroll
        for (int e = 0; e < KP; e++) read_w<GEO>(lp, r + e, w[e]);
    }
};

// The same operand fetch with 32-bit LDS byte addresses: the lane's column offsets are byte constants, so moving
// to another row costs an XOR with the row's swizzle (in bytes) and one three-operand add per pointer (five
// address instructions per trip of the L_inf forward instead of eleven with the pointer form above).  The
// scheduler also keeps a fragment's reads together as one burst with these, which suits the L_inf forward; the
// p-norm forward measured 8 % slower that way and stays on the pointer form.
typedef float vec4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const vec4f lds_vec4f;
typedef __attribute__((address_space(3))) const float lds_float;

__device__ __forceinline__ unsigned lds_address(const float* p) {   // of a pointer into the dynamic LDS array
    return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const float*)p;
}

template <class GEO>
struct LaneCols {
    unsigned x, w, w5;   // byte offsets of the lane's first row run / column run / fifth column inside a panel row
    __device__ __forceinline__ LaneCols(int tx, int ty) : x(ty * 16u), w(tx * 16u), w5((GEO::TX * 4 + tx) * 4u) {}
};

template <class GEO>
struct LaneAddr {
    unsigned x, w, w5;   // as LanePtr, LDS byte addresses
    __device__ __forceinline__ void set(unsigned xp, unsigned wp, int kk, const LaneCols<GEO>& c) {
        const unsigned s = (unsigned)swz(kk) * 4u;
        x = xp + (unsigned)kk * (GEO::SM * 4u) + (c.x ^ s);
        w = wp + (unsigned)kk * (GEO::SN * 4u) + (c.w ^ s);
        if constexpr (GEO::TN == 5) w5 = wp + (unsigned)kk * (GEO::SN * 4u) + (c.w5 ^ s);
    }
};

template <class GEO, int NX, int KP>
__device__ __forceinline__ void read_frag(Frag<GEO, NX, KP>& f, const LaneAddr<GEO>& lp, int r) {
#pragma unroll
    for (int q = 0; q < NX; q++)
#pragma unroll
        for (int e = 0; e < KP; e++) {
            const unsigned at = lp.x + q * (GEO::XS * 4u) + (r + e) * (GEO::SM * 4u);
            const vec4f a = *(lds_vec4f*)(uintptr_t)at;
            f.x[q][e][0] = a.x; f.x[q][e][1] = a.y; f.x[q][e][2] = a.z; f.x[q][e][3] = a.w;
            if constexpr (GEO::TM == 8) {
                const vec4f b = *(lds_vec4f*)(uintptr_t)(at + GEO::BM / 2 * 4u);
                f.x[q][e][4] = b.x; f.x[q][e][5] = b.y; f.x[q][e][6] = b.z; f.x[q][e][7] = b.w;
            }
        }
#pragma unroll
    for (int e = 0; e < KP; e++) {
        const unsigned at = lp.w + (r + e) * (GEO::SN * 4u);
        const vec4f a = *(lds_vec4f*)(uintptr_t)at;
        f.w[e][0] = a.x; f.w[e][1] = a.y; f.w[e][2] = a.z;
        if constexpr (GEO::TN > 3) f.w[e][3] = a.w;
        if constexpr (GEO::TN == 8) {
            const vec4f b = *(lds_vec4f*)(uintptr_t)(at + GEO::BN / 2 * 4u);
            f.w[e][4] = b.x; f.w[e][5] = b.y; f.w[e][6] = b.z; f.w[e][7] = b.w;
        }
        if constexpr (GEO::TN == 5) f.w[e][4] = *(lds_float*)(uintptr_t)(lp.w5 + (r + e) * (GEO::SN * 4u));
    }
}

// Walks one 32-row chunk of the panels and calls f(frag, kk) once per KP k rows
// (kk = first row of the fragment inside the chunk, ascending).
// 2*KP rows per trip, as two fragments: the operands of the next fragment are
// fetched from LDS while the current one is being reduced.  The loop is kept
// rolled on purpose: unrolled, the compiler hoists every LDS read of the chunk
// above the arithmetic and spills the accumulators.  Without the scheduling
// barriers it sinks each fetch down to its first use, which puts the LDS
// latency back on the critical path.
struct NoMid { __device__ __forceinline__ void operator()() const {} };

// mid() runs once, between rows 15 and 16 of the chunk (after the trip that reduces rows 12..15).
template <class GEO, int NX, int KP, bool BYTE_ADDR = false, class F, class MID = NoMid>
__device__ __forceinline__ void sweep_chunk(const float* xp, const float* wp, int tx, int ty, F&& f, MID&& mid = MID()) {
    static_assert(KP == 1 || KP == 2, "a trip must stay inside one aligned run of four rows");
    constexpr int XSTRIDE = GEO::XS;
    // LDS instructions of one fragment read: 128-bit reads of x and w, plus the fifth column
    // (its KP 32-bit reads merge into one ds_read2_b32).  LDS returns in order, so waiting until
    // that many are outstanding means: the fragment fetched before this one has arrived.  The
    // explicit wait is only a hint that keeps the compiler from waiting for everything
    // (lgkmcnt(0)) right after a fetch; it still adds whatever wait correctness needs.
    constexpr int FRAG_LDS = NX * KP * (GEO::TM / 4) + KP * (GEO::TN == 8 ? 2 : 1) + (GEO::TN == 5 ? 1 : 0);
    constexpr int WAIT_PREV = 0xc07f | (FRAG_LDS << 8);   // vmcnt, expcnt at their maxima; lgkmcnt = FRAG_LDS
    static_assert(FRAG_LDS < 16, "lgkmcnt field");
    Frag<GEO, NX, KP> a, b;
    // Nothing but this sweep's own LDS reads may be in flight inside the loop: a scalar load left
    // pending here (they return out of order) would force lgkmcnt(0) at the top of every trip.
    if constexpr (BYTE_ADDR) {
        LaneAddr<GEO> cur, nxt;
        const LaneCols<GEO> cols(tx, ty);
        const unsigned xb = lds_address(xp), wb = lds_address(wp);
        cur.set(xb, wb, 0, cols);
        __builtin_amdgcn_s_waitcnt(0xc07f);
        read_frag(a, cur, 0);
#pragma unroll 1
        for (int kk = 0; kk < kChunk; kk += 2 * KP) {
            read_frag(b, cur, KP);
            __builtin_amdgcn_sched_barrier(0);   // keep each fetch ahead of the arithmetic it overlaps with
            __builtin_amdgcn_s_waitcnt(WAIT_PREV);
            __builtin_amdgcn_sched_barrier(0);
            f(a, kk);
            nxt.set(xb, wb, (kk + 2 * KP) & (kChunk - 1), cols);  // the last trip re-reads row 0; harmless
            read_frag(a, nxt, 0);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(WAIT_PREV);
            __builtin_amdgcn_sched_barrier(0);
            f(b, kk + KP);
            cur = nxt;
            if constexpr (!std::is_same<typename std::decay<MID>::type, NoMid>::value)
                if (kk == kChunk / 2 - 2 * KP) mid();
        }
    } else {
        LanePtr<GEO> cur, nxt;
        cur.set(xp, wp, 0, tx, ty);
        __builtin_amdgcn_s_waitcnt(0xc07f);
        a.read(cur, 0, XSTRIDE);
#pragma unroll 1
        for (int kk = 0; kk < kChunk; kk += 2 * KP) {
            b.read(cur, KP, XSTRIDE);
            __builtin_amdgcn_sched_barrier(0);   // keep each fetch ahead of the arithmetic it overlaps with
            __builtin_amdgcn_s_waitcnt(WAIT_PREV);
            __builtin_amdgcn_sched_barrier(0);
            f(a, kk);
            nxt.set(xp, wp, (kk + 2 * KP) & (kChunk - 1), tx, ty);  // the last trip re-reads row 0; harmless
            a.read(nxt, 0, XSTRIDE);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(WAIT_PREV);
            __builtin_amdgcn_sched_barrier(0);
            f(b, kk + KP);
            cur = nxt;
            if constexpr (!std::is_same<typename std::decay<MID>::type, NoMid>::value)
                if (kk == kChunk / 2 - 2 * KP) mid();
        }
    }
}

// The same walk over rows [k_begin, k_begin + LEN) of the chunk (LEN = 32: all of it, 16: one half) with the first
// fragment taken out of the loop and given to `first`, so that it can read its accumulators from one register array
// and write them to another (the L_inf forward continues the running maximum of the stage before in a second array
// and would otherwise copy forty registers per chunk).  Byte-address form only.  The fragments between the first
// and the last run as trips of two, the last one after the loop.
template <class GEO, int NX, int KP, int LEN, class F0, class F>
__device__ __forceinline__ void sweep_chunk_first(const float* xp, const float* wp, int tx, int ty, int k_begin,
                                                  F0&& first, F&& f) {
    static_assert(KP == 2 && LEN % 4 == 0 && LEN >= 8, "fragments of two k, trips of two fragments");
    constexpr int FRAG_LDS = NX * KP * (GEO::TM / 4) + KP * (GEO::TN == 8 ? 2 : 1) + (GEO::TN == 5 ? 1 : 0);
    constexpr int WAIT_PREV = 0xc07f | (FRAG_LDS << 8);
    static_assert(FRAG_LDS < 16, "lgkmcnt field");
    Frag<GEO, NX, KP> a, b;
    LaneAddr<GEO> cur, nxt;
    const LaneCols<GEO> cols(tx, ty);
    const unsigned xb = lds_address(xp), wb = lds_address(wp);
    cur.set(xb, wb, k_begin, cols);
    __builtin_amdgcn_s_waitcnt(0xc07f);
    read_frag(a, cur, 0);
    read_frag(b, cur, KP);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(WAIT_PREV);
    __builtin_amdgcn_sched_barrier(0);
    first(a, k_begin);
#pragma unroll 1
    for (int kk = k_begin + KP; kk < k_begin + LEN - KP; kk += 2 * KP) {   // b holds rows kk, kk + 1 of the chunk
        nxt.set(xb, wb, kk + KP, cols);
        read_frag(a, nxt, 0);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(WAIT_PREV);
        __builtin_amdgcn_sched_barrier(0);
        f(b, kk);
        read_frag(b, nxt, KP);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(WAIT_PREV);
        __builtin_amdgcn_sched_barrier(0);
        f(a, kk + KP);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    f(b, k_begin + LEN - KP);
}

// Same walk without the operand prefetch, one k row per trip: for rarely taken
// paths that must not add to the register budget of the hot loop.
template <class GEO, int NX, class F>
__device__ __forceinline__ void sweep_chunk_plain(const float* xp, const float* wp, int tx, int ty, F&& f) {
#pragma unroll 1
    for (int kk = 0; kk < kChunk; kk++) {
        LanePtr<GEO> lp;
        lp.set(xp, wp, kk & ~3, tx, ty);
        Frag<GEO, NX, 1> a;
        a.read(lp, kk & 3, GEO::XS);
        f(a, kk);
    }
}

// ---------------------------------------------------------------------------
// Stage loaders: global -> registers (issued early) -> LDS (after the compute).
// RowsK<ROWS, LD, NT, KK, VEC> covers a panel whose rows are k-contiguous in
// memory (weight always; input when HW == 1).  Lanes run along k first, so a
// wave reads whole 64..256-byte row segments; the store transposes into P[kk][r].
// Values outside the matrix (r >= rows_valid, k >= K) are loaded as 0, which is
// neutral for every reduction here (|0 - 0| never raises a maximum or a sum).
// ---------------------------------------------------------------------------
template <int ROWS, int LD, int NT, int KK, int VEC>
struct RowsK {
    static constexpr int PER_ROW = KK / VEC;               // vectors per panel row
    static constexpr int TOTAL = ROWS * PER_ROW;
    static constexpr int N = (TOTAL + NT - 1) / NT;        // vectors per lane
    float v[N][VEC];

    // base: pointer to (row 0 of the tile, k = 0); ld: elements between rows.  Rows and k outside the matrix read
    // as zeros, which every reduction here ignores.
    __device__ __forceinline__ void load(const float* __restrict__ base, int ld, int rows_valid, int k0, int K,
                                         int tid) {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int id = tid + i * NT;
            const int r = id / PER_ROW, kq = id % PER_ROW;
            const int k = k0 + kq * VEC;
            const bool ok = (TOTAL % NT == 0 || id < TOTAL) && r < rows_valid;
            const float* p = base + (size_t)r * ld + k;
            if constexpr (VEC == 4) {
                float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                if (ok && k < K) t = *reinterpret_cast<const float4*>(p);  // K % 4 == 0 on this path
                v[i][0] = t.x; v[i][1] = t.y; v[i][2] = t.z; v[i][3] = t.w;
            } else {
                v[i][0] = (ok && k < K) ? *p : 0.f;
            }
        }
    }
    // For callers that never use the results of rows past the matrix (the forward kernels: they are not stored):
    // such rows read the matrix's last row instead, so a row needs no predicate, and a lane's byte offsets from the
    // tile's first row are fixed for the whole reduction.  The loads are buffer loads: a descriptor of the tile's
    // first row in scalar registers (the same for every lane), the lane's 32-bit offset, and the stage's k0 as the
    // scalar offset, so a load costs no address arithmetic; an offset of all ones lies outside the descriptor's 2 GB
    // range and reads as zeros, which takes the place of every predicate (lanes without a vector in a round, k >= K
    // in the last stage) without zeros in registers or branches.  The host checks that real offsets stay below 2 GB.
    unsigned off[N];   // bytes
    __amdgpu_buffer_rsrc_t rsrc;
    typedef float F4 __attribute__((ext_vector_type(4)));
    __device__ __forceinline__ void init_clamped(const float* base, int ld, int rows_valid, int tid) {
        rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)0x80000000u, 0x00020000);
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int id = tid + i * NT;
            off[i] = 4u * ((unsigned)min(id / PER_ROW, rows_valid - 1) * (unsigned)ld + (unsigned)(id % PER_ROW) * VEC);
            if (TOTAL % NT != 0 && id >= TOTAL) off[i] = ~0u;
        }
    }
    // INSIDE: the stage lies inside the reduction axis (k0 + KK <= K; uniform over the workgroup).
    template <bool INSIDE>
    __device__ __forceinline__ void load_clamped(int k0, int K, int tid) {
        static_assert(VEC == 4 && NT % PER_ROW == 0, "128-bit loads; a lane keeps its k offset over the rounds");
        const bool k_ok = INSIDE || k0 + (tid % PER_ROW) * VEC < K;
#pragma unroll
        for (int i = 0; i < N; i++) {
            const F4 t = __builtin_bit_cast(F4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, k_ok ? off[i] : ~0u, k0 * 4, 0));
            v[i][0] = t.x; v[i][1] = t.y; v[i][2] = t.z; v[i][3] = t.w;
        }
    }
    __device__ __forceinline__ void store(float* __restrict__ panel, int tid) const {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int id = tid + i * NT;
            if (TOTAL % NT != 0 && id >= TOTAL) continue;
            const int r = id / PER_ROW, kq = id % PER_ROW;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                const int kk = kq * VEC + e;
                panel[kk * LD + (r ^ swz(kk))] = v[i][e];
            }
        }
    }
};

// RowsM covers the input panel of the conv layout: for a fixed k the rows
// m = b*HW + hw are contiguous in memory (within one b), so lanes run along m
// and the LDS store needs no transpose.  VEC == 4 requires HW % 4 == 0, which
// keeps every aligned run of four rows inside one image b.
template <int ROWS, int LD, int NT, int KK, int VEC>
struct RowsM {
    static constexpr int PER_K = ROWS / VEC;
    static constexpr int TOTAL = KK * PER_K;
    static constexpr int N = (TOTAL + NT - 1) / NT;
    static_assert(NT % PER_K == 0 || PER_K % NT == 0, "lane keeps its rows across iterations");
    float v[N][VEC];

    // off_m: element offset of (row, k = group's first channel) for this lane's
    // first row, or -1 if that row is outside the matrix; kstride = HW.
    __device__ __forceinline__ void load(const float* __restrict__ input, const int (&off_m)[N], int kstride, int k0,
                                         int K, int tid) {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int id = tid + i * NT;
            const int kk = id / PER_K;
            const int k = k0 + kk;
            const bool ok = (TOTAL % NT == 0 || id < TOTAL) && off_m[i] >= 0 && k < K;
            const float* p = input + (size_t)off_m[i] + (size_t)k * kstride;
            if constexpr (VEC == 4) {
                float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                if (ok) t = *reinterpret_cast<const float4*>(p);
                v[i][0] = t.x; v[i][1] = t.y; v[i][2] = t.z; v[i][3] = t.w;
            } else {
                v[i][0] = ok ? *p : 0.f;
            }
        }
    }
    __device__ __forceinline__ void store(float* __restrict__ panel, int tid) const {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int id = tid + i * NT;
            if (TOTAL % NT != 0 && id >= TOTAL) continue;
            const int kk = id / PER_K, mq = id % PER_K;
            if constexpr (VEC == 4) {
                *reinterpret_cast<float4*>(panel + kk * LD + ((mq * 4) ^ swz(kk))) =
                    make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
            } else {
                panel[kk * LD + (mq ^ swz(kk))] = v[i][0];
            }
        }
    }
    // Fills off_m for this lane: rows of the tile start at global row m0.
    __device__ __forceinline__ static void offsets(int (&off_m)[N], int m0, int M, int HW, int G, int g, int K,
                                                   int tid) {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int id = tid + i * NT;
            const int mq = id % PER_K;
            const int m = m0 + mq * VEC;
            if (m < M) {
                const int b = m / HW, hw = m % HW;
                off_m[i] = ((b * G + g) * K) * HW + hw;
            } else {
                off_m[i] = -1;
            }
        }
    }
};

// Panel whose columns are contiguous in memory for a fixed row of the reduction: P[rr][col] = src[n0 + rr][k0 + col]
// (the weights of a stage of outputs for grad_input, the inputs of a stage of rows for grad_weight).  Lanes run
// along the columns and nothing is transposed.  VEC == 4 needs K % 4 == 0 and a 16-byte aligned base.
template <int COLS, int LD, int NT, int KK, int VEC>
struct RowsT {
    static constexpr int PER_ROW = COLS / VEC;
    static constexpr int TOTAL = KK * PER_ROW;
    static constexpr int N = (TOTAL + NT - 1) / NT;
    float v[N][VEC];
    // base: pointer to (first row of the reduction, column 0); rows are `stride` apart, R of them, K columns
    __device__ __forceinline__ void load(const float* __restrict__ base, int stride, int n0, int R, int k0, int K, int tid) {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int id = tid + i * NT;
            const int rr = id / PER_ROW, cq = id % PER_ROW;
            const int n = n0 + rr, k = k0 + cq * VEC;
            const bool ok = (TOTAL % NT == 0 || id < TOTAL) && n < R && k < K;
            const float* p = base + (size_t)n * stride + k;
            if constexpr (VEC == 4) {
                float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                if (ok) t = *reinterpret_cast<const float4*>(p);
                v[i][0] = t.x; v[i][1] = t.y; v[i][2] = t.z; v[i][3] = t.w;
            } else {
                v[i][0] = ok ? *p : 0.f;
            }
        }
    }
    __device__ __forceinline__ void store(float* __restrict__ panel, int tid) const {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int id = tid + i * NT;
            if (TOTAL % NT != 0 && id >= TOTAL) continue;
            const int rr = id / PER_ROW, cq = id % PER_ROW;
            if constexpr (VEC == 4)
                *reinterpret_cast<float4*>(panel + rr * LD + ((cq * 4) ^ swz(rr))) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
            else
                panel[rr * LD + (cq ^ swz(rr))] = v[i][0];
        }
    }
};

// Sum over groups of N = 8 or 16 neighbouring lanes of a DPP row (log2 N row shifts): the total arrives in each
// group's last lane, the others hold prefix sums.  Every lane of the row must be active.  With N = 8 a shift pulls
// values across the border between a row's two groups, but only into lanes whose result is not used: lane 7 sums
// lanes 0 .. 7 and lane 15 lanes 8 .. 15.
template <int N>
__device__ __forceinline__ float dpp_lanes_total(float v) {
    static_assert(N == 8 || N == 16, "groups of 8 or 16 lanes");
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, true));  // row_shr:1
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x112, 0xf, 0xf, true));  // row_shr:2
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xf, 0xf, true));  // row_shr:4
    if constexpr (N == 16)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x118, 0xf, 0xf, true));  // row_shr:8
    return v;
}

// The input panel of the convolution-shaped layer gathered from the image (see conv_window.hpp): same panel as
// RowsM would load from the unfolded tensor.  A lane keeps one row of the tile, i.e. one window, and walks k.
template <int ROWS, int LD, int NT, int KK>
struct RowsImg {
    static constexpr int TOTAL = KK * ROWS;
    static constexpr int N = TOTAL / NT;
    static constexpr int KSTEP = NT / ROWS;
    static_assert(NT % ROWS == 0 && TOTAL % NT == 0, "lane keeps its row across iterations");
    float v[N];
    WinRow row;
    bool row_ok;

    __device__ __forceinline__ void init(const ImgWin& q, int m0, int M, int tid) {
        const int m = m0 + tid % ROWS;
        row_ok = m < M;
        row.set(q, row_ok ? m : 0);
    }
    __device__ __forceinline__ void load(const float* __restrict__ img, const ImgWin& q, int g, int k0, int K, int tid) {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int k = k0 + tid / ROWS + i * KSTEP;
            size_t off;
            const bool ok = win_tap(q, row, g, k < K ? k : 0, off) && row_ok && k < K;
            v[i] = ok ? img[off] : 0.f;
        }
    }
    __device__ __forceinline__ void store(float* __restrict__ panel, int tid) const {
        const int mq = tid % ROWS;
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int kk = tid / ROWS + i * KSTEP;
            panel[kk * LD + (mq ^ swz(kk))] = v[i];
        }
    }
};

// Maps the linear workgroup id to (tile_m, tile_n, group).  Consecutive ids go
// to different XCDs (8 per device, each with its own L2); the remap hands every
// XCD one contiguous run of tiles, m fastest, so the workgroups that share an
// L2 also share their w strip (and, across runs, their x strips).
// With many row tiles a run is longer than what an XCD holds at a time, and walking all row tiles before the next
// column tile would make each round of resident workgroups read every x strip again.  m_block > 0 walks the row
// tiles in blocks of that many instead (block, then column tile, then row tile inside the block), so that a
// round covers a near-square piece of the output: few x strips and few w strips (choose_m_block() on the host).
__device__ __forceinline__ void tile_of_block(const Dims& d, int& tm, int& tn, int& g) {
    const int total = gridDim.x;
    int id = blockIdx.x;
    constexpr int XCD = 8;
    if (d.xcd_remap && total % XCD == 0) id = (id % XCD) * (total / XCD) + id / XCD;
    const int per_group = d.tiles_m * d.tiles_n;
    g = id / per_group;
    const int j = id - g * per_group;
    if (d.m_block > 0) {                       // tiles_m is a multiple of m_block
        const int per_block = d.m_block * d.tiles_n;
        const int mb = j / per_block, r = j - mb * per_block;
        tn = r / d.m_block;
        tm = mb * d.m_block + (r - tn * d.m_block);
    } else {
        tn = j / d.tiles_m;
        tm = j - tn * d.tiles_m;
    }
}

}  // namespace ldist

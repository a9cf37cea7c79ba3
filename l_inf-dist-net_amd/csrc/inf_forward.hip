// L_inf distance forward with argmax: out[m,n] = max_k |x[m,k] - w[n,k]|,
// pos[m,n] = lowest k attaining it (bit 31 set when x - w < 0 there).
// Semantics follow the reference kernel model/inf_dist_cuda.cu:10-68.
//
// Hot loop: per (m,n,k) one v_sub_f32 plus half a v_max3_f32 (|.| is a free
// source modifier), with no index bookkeeping.  Only once per 32-wide chunk of
// k is the chunk maximum compared with the running maximum; a strict '>' there
// records the chunk.  After the k loop the lowest k with |x-w| == out is found
// by scanning that one chunk again, which reproduces "scan k ascending, update
// on strict >" exactly (the first chunk to reach the final maximum contains the
// first k to reach it).
#include "fwd_engine.hpp"
#include "inf_locate.hpp"
#include "skinny.hpp"

namespace ldist {

// EXACT = false: track the chunk of the maximum and locate k afterwards (1.5 + 3/32 VALU
// instructions per element, plus one re-read of a 32-wide chunk per output).
// EXACT = true: track k itself (subtract, compare, two selects = 4 instructions per
// element, no re-read).  That pays in the conv layout with short K, where the re-read is a
// strided gather that costs more than the whole reduction.
// HALF (fc layout with vector loads, short reductions): the chunk is recorded in halves of 16, which halves what the
// search after the loop reads per output, for one more compare, select and copy per output and chunk in the loop.
template <class GEO, bool CONV, int VEC, bool EXACT, bool HALF = false>
__global__ void __launch_bounds__(GEO::NT, 2)
inf_forward_kernel(const float* __restrict__ input, const float* __restrict__ weight, float* __restrict__ output,
                   int32_t* __restrict__ pos, Dims d) {
    constexpr int BM = GEO::BM, BN = GEO::BN, TM = GEO::TM, TN = GEO::TN, KS = GEO::KS, KK = GEO::KK;
    constexpr int NGRP = GEO::NGRP;
    using Stage = Stager<GEO, CONV, VEC, 1>;
    constexpr int STAGE = Stage::STAGE, NBUF = Stage::NBUF;
    extern __shared__ __align__(16) float lds[];

    int tm, tn, g;
    tile_of_block(d, tm, tn, g);
    const int m0 = tm * BM, n0 = tn * BN;
    const int tid = threadIdx.x;
    const int grp = tid / NGRP, t = tid % NGRP;
    const int tx = t % GEO::TX, ty = t / GEO::TX;
    const int K = d.K;

    Stage st;
    const float* const ins[1] = {input};
    st.init(ins, weight, d, m0, n0, g, tid);

    float acc[TM][TN], cm[TM][TN];   // running maxima; the stages alternate between them
    int cidx[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) { acc[i][j] = 0.f; cm[i][j] = 0.f; cidx[i][j] = 0; }

    const int nstage = (K + KK - 1) / KK;
    st.load(0);
    st.store(lds);
    __syncthreads();
    // One stage: a k-group sweeps its chunk of the resident panels.  prev holds the running
    // maximum before the chunk and is left alone; cur continues from it, so the chunk raised the
    // maximum iff cur > prev afterwards.  The two arrays swap roles from stage to stage, which
    // saves copying cur back (EXACT keeps everything in prev; with HALF the two halves of a chunk
    // swap them twice, so the result is in prev again).
    auto run_stage = [&](float (&prev)[TM][TN], float (&cur)[TM][TN], int s) {
        const float* stage = lds + (s % NBUF) * STAGE;
        if (s + 1 < nstage) st.load((s + 1) * KK);
        const float* xp = stage + grp * kChunk * GEO::SM;
        const float* wp = stage + GEO::XS + grp * kChunk * GEO::SN;
        const int c = s * KS + grp;
        if constexpr (EXACT) {
            sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int kk) {
                const int k0 = c * kChunk + kk;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float d0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]);
                        const float d1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]);
                        if (d0 > prev[i][j]) { prev[i][j] = d0; cidx[i][j] = k0; }
                        if (d1 > prev[i][j]) { prev[i][j] = d1; cidx[i][j] = k0 + 1; }
                    }
            });
        } else {
            // Sweeps rows [k_begin, k_begin + LEN) of the chunk: the first fragment takes the running maximum from
            // `from` and leaves it in `to` (no copy), the others continue in `to`.
            auto sweep_into = [&](const float (&from)[TM][TN], float (&to)[TM][TN], int k_begin, auto len) {
                auto body_first = [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            const float d0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]);
                            const float d1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]);
                            to[i][j] = __builtin_fmaxf(__builtin_fmaxf(from[i][j], d0), d1);
                        }
                };
                auto body = [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            const float d0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]);
                            const float d1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]);
                            to[i][j] = __builtin_fmaxf(__builtin_fmaxf(to[i][j], d0), d1);
                        }
                };
                sweep_chunk_first<GEO, 1, 2, decltype(len)::value>(xp, wp, tx, ty, k_begin, body_first, body);
            };
            // Records `tag` for the outputs whose maximum a sweep raised (newer > older).  Two patch rows' compares
            // first, each into its own pair of scalar registers, then their selects: a select straight after its
            // compare (what the compiler makes of the plain form) waits two cycles for the lane mask.  The empty asm
            // statements keep their order: the first kind keeps the compiler from folding a mask back into the plain
            // form, the second ends a group, so that no more than ten masks are live (all forty would push other
            // scalars out of their registers).
            static_assert(TM % 2 == 0, "rows in pairs");
            auto record = [&](const float (&newer)[TM][TN], const float (&older)[TM][TN], int tag) {
#pragma unroll
                for (int i = 0; i < TM; i += 2) {
                    unsigned long long raised[2][TN];
#pragma unroll
                    for (int a = 0; a < 2; a++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            raised[a][j] = __builtin_amdgcn_fcmpf(newer[i + a][j], older[i + a][j], 2 /* ordered > */);
                            asm volatile("" : "+s"(raised[a][j]));
                        }
#pragma unroll
                    for (int a = 0; a < 2; a++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            if (__builtin_amdgcn_inverse_ballot_w64(raised[a][j])) cidx[i + a][j] = tag;
                            asm volatile("" : "+v"(cidx[i + a][j]));
                        }
                }
            };
            if constexpr (HALF) {   // two halves of 16: the second goes back into prev, which ends up holding the result
                sweep_into(prev, cur, 0, std::integral_constant<int, kChunk / 2>{});
                record(cur, prev, 2 * c);
                sweep_into(cur, prev, kChunk / 2, std::integral_constant<int, kChunk / 2>{});
                record(prev, cur, 2 * c + 1);
            } else {
                sweep_into(prev, cur, 0, std::integral_constant<int, kChunk>{});
                record(cur, prev, c);
            }
        }
        if (NBUF == 1) __syncthreads();  // everyone is done reading the only buffer
        if (s + 1 < nstage) st.store(lds + ((s + 1) % NBUF) * STAGE);
        __syncthreads();
    };
    if constexpr (EXACT) {
        for (int s = 0; s < nstage; s++) run_stage(acc, acc, s);
    } else if constexpr (HALF) {
        for (int s = 0; s < nstage; s++) run_stage(acc, cm, s);
    } else {
        for (int s = 0; s < nstage; s += 2) {
            run_stage(acc, cm, s);
            if (s + 1 < nstage) {
                run_stage(cm, acc, s + 1);
            } else {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) acc[i][j] = cm[i][j];
            }
        }
    }

    // Epilogue, independent of the lane patch: the tile's (value, chunk or k) pairs are parked in
    // LDS (free by now), k-groups merge there in turn, the whole workgroup turns the recorded
    // chunk into the reference's pos, and the tile goes out with stores along the contiguous axis.
    // cand index of tile-local (row ml, column nl): the contiguous output axis is innermost.
    auto slot = [](int ml, int nl) { return CONV ? nl * BM + ml : ml * BN + nl; };
    float* cand_v = lds;
    int* cand_c = reinterpret_cast<int*>(lds) + BM * BN;
    // A lane's patch comes in runs of four along the contiguous axis of the parking area (four neighbouring
    // columns in the fc layout, four neighbouring rows in the conv layout): those go through 128-bit LDS accesses,
    // the fifth column of a 5-wide patch singly.
    auto merge4 = [&](int o, float (&v)[4], int (&c)[4], bool compare) {
        if (compare) {   // larger value wins; equal values keep the lower chunk (or k)
            const float4 ov = *reinterpret_cast<const float4*>(cand_v + o);
            const int4 oc = *reinterpret_cast<const int4*>(cand_c + o);
            const float pv[4] = {ov.x, ov.y, ov.z, ov.w};
            const int pc[4] = {oc.x, oc.y, oc.z, oc.w};
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (!(v[e] > pv[e] || (v[e] == pv[e] && c[e] < pc[e]))) { v[e] = pv[e]; c[e] = pc[e]; }
        }
        *reinterpret_cast<float4*>(cand_v + o) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<int4*>(cand_c + o) = make_int4(c[0], c[1], c[2], c[3]);
    };
#pragma unroll 1
    for (int turn = 0; turn < KS; turn++) {
        if (grp == turn) {
            if constexpr (!CONV) {
#pragma unroll
                for (int i = 0; i < TM; i++) {
#pragma unroll
                    for (int q = 0; q < TN / 4; q++) {
                        float v[4] = {acc[i][4 * q], acc[i][4 * q + 1], acc[i][4 * q + 2], acc[i][4 * q + 3]};
                        int c[4] = {cidx[i][4 * q], cidx[i][4 * q + 1], cidx[i][4 * q + 2], cidx[i][4 * q + 3]};
                        merge4(slot(GEO::row(ty, i), GEO::col(tx, 4 * q)), v, c, turn > 0);
                    }
#pragma unroll
                    for (int j = TN / 4 * 4; j < TN; j++) {
                        const int o = slot(GEO::row(ty, i), GEO::col(tx, j));
                        bool take = true;
                        if (turn > 0) {
                            const float v = cand_v[o];
                            take = acc[i][j] > v || (acc[i][j] == v && cidx[i][j] < cand_c[o]);
                        }
                        if (take) { cand_v[o] = acc[i][j]; cand_c[o] = cidx[i][j]; }
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int r = 0; r < TM / 4; r++) {
                        float v[4] = {acc[4 * r][j], acc[4 * r + 1][j], acc[4 * r + 2][j], acc[4 * r + 3][j]};
                        int c[4] = {cidx[4 * r][j], cidx[4 * r + 1][j], cidx[4 * r + 2][j], cidx[4 * r + 3][j]};
                        merge4(slot(GEO::row(ty, 4 * r), GEO::col(tx, j)), v, c, turn > 0);
                    }
            }
        }
        __syncthreads();
    }

    if constexpr (!EXACT && !CONV && VEC == 4) {
        // fc layout: a recorded chunk is 128 contiguous, 16-byte aligned bytes of the x row and of
        // the w row.  Four neighbouring lanes take one output: each loads 32 bytes of both rows,
        // so a wave's load instruction touches 16 whole lines instead of 64 partial ones (a lane
        // that walks its own outputs alone is bound by the tag look-ups of the vector cache, not
        // by bytes).  The lowest matching k is the match of the lowest lane that has one: a ballot
        // tells every lane whether a lower lane of its four matched.  Rows and columns past the
        // edge of the tensor read a clamped, valid address and are never stored.
        // The walk is as much a matter of vector instructions as of bytes (about fifty per output and lane group
        // with eight lanes of 16 bytes each; four lanes of 32 bytes need 30 per output), so the row and column
        // of the next output and their offsets are carried along instead of divided and multiplied out.
        constexpr int RUN = HALF ? kChunk / 2 : kChunk;   // k values a recorded index stands for
        constexpr int VPL = 2;                      // 16-byte vectors per lane and operand
        constexpr int LPO = RUN / (4 * VPL);        // lanes per output
        constexpr int NGQ = GEO::NT / LPO;          // outputs in flight per trip of the workgroup
        constexpr int NIT = BM * BN / NGQ;          // trips
        constexpr int DEPTH = NIT % 8 == 0 ? 4 : NIT % 4 == 0 ? 2 : 1;   // outputs per lane group whose loads are issued together
        static_assert(BM * BN % NGQ == 0 && NIT % (2 * DEPTH) == 0, "whole batches");
        const int sub = tid % LPO, gq = tid / LPO;
        const int shift = (tid & 63) - sub;         // bit of this lane group's first lane in a ballot
        const float* xg = input + (size_t)g * K;
        const float* wg = weight + (size_t)g * d.NG * K;
        // element offsets fit 32 bits: the entry point rejects tensors of 2^31 elements or more
        const unsigned ldx = (unsigned)d.G * K;
        // output gq of trip 0, then NGQ further per trip: tile row, tile column and the element offsets of both rows
        int ml = gq / BN, nl = gq % BN;
        unsigned xrow = (unsigned)(m0 + ml) * ldx, wrow = (unsigned)(n0 + nl) * (unsigned)K;
        const unsigned xrow_last = (unsigned)(d.M - 1) * ldx, wrow_last = (unsigned)(d.NG - 1) * (unsigned)K;
        const unsigned wstep = (unsigned)(NGQ % BN) * (unsigned)K, wwrap = (unsigned)BN * (unsigned)K;
        struct Slot { float4 x[VPL], w[VPL]; int kb, o; };
        auto issue = [&](int it, Slot& sl) {             // called with it = 0, 1, 2, ... in this order
            if (it >= NIT) return;                       // the last trip has nothing left to prefetch
            const int o = ml * BN + nl;
            const int kb = cand_c[o] * RUN;
            // a lane whose bytes lie past the end of the row reads the chunk's first ones instead (masked
            // below); the offset must never go negative, it is added as an unsigned 32-bit quantity
            sl.kb = kb;
            sl.o = o;
            const unsigned xo = min(xrow, xrow_last), wo = min(wrow, wrow_last);
#pragma unroll
            for (int v = 0; v < VPL; v++) {
                const int kv = kb + 4 * (VPL * sub + v);
                const unsigned off = kv < K ? kv : kb;
                sl.x[v] = *reinterpret_cast<const float4*>(xg + (xo + off));
                sl.w[v] = *reinterpret_cast<const float4*>(wg + (wo + off));
            }
            ml += NGQ / BN; xrow += (NGQ / BN) * ldx;
            nl += NGQ % BN; wrow += wstep;
            if (nl >= BN) { nl -= BN; wrow -= wwrap; ml += 1; xrow += ldx; }
        };
        auto finish = [&](const Slot& sl) {
            const int o = sl.o;
            const float target = cand_v[o];
            int found = -1;                              // element index inside the lane's 4 * VPL, sign in bit 31
#pragma unroll
            for (int v = VPL - 1; v >= 0; v--) {         // descending: the lowest match is kept
                const float dd[4] = {sl.x[v].x - sl.w[v].x, sl.x[v].y - sl.w[v].y, sl.x[v].z - sl.w[v].z, sl.x[v].w - sl.w[v].w};
                const bool inside = sl.kb + 4 * (VPL * sub + v) < K;
#pragma unroll
                for (int e = 3; e >= 0; e--)
                    if (__builtin_fabsf(dd[e]) == target && inside) found = (4 * v + e) | (__float_as_int(dd[e]) & 0x80000000);
            }
            const bool hit = found != -1 && target > 0.f;
            const unsigned mine = (unsigned)(__builtin_amdgcn_ballot_w64(hit) >> shift) & ((1u << LPO) - 1);
            if (hit && (mine & ((1u << sub) - 1)) == 0) cand_c[o] = found + sl.kb + 4 * VPL * sub;   // adds to the low bits only
            if (sub == 0 && mine == 0) cand_c[o] = 0;
        };
        Slot sa[DEPTH], sb[DEPTH];
#pragma unroll
        for (int e = 0; e < DEPTH; e++) issue(e, sa[e]);
#pragma unroll 1
        for (int it = 0; it < NIT; it += 2 * DEPTH) {
#pragma unroll
            for (int e = 0; e < DEPTH; e++) issue(it + DEPTH + e, sb[e]);
#pragma unroll
            for (int e = 0; e < DEPTH; e++) finish(sa[e]);
#pragma unroll
            for (int e = 0; e < DEPTH; e++) issue(it + 2 * DEPTH + e, sa[e]);
#pragma unroll
            for (int e = 0; e < DEPTH; e++) finish(sb[e]);
        }
    } else {
        // Other layouts: every lane takes outputs tid, tid + NT, ... of the tile on its own.
#pragma unroll 1
        for (int o = tid; o < BM * BN; o += GEO::NT) {
            const int ml = CONV ? o % BM : o / BN, nl = CONV ? o / BM : o % BN;
            const int m = m0 + ml, n = n0 + nl;
            const float v = cand_v[o];
            int p = 0;
            if (m < d.M && n < d.NG && v > 0.f) {
                const RowAddr<CONV> ra(d, m, g);
                const float* wr = weight + ((size_t)g * d.NG + n) * K;
                if constexpr (EXACT) {
                    const int k = cand_c[o];  // only the sign of the difference is missing
                    const float df = input[ra.x + (size_t)k * ra.xk] - wr[k];
                    p = k | (__float_as_int(df) & 0x80000000);
                } else {
                    const int kb = cand_c[o] * kChunk;
                    p = locate_in_chunk<false>(input + ra.x + (size_t)kb * ra.xk, ra.xk, wr + kb, min(kChunk, K - kb),
                                               v, kb);
                }
            }
            cand_c[o] = p;
        }
    }
    __syncthreads();

    // Tile -> global.  Groups of four along the contiguous axis (n for fc, the row index for conv)
    // go out as one 128-bit store where the tensor allows it (d.ovec: bases 16-byte aligned and
    // NG % 4 == 0, resp. HW % 4 == 0 which keeps four rows inside one image).
    constexpr int CW = CONV ? BM : BN;              // tile extent along the contiguous axis
    static_assert(CW % 4 == 0, "");
#pragma unroll 1
    for (int q = tid; q < BM * BN / 4; q += GEO::NT) {
        const int outer = q / (CW / 4), inner = (q % (CW / 4)) * 4;
        const int ml = CONV ? inner : outer, nl = CONV ? outer : inner;
        const int m = m0 + ml, n = n0 + nl;
        if (m >= d.M || n >= d.NG) continue;
        const float4 v4 = *reinterpret_cast<const float4*>(cand_v + 4 * q);
        const int4 p4 = *reinterpret_cast<const int4*>(cand_c + 4 * q);
        const float vs[4] = {v4.x, v4.y, v4.z, v4.w};
        const int ps[4] = {p4.x, p4.y, p4.z, p4.w};
        if constexpr (!CONV) {
            const size_t at = ((size_t)m * d.G + g) * d.NG + n;
            if (d.ovec && n + 3 < d.NG) {
                *reinterpret_cast<float4*>(output + at) = v4;
                *reinterpret_cast<int4*>(pos + at) = p4;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < d.NG) { output[at + e] = vs[e]; pos[at + e] = ps[e]; }
            }
        } else {
            if (d.ovec && m + 3 < d.M) {
                const int b = m / d.HW, hw = m % d.HW;
                const size_t at = ((size_t)(b * d.G + g) * d.NG + n) * d.HW + hw;
                *reinterpret_cast<float4*>(output + at) = v4;
                *reinterpret_cast<int4*>(pos + at) = p4;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (m + e < d.M) {
                        const int b = (m + e) / d.HW, hw = (m + e) % d.HW;
                        const size_t at = ((size_t)(b * d.G + g) * d.NG + n) * d.HW + hw;
                        output[at] = vs[e];
                        pos[at] = ps[e];
                    }
            }
        }
    }
}

// Above this K the chunk re-read is cheaper than tracking k in the loop (conv layout).
constexpr int kExactMaxK = 1024;
// Up to this K the fc kernel records halves of a chunk: the loop runs about 10 % longer for it, the search after the
// loop (whose cost hardly depends on K) takes half as long.  Measured on 512 x K -> 5120: K = 784 120 against 128 us,
// K = 2048 a loss.
constexpr int kHalfMaxK = 1024;

template <class GEO, bool CONV, int VEC>
struct InfForward {
    template <bool EXACT, bool HALF = false>
    static hipError_t go(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* input,
                         const float* weight, float* output, int32_t* pos) {
        // pipeline buffers, or the tile's (value, chunk) parking area of the epilogue if larger
        constexpr size_t park = (size_t)GEO::BM * GEO::BN * 2 * sizeof(float);
        constexpr size_t pipe = Stager<GEO, CONV, VEC, 1>::LDS_BYTES;
        const size_t lds = park > pipe ? park : pipe;
        auto kern = inf_forward_kernel<GEO, CONV, VEC, EXACT, HALF>;
        static LdsRecord lds_allowed = {};   // per instantiation of this launcher, i.e. per kernel
        if (hipError_t e = allow_lds(kern, lds, device, lds_allowed); e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(GEO::NT), lds, stream, input, weight, output, pos, d);
        return hipGetLastError();
    }
    static hipError_t launch(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* input,
                             const float* weight, float* output, int32_t* pos) {
        if constexpr (CONV) {
            if (d.K <= kExactMaxK) return go<true>(grid, d, device, stream, input, weight, output, pos);
        }
        if constexpr (!CONV && VEC == 4) {
            if (d.K <= kHalfMaxK) return go<false, true>(grid, d, device, stream, input, weight, output, pos);
        }
        return go<false>(grid, d, device, stream, input, weight, output, pos);
    }
};

// ---------------------------------------------------------------------------
// Values only (no pos): what a forward pass that no gradient will follow needs -- evaluation, and the value path of
// a certification pass.  The reference always computes pos (model/norm_dist.py:14-15, inf_dist_cuda.cu:36-43); without
// it the loop is one v_sub_f32 and half a v_max3_f32 per (row, output, input) and nothing else: no second register
// array, no chunk records, and no search after the loop (which is a twelfth of the full kernel's launch at K = 5120
// and a third at K = 784).  The k-groups meet in LDS and the first writes the tile.  Same subtractions and maxima
// of the same numbers: the values are those of inf_forward_kernel bit for bit.  fc layout with 128-bit loads.
// ---------------------------------------------------------------------------
template <class GEO>
__global__ void __launch_bounds__(GEO::NT, 2)
inf_forward_values_kernel(const float* __restrict__ input, const float* __restrict__ weight, float* __restrict__ output,
                          Dims d) {
    constexpr int BM = GEO::BM, BN = GEO::BN, TM = GEO::TM, TN = GEO::TN, KS = GEO::KS, KK = GEO::KK;
    constexpr int NGRP = GEO::NGRP;
    using Stage = Stager<GEO, false, 4, 1>;
    constexpr int STAGE = Stage::STAGE, NBUF = Stage::NBUF;
    static_assert((KS - 1) * TM * TN * NGRP <= NBUF * STAGE, "merge area fits in the panels");
    extern __shared__ __align__(16) float lds[];

    int tm, tn, g;
    tile_of_block(d, tm, tn, g);
    const int m0 = tm * BM, n0 = tn * BN;
    const int tid = threadIdx.x;
    const int grp = tid / NGRP, t = tid % NGRP;
    const int tx = t % GEO::TX, ty = t / GEO::TX;

    Stage st;
    const float* const ins[1] = {input};
    st.init(ins, weight, d, m0, n0, g, tid);
    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = 0.f;

    const int nstage = (d.K + KK - 1) / KK;
    st.load(0);
    st.store(lds);
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        const float* stage = lds + (s % NBUF) * STAGE;
        if (s + 1 < nstage) st.load((s + 1) * KK);
        sweep_chunk<GEO, 1, 2, true>(stage + grp * kChunk * GEO::SM, stage + GEO::XS + grp * kChunk * GEO::SN, tx, ty,
                                     [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const float d0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]);
                    const float d1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]);
                    acc[i][j] = __builtin_fmaxf(__builtin_fmaxf(acc[i][j], d0), d1);
                }
        });
        if (NBUF == 1) __syncthreads();
        if (s + 1 < nstage) st.store(lds + ((s + 1) % NBUF) * STAGE);
        __syncthreads();
    }
    if constexpr (KS > 1) {   // the other k-groups hand their maxima to the first
        float* part = lds;    // [KS-1][TM*TN][NGRP]
        if (grp > 0) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) part[((grp - 1) * TM * TN + i * TN + j) * NGRP + t] = acc[i][j];
        }
        __syncthreads();
        if (grp > 0) return;
#pragma unroll
        for (int q = 0; q < KS - 1; q++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_fmaxf(acc[i][j], part[(q * TM * TN + i * TN + j) * NGRP + t]);
    }
    store_patch<GEO, false>(output, acc, d, m0, n0, g, tx, ty, d.ovec != 0);
}

template <class GEO>
static hipError_t launch_values(const Problem& pr, bool ovec, hipStream_t stream, const float* input, const float* weight,
                                float* output) {
    Dims d = make_dims(pr);
    d.ovec = ovec;
    d.tiles_m = (d.M + GEO::BM - 1) / GEO::BM;
    d.tiles_n = (d.NG + GEO::BN - 1) / GEO::BN;
    const size_t lds = Stager<GEO, false, 4, 1>::LDS_BYTES;
    d.m_block = choose_m_block(d.tiles_m, GEO::BM, GEO::BN, resident_per_xcd(GEO::NT, lds, pr.num_cu));
    auto kern = inf_forward_values_kernel<GEO>;
    static LdsRecord lds_allowed = {};
    if (hipError_t e = allow_lds(kern, lds, pr.device, lds_allowed); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)d.tiles_m * d.tiles_n * d.G), dim3(GEO::NT), lds, stream, input, weight,
                       output, d);
    return hipGetLastError();
}

// The shapes the values-only kernel takes: the fc layout with 128-bit loads and more than a handful of outputs per
// group (the skinny kernels serve those, and pos costs them nothing).  Everything else computes pos as well.
bool inf_forward_values_applicable(const Problem& pr, const void* input, const void* weight) {
    return pr.HW == 1 && pr.NG > kSkinnyMaxNG && can_vec4(pr, input, weight);
}

hipError_t inf_forward_values(const float* input, const float* weight, float* output, const Problem& pr,
                              hipStream_t stream) {
    const bool ovec = can_vec4_out(pr, output);
    if (g_tile_override == 4) return launch_values<Geo<64, 80, 8, 5, 2>>(pr, ovec, stream, input, weight, output);
    switch (choose_tile(pr.B, pr.NG, pr.G, pr.num_cu)) {
        case TileChoice::M128N80K2:
            // as in inf_forward(): two 256-lane workgroups per CU where one 512-lane workgroup would be chosen
            if (pr.B > 64 && g_tile_override < 0) return launch_values<Geo<64, 80, 8, 5, 2>>(pr, ovec, stream, input, weight, output);
            return launch_values<Geo<128, 80, 8, 5, 2>>(pr, ovec, stream, input, weight, output);
        case TileChoice::M256N32K1: return launch_values<Geo<256, 32, 8, 4, 1>>(pr, ovec, stream, input, weight, output);
        case TileChoice::M32N32K8: return launch_values<Geo<32, 32, 4, 4, 8>>(pr, ovec, stream, input, weight, output);
        default: return launch_values<Geo<128, 64, 8, 4, 1>>(pr, ovec, stream, input, weight, output);
    }
}

// ---------------------------------------------------------------------------
// Few outputs per group (the 10-way classification head): a workgroup takes RW
// rows m of one group, its 256 lanes split k, each lane keeps the exact
// (value, k) pair per (row, output), and the pairs are reduced with "larger
// value, then lower k" first inside each wave, then across the four waves
// through LDS.  Bound by reading x once and w from L2.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void take_better(float& v, int& p, float ov, int op) {
    if (ov > v || (ov == v && (op & 0x7fffffff) < (p & 0x7fffffff))) { v = ov; p = op; }
}

// Within a lane k ascends (see skinny_sweep), so the strict comparison keeps the lowest k of a tie.
template <int RW, int NB, bool VEC>
__global__ void __launch_bounds__(256)
inf_forward_skinny_kernel(const float* __restrict__ input, const float* __restrict__ weight,
                          float* __restrict__ output, int32_t* __restrict__ pos, Dims d) {
    __shared__ float sv[4][RW * NB];
    __shared__ int sp[4][RW * NB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    SkinnyRows<RW> rows;
    rows.init(d);
    for (int nb = 0; nb < d.NG; nb += NB) {
        float best[RW][NB];
        int bp[RW][NB];
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int j = 0; j < NB; j++) { best[r][j] = 0.f; bp[r][j] = 0; }
        // The walk is spelled out here instead of going through skinny_sweep: with the four k of a 128-bit load
        // innermost (per row and output) the compare-and-select chains came out a third faster (24 against 38 us
        // on 512 x 5120 -> 10) than with k outermost.
        const int K = d.K;
        if constexpr (VEC) {
            for (int k = tid * 4; k < K; k += 1024) {
                float4 xv[RW], wv[NB];
#pragma unroll
                for (int r = 0; r < RW; r++) xv[r] = *reinterpret_cast<const float4*>(input + rows.xoff[r] + k);
#pragma unroll
                for (int j = 0; j < NB; j++)
                    wv[j] = *reinterpret_cast<const float4*>(weight + ((size_t)rows.g * d.NG + min(nb + j, d.NG - 1)) * K + k);
#pragma unroll
                for (int r = 0; r < RW; r++)
#pragma unroll
                    for (int j = 0; j < NB; j++) {
                        const float df[4] = {xv[r].x - wv[j].x, xv[r].y - wv[j].y, xv[r].z - wv[j].z, xv[r].w - wv[j].w};
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float a = __builtin_fabsf(df[e]);
                            if (a > best[r][j]) { best[r][j] = a; bp[r][j] = (k + e) | (__float_as_int(df[e]) & 0x80000000); }
                        }
                    }
            }
        } else {
            const int xk = d.HW;
            for (int k = tid; k < K; k += 256) {
                float xv[RW], wv[NB];
#pragma unroll
                for (int r = 0; r < RW; r++) xv[r] = input[rows.xoff[r] + (size_t)k * xk];
#pragma unroll
                for (int j = 0; j < NB; j++) wv[j] = weight[((size_t)rows.g * d.NG + min(nb + j, d.NG - 1)) * K + k];
#pragma unroll
                for (int r = 0; r < RW; r++)
#pragma unroll
                    for (int j = 0; j < NB; j++) {
                        const float df = xv[r] - wv[j];
                        const float a = __builtin_fabsf(df);
                        if (a > best[r][j]) { best[r][j] = a; bp[r][j] = k | (__float_as_int(df) & 0x80000000); }
                    }
            }
        }
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int j = 0; j < NB; j++) {
                float v = best[r][j];
                int p = bp[r][j];
                wave_best(v, p);
                if (lane == 63) { sv[wave][r * NB + j] = v; sp[wave][r * NB + j] = p; }
            }
        __syncthreads();
        if (tid < RW * NB) {
            float v = sv[0][tid];
            int p = sp[0][tid];
#pragma unroll
            for (int q = 1; q < 4; q++) take_better(v, p, sv[q][tid], sp[q][tid]);
            const int r = tid / NB, j = tid % NB;
            if (rows.m0 + r < d.M && nb + j < d.NG) {
                output[rows.ooff[r] + (size_t)(nb + j) * d.HW] = v;
                pos[rows.ooff[r] + (size_t)(nb + j) * d.HW] = v > 0.f ? p : 0;
            }
        }
        __syncthreads();
    }
}

hipError_t inf_forward(const float* input, const float* weight, float* output, int32_t* pos, const Problem& pr,
                       hipStream_t stream) {
    if (pr.NG <= kSkinnyMaxNG) {
        const Dims d = make_dims(pr);
        const bool vec = pr.HW == 1 && pr.K % 4 == 0 && aligned16(input) && aligned16(weight);
#define LDIST_LAUNCH_RW(RW, NB, VEC)                                                                                       \
    hipLaunchKernelGGL((inf_forward_skinny_kernel<RW, NB, VEC>), dim3(skinny_grid(d, RW)), dim3(256), 0, stream, input, \
                       weight, output, pos, d)
        // two rows per workgroup share the weight loads; with few rows (up to eight per CU) one each: more workgroups hide more latency
#define LDIST_LAUNCH_1(NB, VEC) LDIST_LAUNCH_RW(1, NB, VEC)
#define LDIST_LAUNCH_2(NB, VEC) LDIST_LAUNCH_RW(2, NB, VEC)
        if ((long)d.M * d.G <= 8L * pr.num_cu) LDIST_SKINNY_DISPATCH(pr.NG, vec, LDIST_LAUNCH_1);
        else LDIST_SKINNY_DISPATCH(pr.NG, vec, LDIST_LAUNCH_2);
#undef LDIST_LAUNCH_1
#undef LDIST_LAUNCH_2
#undef LDIST_LAUNCH_RW
        return hipGetLastError();
    }
    // unfolded-conv layout with a short reduction: the kernel that keeps the whole K of a tile in LDS
    if (g_tile_override < 0 && inf_forward_shortk_applicable(pr, input, output, pos))
        return inf_forward_shortk(input, weight, output, pos, pr, stream);
    const bool vec4 = can_vec4(pr, input, weight), ovec = can_vec4_out(pr, output, pos);
    // fc layout: where the 128 x 80 tiles (one 512-lane workgroup per CU) would be chosen, tiles of 64 x 80 with 256
    // lanes run two workgroups per CU instead.  Same patch per lane, same two waves per SIMD, but the two workgroups
    // drift apart, so one's epilogue (no arithmetic: merge, argmax search, stores) runs beside the other's k loop.
    if (pr.HW == 1 && vec4 &&
        (g_tile_override == 4 ||
         (g_tile_override < 0 && pr.B > 64 && choose_tile(pr.B, pr.NG, pr.G, pr.num_cu) == TileChoice::M128N80K2))) {
        using G64 = Geo<64, 80, 8, 5, 2>;
        Dims d = make_dims(pr);
        d.ovec = ovec;
        d.tiles_m = (d.M + G64::BM - 1) / G64::BM;
        d.tiles_n = (d.NG + G64::BN - 1) / G64::BN;
        d.m_block = choose_m_block(d.tiles_m, G64::BM, G64::BN,
                                   resident_per_xcd(G64::NT, Stager<G64, false, 4, 1>::LDS_BYTES, pr.num_cu));
        return InfForward<G64, false, 4>::launch((unsigned)d.tiles_m * d.tiles_n * d.G, d, pr.device, stream, input, weight,
                                                 output, pos);
    }
    return dispatch_forward<InfForward>(pr, vec4, ovec, stream, input, weight, output, pos);
}

}  // namespace ldist

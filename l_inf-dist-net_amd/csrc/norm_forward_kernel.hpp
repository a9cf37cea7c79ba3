// The register-tiled p-norm forward kernel and its launcher, shared by the column entry point (norm_forward.hip)
// and the one that reads the image of a convolution-shaped layer (norm_conv.hip).
#pragma once
#include "fwd_engine.hpp"
#include "pow.hpp"
#include "wave_reduce.hpp"

namespace ldist {

// Largest exponent for the one-sweep kernel.  A chunk goes back the long way once it exceeds the
// scale by 10^(30/p): a factor of 70 at p = 16, 2.9 at p = 64, still 1.7 at p = 128, which later chunks
// (the scale is the maximum of all chunks before) rarely do: on 512 x 5120 -> 5120 one sweep takes 3.08 ms
// for any p from 37 to 127, against 3.4 ms for sweeping every chunk twice.  A general-p term is a logarithm
// and an exponential, and 13.4 G of them in 3.08 ms is 89 % of what the transcendental unit issues.
constexpr float kOneSweepMaxP = 127.99f;

// Exponents from which the forward runs its two passes with tests (MODE 2).  With normally distributed
// differences over 5120 inputs it overtakes the chunk-by-chunk kernel at p of about 120.
constexpr float kForwardSparseMinP = 128.f;


// IP: the exponent when it is one of the multiply-only cases (2, 3, 4, 8), else 0.  A template
// parameter rather than a run-time switch: one kernel holding all five power sweeps next to
// the maximum sweep pushed the hot loops into scratch.
//
// MODE 1 (p <= kOneSweepMaxP): a chunk is swept once.  Any scale s gives the same result,
// out = s * (sum_k (|x-w|/s)^p)^(1/p); the maximum only keeps the powers in range.  So a chunk
// adds (|x-w| / s)^p with the scale s left by earlier chunks, and only a wave that sees a chunk
// sum overflow (or turn NaN) goes back over that chunk the long way: find its maximum, move
// the scale there as the reference does, add the powers again.  The first chunk always takes
// that road (the scale starts at the reference's seed 1e-10).  MODE 0: every chunk is swept twice
// (maximum, then powers), for exponents so large that almost any increase would overflow.
// MODE 2 (p >= kForwardSparseMinP): two passes over all of k, the second with tests that skip the powers
// of negligible terms; described where it starts below.
//
// IMG: `input` is the image of a convolution-shaped layer (3x3 window, geometry in `win`) and the input panel is
// gathered from it; d describes the unfolded problem (K = 9 channels-per-group, HW = output positions).
template <class GEO, bool CONV, int VEC, int IP, int MODE, bool IMG>
__global__ void __launch_bounds__(GEO::NT, 2)
norm_forward_kernel(const float* __restrict__ input, const float* __restrict__ weight, float* __restrict__ output,
                    float p, Dims d, ImgWin win) {
    constexpr int BM = GEO::BM, BN = GEO::BN, TM = GEO::TM, TN = GEO::TN, KS = GEO::KS, KK = GEO::KK;
    constexpr int NGRP = GEO::NGRP;
    using Stage = Stager<GEO, CONV, VEC, 1, IMG>;
    constexpr int STAGE = Stage::STAGE, NBUF = Stage::NBUF;
    static_assert(2 * (KS - 1) * TM * TN * NGRP <= NBUF * STAGE, "merge area fits in the panels");
    extern __shared__ __align__(16) float lds[];

    int tm, tn, g;
    tile_of_block(d, tm, tn, g);
    const int m0 = tm * BM, n0 = tn * BN;
    const int tid = threadIdx.x;
    const int grp = tid / NGRP, t = tid % NGRP;
    const int tx = t % GEO::TX, ty = t / GEO::TX;
    const float pv = in_vgpr(p);
    auto power = [&](float v) {   // by reference: the integer-exponent instantiations do not use p
        if constexpr (IP > 0) return pow_int<IP>(v);
        else return pow_pos(v, pv);
    };
    // General exponent, one sweep (MODE 1): the scale of an output is kept as ls = p * log2(1 / scale) and a term
    // (|x - w| / scale)^p is exp2(p * log2|x - w| + ls): the division by the scale rides in the fused multiply-add of
    // the exponent (three plain instructions per term beside the logarithm and the exponential instead of four:
    // 2.97 -> 2.65 ms on 512 x 5120 -> 5120 at p = 20.5).  Any scale gives the same result as long as the sum and the
    // final multiplication use the same one, and here both are defined by ls; what the form costs is the rounding
    // of an exponent that is a difference of two numbers of the size of p * |log2 scale|: a relative error of
    // about 1e-7 * |log2 scale| in the output, 9e-6 for data of the size of 1e30.  So the kernel works in units of a
    // power of two read off the workgroup's first stage (the largest |x| or |w| there; every stage's panels are
    // scaled by its reciprocal on their way into LDS, which is exact, and the outputs multiplied by it at the end):
    // log2 scale is then small whatever the magnitude of the data, unless the differences are orders of magnitude
    // smaller than the values themselves.  The unit follows the scales: at the end of a stage every wave leaves the
    // largest scale among its outputs in LDS, after the stage's barrier everybody reads the workgroup's largest, and
    // when that is 2^8 or more away from the unit, the panels stored from then on (those of the stage after next:
    // the next one is in LDS already) are taken in the new unit, and every ls moves by p times the change of exponent
    // when their stage begins.  Data whose magnitude runs away along k costs accuracy for two stages' growth only.
    constexpr bool LOGS = IP == 0 && MODE == 1;
    int ue_cur = 0, ue_next = 0;   // exponents of the unit: of the stage being reduced / of the panels stored next
    __shared__ float wave_ls[LOGS ? 2 : 1][LOGS ? GEO::NT / 64 : 1];   // the smallest ls (largest scale) of each wave, by stage parity
    auto log_term = [&](float df, float ls) {   // (|df| / scale)^p; df == 0: exp2(-inf) = 0
        return __builtin_amdgcn_exp2f(__builtin_fmaf(__builtin_amdgcn_logf(__builtin_fabsf(df)), pv, ls));
    };

    Stage st;
    const float* const ins[1] = {input};
    if constexpr (IMG) st.win = win;
    st.init(ins, weight, d, m0, n0, g, tid);

    // acc = sum of (|x-w| * rs)^p over the k seen so far; rs = 1 / scale (LOGS: rs holds ls = p * log2(1 / scale)
    // instead).  Seeds as in the reference.
    float acc[TM][TN], rs[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) { acc[i][j] = grp == 0 ? 1e-10f : 0.f; rs[i][j] = LOGS ? p * 33.21928095f : 1e10f; }   // LOGS: rs holds ls

    const int nstage = (d.K + KK - 1) / KK;
    if constexpr (MODE == 2) {
        // Large p, two passes over all of k.  Pass one finds every output's maximum, which becomes its scale.  In pass
        // two a normalised difference u below  cut = 2^(-32/p)  has a power below 2^-32, nothing against a sum that
        // holds the maximum's own 1 -- and nearly all differences are that small, while the logarithm and the
        // exponential are most of a term's cost.  So pass two only takes the largest u per row of the lane's patch
        // (a subtraction, a multiplication and half a v_max3 per term), and the powers of a row are taken only when
        // some lane of the wave has a u above the cut in it.  The rows are tested one by one only after a test of
        // the whole fragment: every test makes a branch wait for the vector unit.
        auto all_stages = [&](auto&& body) {
            st.load(0);
            st.store(lds);
            __syncthreads();
            for (int s = 0; s < nstage; s++) {
                const float* stage = lds + (s % NBUF) * STAGE;
                if (s + 1 < nstage) st.load((s + 1) * KK);
                body(stage + grp * kChunk * GEO::SM, stage + GEO::XS + grp * kChunk * GEO::SN, s);
                if (NBUF == 1) __syncthreads();
                if (s + 1 < nstage) st.store(lds + ((s + 1) % NBUF) * STAGE);
                __syncthreads();
            }
        };
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) rs[i][j] = 0.f;   // the maximum, until pass one is over
        all_stages([&](const float* xp, const float* wp, int) {
            sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float d0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]);
                        const float d1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]);
                        rs[i][j] = __builtin_fmaxf(__builtin_fmaxf(rs[i][j], d0), d1);
                    }
            });
        });
        // An output that stays on the seed scale 1e-10 has a sum of about 1e-10, not of at least 1: nothing is
        // negligible against that, so a lane that holds one takes every power (its cut is below every u).
        float cut = __builtin_exp2f(-32.0f / p);
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const bool seeded = !(rs[i][j] > 1e-10f);
                rs[i][j] = seeded ? 1e10f : __builtin_amdgcn_rcpf(rs[i][j]);
                if (grp == 0) acc[i][j] = 1e-10f * pow_pos(1e-10f * rs[i][j], pv);   // the seed, on the final scale
                if (seeded) cut = -1.f;
            }
        // Where most rows do hold a term that counts (moderate p, or differences that crowd below their maximum) the
        // tests only cost: a wave that took the powers of more than 85 % of a stage's rows sweeps the next seven
        // stages without tests, then probes again.
        constexpr int ROWS_PER_STAGE = kChunk / 2 * TM;
        int taken = 0;   // rows whose powers this wave took in the last tested stage (the same in every lane)
        all_stages([&](const float* xp, const float* wp, int s) {
            if (taken * 20 > ROWS_PER_STAGE * 17 && (s & 7) != 0) {
                sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            acc[i][j] += pow_pos(__builtin_fabsf(f.x[0][0][i] - f.w[0][j]) * rs[i][j], pv);
                            acc[i][j] += pow_pos(__builtin_fabsf(f.x[0][1][i] - f.w[1][j]) * rs[i][j], pv);
                        }
                });
                return;
            }
            taken = 0;
            sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int) {
                float top[TM], all = 0.f;
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    top[i] = 0.f;
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float u0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]) * rs[i][j];
                        const float u1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]) * rs[i][j];
                        top[i] = __builtin_fmaxf(__builtin_fmaxf(top[i], u0), u1);
                    }
                    all = __builtin_fmaxf(all, top[i]);
                }
                if (__builtin_amdgcn_ballot_w64(all > cut) != 0) {
#pragma unroll
                    for (int i = 0; i < TM; i++)
                        if (__builtin_amdgcn_ballot_w64(top[i] > cut) != 0) {
                            taken++;
                            // the differences are taken again: kept from the tests they would hold eighty registers
                            float x0 = f.x[0][0][i], x1 = f.x[0][1][i];
                            asm volatile("" : "+v"(x0), "+v"(x1));
#pragma unroll
                            for (int j = 0; j < TN; j++) {
                                acc[i][j] += pow_pos(__builtin_fabsf(x0 - f.w[0][j]) * rs[i][j], pv);
                                acc[i][j] += pow_pos(__builtin_fabsf(x1 - f.w[1][j]) * rs[i][j], pv);
                            }
                        }
                }
            });
        });
    } else {
    st.load(0);
    if constexpr (LOGS) {
        float top = 0.f;   // the largest finite magnitude this lane loaded
        st.for_each_parked([&](float& v) {
            const float a = __builtin_fabsf(v);
            top = __builtin_fmaxf(top, a < __builtin_inff() ? a : 0.f);   // a NaN is not taken either
        });
        top = wave_max(top);
        if ((tid & 63) == 63) lds[tid >> 6] = top;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < GEO::NT / 64; w++) top = __builtin_fmaxf(w == 0 ? lds[0] : top, lds[w]);
        __syncthreads();   // before the panels overwrite those words
        if (top > 0.f) ue_cur = ue_next = min(100, max(-100, (int)((__float_as_uint(top) >> 23) & 0xff) - 127));
        // the reference's seed scale 1e-10, in units
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) rs[i][j] = p * (33.21928095f + (float)ue_cur);
        const float unit_inv = __uint_as_float((unsigned)(127 - ue_next) << 23);
        st.for_each_parked([&](float& v) { v *= unit_inv; });
    }
    st.store(lds);
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        const float* stage = lds + (s % NBUF) * STAGE;
        if (s + 1 < nstage) st.load((s + 1) * KK);
        if constexpr (LOGS) {
            // ue_cur: exponent of the unit of the panels reduced in this stage; ue_next: of those stored at its end
            const int moved = ue_next - ue_cur;   // from the last stage's unit to this one's
            if (moved != 0) {
                const float by = pv * (float)moved;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) rs[i][j] += by;
            }
            ue_cur = ue_next;
            if (s > 0) {   // the largest scale at the end of the last stage, in this stage's unit
                float low = wave_ls[(s - 1) & 1][0];
#pragma unroll
                for (int w = 1; w < GEO::NT / 64; w++) low = __builtin_fminf(low, wave_ls[(s - 1) & 1][w]);
                const float e2 = -(low + pv * (float)moved) * __builtin_amdgcn_rcpf(pv);   // log2(largest scale / unit)
                if (e2 >= 8.f || e2 <= -8.f)   // (a NaN changes nothing)
                    ue_next = min(100, max(-100, ue_cur + (int)__builtin_floorf(__builtin_fminf(__builtin_fmaxf(e2, -200.f), 200.f))));
            }
        }
        const float* xp = stage + grp * kChunk * GEO::SM;
        const float* wp = stage + GEO::XS + grp * kChunk * GEO::SN;
        float cs[TM][TN];  // chunk maximum, or chunk sum
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) cs[i][j] = 0.f;
        // moves the scale of every output whose chunk maximum (in cs) exceeds it
        auto raise_scale = [&]() {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    if constexpr (LOGS) {
                        const float lm = pv * __builtin_amdgcn_logf(cs[i][j]);   // p * log2(chunk maximum); -inf for 0
                        const float up = lm + rs[i][j];                           // p * log2(maximum / scale)
                        if (up > 0.f) {
                            acc[i][j] *= __builtin_amdgcn_exp2f(-up);
                            rs[i][j] = -lm;
                        }
                    } else {
                        const float r = cs[i][j] * rs[i][j];
                        if (r > 1.f) {
                            acc[i][j] *= pow_pos(__builtin_amdgcn_rcpf(r), pv);
                            rs[i][j] = __builtin_amdgcn_rcpf(cs[i][j]);
                        }
                    }
                    cs[i][j] = 0.f;
                }
        };
        if constexpr (MODE == 1) {
            bool redo = false;
            if constexpr (IP > 0) {
                // Small integer p: sum the raw powers |x-w|^p and multiply the chunk sum by rs^p afterwards, which
                // saves the multiplication by rs per term (5 instead of 6 instructions at p = 8; even powers need no
                // absolute value).  Both factors must stay well inside the float range: every scale of the wave
                // within 2^(+-96/p) (p = 8: distances between 2.4e-4 and 4096).  Outside -- the seed scale of the
                // first chunk included -- and whenever the sum overflows, the chunk takes the careful path below.
                constexpr float HI = IP == 2 ? 0x1p48f : IP == 3 ? 0x1p32f : IP == 4 ? 0x1p24f : 0x1p12f;
                bool wide = false;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) wide |= !(rs[i][j] <= HI && rs[i][j] >= 1.0f / HI);
                if (__builtin_amdgcn_ballot_w64(wide) == 0) {
                    auto raw = [](float df) { return IP % 2 == 0 ? pow_int<IP>(df) : pow_int<IP>(__builtin_fabsf(df)); };
                    sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                        for (int i = 0; i < TM; i++)
#pragma unroll
                            for (int j = 0; j < TN; j++) {
                                cs[i][j] += raw(f.x[0][0][i] - f.w[0][j]);
                                cs[i][j] += raw(f.x[0][1][i] - f.w[1][j]);
                            }
                    });
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            cs[i][j] *= pow_int<IP>(rs[i][j]);
                            redo |= !(cs[i][j] < 1e30f);
                        }
                } else {
                    redo = true;
                }
            } else {
                sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            cs[i][j] += log_term(f.x[0][0][i] - f.w[0][j], rs[i][j]);
                            cs[i][j] += log_term(f.x[0][1][i] - f.w[1][j], rs[i][j]);
                        }
                });
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) redo |= !(cs[i][j] < 1e30f);
            }
            if (__builtin_amdgcn_ballot_w64(redo) != 0) {   // rare: kept lean, no operand prefetch
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) cs[i][j] = 0.f;
                sweep_chunk_plain<GEO, 1>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 1>& f, int) {
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++)
                            cs[i][j] = __builtin_fmaxf(cs[i][j], __builtin_fabsf(f.x[0][0][i] - f.w[0][j]));
                });
                raise_scale();
                sweep_chunk_plain<GEO, 1>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 1>& f, int) {
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) {
                            if constexpr (LOGS) cs[i][j] += log_term(f.x[0][0][i] - f.w[0][j], rs[i][j]);
                            else cs[i][j] += power(__builtin_fabsf(f.x[0][0][i] - f.w[0][j]) * rs[i][j]);
                        }
                });
            }
        } else {
            sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float d0 = __builtin_fabsf(f.x[0][0][i] - f.w[0][j]);
                        const float d1 = __builtin_fabsf(f.x[0][1][i] - f.w[1][j]);
                        cs[i][j] = __builtin_fmaxf(__builtin_fmaxf(cs[i][j], d0), d1);
                    }
            });
            raise_scale();
            sweep_chunk<GEO, 1, 2>(xp, wp, tx, ty, [&](const Frag<GEO, 1, 2>& f, int) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        cs[i][j] += power(__builtin_fabsf(f.x[0][0][i] - f.w[0][j]) * rs[i][j]);
                        cs[i][j] += power(__builtin_fabsf(f.x[0][1][i] - f.w[1][j]) * rs[i][j]);
                    }
            });
        }
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) acc[i][j] += cs[i][j];
        if (NBUF == 1) __syncthreads();  // everyone is done reading the only buffer
        if (s + 1 < nstage) {
            if constexpr (LOGS) {
                float low = rs[0][0];
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) low = __builtin_fminf(low, rs[i][j]);
                low = -wave_max(-low);
                if ((tid & 63) == 63) wave_ls[s & 1][tid >> 6] = low;
                const float unit_inv = __uint_as_float((unsigned)(127 - ue_next) << 23);
                st.for_each_parked([&](float& v) { v *= unit_inv; });
            }
            st.store(lds + ((s + 1) % NBUF) * STAGE);
        }
        __syncthreads();
    }
    }

    // Merge the k-groups onto the larger scale.
    if constexpr (KS > 1) {
        float* ma = lds;  // [KS-1][TM*TN][NGRP] sums, then as many reciprocal scales
        float* mr = lds + (KS - 1) * TM * TN * NGRP;
        if (grp > 0) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int o = ((grp - 1) * TM * TN + i * TN + j) * NGRP + t;
                    ma[o] = acc[i][j];
                    mr[o] = rs[i][j];
                }
        }
        __syncthreads();
        if (grp > 0) return;
#pragma unroll
        for (int q = 0; q < KS - 1; q++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int o = (q * TM * TN + i * TN + j) * NGRP + t;
                    const float a2 = ma[o], r2 = mr[o];
                    const float r = __builtin_fminf(rs[i][j], r2);   // the larger scale
                    if constexpr (LOGS)
                        acc[i][j] = acc[i][j] * __builtin_amdgcn_exp2f(r - rs[i][j]) + a2 * __builtin_amdgcn_exp2f(r - r2);
                    else
                        acc[i][j] = acc[i][j] * pow_pos(r * __builtin_amdgcn_rcpf(rs[i][j]), pv) +
                                    a2 * pow_pos(r * __builtin_amdgcn_rcpf(r2), pv);
                    rs[i][j] = r;
                }
    }

    const float inv_p = 1.0f / p;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if constexpr (LOGS)
                acc[i][j] = __uint_as_float((unsigned)(127 + ue_cur) << 23) *
                            __builtin_amdgcn_exp2f((__builtin_amdgcn_logf(acc[i][j]) - rs[i][j]) * inv_p);
            else acc[i][j] = pow_pos(acc[i][j], inv_p) * __builtin_amdgcn_rcpf(rs[i][j]);
        }
    store_patch<GEO, CONV>(output, acc, d, m0, n0, g, tx, ty, d.ovec != 0);
}

template <class GEO, bool CONV, int VEC, bool IMG>
struct NormForwardLaunch {
    template <int IP, int MODE>
    static hipError_t go(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* input,
                         const float* weight, float* output, float p, const ImgWin& win) {
        const size_t lds = Stager<GEO, CONV, VEC, 1, IMG>::LDS_BYTES;
        auto kern = norm_forward_kernel<GEO, CONV, VEC, IP, MODE, IMG>;
        static LdsRecord lds_allowed = {};   // per instantiation of this launcher, i.e. per kernel
        if (hipError_t e = allow_lds(kern, lds, device, lds_allowed); e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(GEO::NT), lds, stream, input, weight, output, p, d, win);
        return hipGetLastError();
    }
    static hipError_t launch(unsigned grid, const Dims& d, int device, hipStream_t stream, const float* input,
                             const float* weight, float* output, float p, const ImgWin& win) {
        switch (small_int_power(p)) {
            case 2: return go<2, 1>(grid, d, device, stream, input, weight, output, p, win);
            case 3: return go<3, 1>(grid, d, device, stream, input, weight, output, p, win);
            case 4: return go<4, 1>(grid, d, device, stream, input, weight, output, p, win);
            case 8: return go<8, 1>(grid, d, device, stream, input, weight, output, p, win);
            default:
                // a row of the test holds 640 terms per wave and every output has one term equal to 1: K must be long
                if (p >= kForwardSparseMinP && d.K >= 2048) return go<0, 2>(grid, d, device, stream, input, weight, output, p, win);
                return p <= kOneSweepMaxP ? go<0, 1>(grid, d, device, stream, input, weight, output, p, win)
                                          : go<0, 0>(grid, d, device, stream, input, weight, output, p, win);
        }
    }
};

}  // namespace ldist

// L_inf distance layer on an image without the unfolded tensor (the reference unfolds with F.unfold,
// model/norm_dist.py:132, and then calls inf_dist_forward_cuda on the nine times larger columns):
//   out[b, g*NG + n, h*WO + w] = max_k |x_k - weight[g*NG + n, k]|,  k = (c*3 + i)*3 + j,
//   x_k = img[b, g*CG + c, h*S + i - P, w*S + j - P]   (0 outside the image),
// pos as in the column kernel (lowest k of the maximum, bit 31 = sign of the difference, 0 for a zero maximum).
// Values and indices equal the column path's bit for bit: the same fp32 subtractions of the same numbers.
//
// A workgroup owns R output rows of one (image, group) and BN of the group's outputs.  The weights stream
// through a double-buffered LDS stage of CC channels (9*CC values of k), stored k-major so that a lane's four
// outputs are one 128-bit read.  The image rows those positions look at, zero padding materialised, are in LDS
// too, in one of two ways:
//   RESIDENT  all CG channels are copied once and stay (few channels per group: they fit);
//   staged    CC channels at a time travel through a second double-buffered stage beside the weights.
// A lane owns 8 neighbouring positions of one output row times 4 outputs.  For a window row (c, i) it reads the
// 8 + 2 pixels its positions cover for j = 0, 1, 2 with three (stride 2: five) aligned 128-bit reads, so 12 LDS
// words serve 24 differences.  The loop takes the running maximum through a channel and records the channel where
// that raised it (subtract + half a v_max3 per difference, two instructions per channel and output, three in the
// staged variant); the lowest k inside the recorded channel is found afterwards from nine pixels (LDS when
// RESIDENT, else the image in global memory) and the channel's nine contiguous weights.
#include "conv_image.hpp"

namespace ldist {

int g_conv_rows_override = 0;      // > 0: output rows per workgroup forced (tests and tuning)
int g_conv_staging_override = 0;   // 1: image rows resident in LDS only; 2: staged only; 3: neither; 0: by shape

namespace {

using namespace convimg;

// POS = false: values only, for a forward pass that no gradient follows (pos has no reader then): the maximum is kept
// across channels without the per-channel record, and the search after the loop is left out.  Same subtractions and
// maxima: the values are those of POS = true bit for bit.
template <int S, bool RESIDENT, bool POS>
__global__ void __launch_bounds__(kMaxThreads, 2)
inf_conv_forward_kernel(const float* __restrict__ img, const float* __restrict__ weight, float* __restrict__ out,
                        int32_t* __restrict__ pos, ConvFwd a) {
    constexpr int NXR = (7 * S + 2) / 4 + 1;          // 128-bit reads per window row: pixels 0 .. 7*S + 2
    extern __shared__ __align__(16) float lds[];
    float* tile = lds;                                  // RESIDENT: [CGP][NR][WP]; staged: 2 x [xwords / 2]
    float* wst = lds + a.xwords;                        // 2 x [kKC][kBNP]
    const int tid = threadIdx.x, NT = blockDim.x;

    int id = blockIdx.x;
    const int tn = id % a.tiles_n; id /= a.tiles_n;
    const int th = id % a.tiles_h; id /= a.tiles_h;
    const int g = id % a.G, b = id / a.G;
    const int h0 = th * a.R, n0 = tn * a.BN;
    const int y0 = h0 * S - a.P;
    const int NR = a.NR, WP = a.WP, K = a.K;
    // floats between the channels of the image area: resident, padded so that lanes that look into different
    // channels (the argmax search) spread over the banks; staged, the channels of a stage are packed
    const int CST = RESIDENT ? a.cstride : NR * WP;
    constexpr int BNP = kBNP;

    // ---- weights: global -> registers -> LDS stage, k-major ----
    const float* wgrp = weight + ((size_t)g * a.NG + n0) * K;
    const int nvalid = min(a.NG - n0, a.BN);            // outputs of this tile that exist
    float wreg[kWRegs];
    auto wload = [&](int ch) {
        const int kb = ch * kKC;
#pragma unroll
        for (int r = 0; r < kWRegs; r++) {
            const int idx = tid + r * NT;
            const int n = idx / kKC, kk = idx - n * kKC;
            // branch-free: an entry that does not exist reads the tile's first weight and is replaced by zero
            const bool real = n < nvalid && kb + kk < K;
            const float v = wgrp[real ? (unsigned)(n * K + kb + kk) : 0u];
            wreg[r] = real ? v : 0.f;
        }
    };
    auto wstore = [&](float* stage) {
#pragma unroll
        for (int r = 0; r < kWRegs; r++) {
            const int idx = tid + r * NT;
            const int n = idx / kKC, kk = idx - n * kKC;
            stage[kk * BNP + n] = wreg[r];   // n <= 63 (idx < kWRegs * 256 = 36 * 64): inside the stage, zeros beyond BN
        }
    };
    // A workgroup too small to carry a whole stage in kWRegs words per lane (tiny images) moves the rest
    // directly; with 256 lanes this loop is empty.
    auto wrest = [&](int ch, float* stage) {
        const int kb = ch * kKC;
        for (int idx = tid + kWRegs * NT; idx < kKC * a.BN; idx += NT) {
            const int n = idx / kKC, kk = idx - n * kKC;
            const bool real = n < nvalid && kb + kk < K;
            stage[kk * BNP + n] = real ? wgrp[(unsigned)(n * K + kb + kk)] : 0.f;
        }
    };
    wload(0);

    const float* src = img + ((size_t)b * a.G + g) * a.CG * a.H * a.W;   // the group's channels of this image
    // ---- staged: what each lane moves per stage is the same every time, only the channel base advances ----
    const int xhalf = a.xwords / 2;                     // one stage buffer: at least kCC*NR*WP and kXRegs*NT words
    constexpr int kXRegs = x_regs(S);
    int goff[kXRegs];                                   // element offset inside the stage's kCC channels; -1 = padding
    float xreg[kXRegs];
    if constexpr (!RESIDENT) {
        const int plane = NR * WP;
#pragma unroll
        for (int r = 0; r < kXRegs; r++) {
            const int idx = tid + r * NT;
            const int c = idx / plane, rem = idx - c * plane;
            const int row = rem / WP, col = rem - row * WP;
            const int y = y0 + row, x = col - a.P;
            const bool real = c < kCC && (unsigned)y < (unsigned)a.H && (unsigned)x < (unsigned)a.W;
            goff[r] = real ? (c * a.H + y) * a.W + x : -1;
        }
    }
    auto xload = [&](int ch) {
        const float* base = src + (size_t)ch * kCC * a.H * a.W;
#pragma unroll
        for (int r = 0; r < kXRegs; r++) {
            const float v = base[goff[r] < 0 ? 0 : goff[r]];   // branch-free: padding reads a valid word, replaced by 0
            xreg[r] = goff[r] < 0 ? 0.f : v;
        }
    };
    auto xstore = [&](float* stage) {
#pragma unroll
        for (int r = 0; r < kXRegs; r++) stage[tid + r * NT] = xreg[r];   // < kXRegs*NT <= xhalf
    };
    // A workgroup too small to carry a whole stage in kXRegs words per lane (tiny images) moves the rest
    // directly; with 256 lanes this loop is empty.
    auto xrest = [&](int ch, float* stage) {
        const float* base = src + (size_t)ch * kCC * a.H * a.W;
        const int plane = NR * WP;
        for (int idx = tid + kXRegs * NT; idx < kCC * plane; idx += NT) {
            const int c = idx / plane, rem = idx - c * plane;
            const int row = rem / WP, col = rem - row * WP;
            const int y = y0 + row, x = col - a.P;
            const bool real = (unsigned)y < (unsigned)a.H && (unsigned)x < (unsigned)a.W;
            stage[idx] = real ? base[(c * a.H + y) * a.W + x] : 0.f;
        }
    };

    // ---- RESIDENT: image rows -> LDS once, padding as zeros ----
    if constexpr (RESIDENT) {
        const int words = a.CGP * CST;
        for (int i = tid * 4; i < words; i += NT * 4) *reinterpret_cast<float4*>(tile + i) = make_float4(0.f, 0.f, 0.f, 0.f);
        __syncthreads();
        const int rows = a.CG * NR;
        if (a.vec_in) {
            // four 16-byte loads in flight per lane, then their stores: one at a time, a workgroup would wait out
            // a memory latency per 4 KB before it can start
            const int QW = a.W / 4, total = rows * QW;
            constexpr int UN = 4;
            for (int i0 = tid; i0 < total; i0 += UN * NT) {
                float4 v[UN];
                int at[UN];
#pragma unroll
                for (int u = 0; u < UN; u++) {
                    const int i = i0 + u * NT;
                    const int row = i / QW, xq = i - row * QW;
                    const int c = row / NR, r = row - c * NR;
                    const int y = y0 + r;
                    const bool real = i < total && (unsigned)y < (unsigned)a.H;
                    at[u] = real ? c * CST + r * WP + a.P + 4 * xq : -1;
                    v[u] = *reinterpret_cast<const float4*>(src + (real ? ((size_t)c * a.H + y) * a.W + 4 * xq : 0));
                }
#pragma unroll
                for (int u = 0; u < UN; u++)
                    if (at[u] >= 0) {
                        float* dst = tile + at[u];
                        dst[0] = v[u].x; dst[1] = v[u].y; dst[2] = v[u].z; dst[3] = v[u].w;
                    }
            }
        } else {
            for (int i = tid; i < rows * a.W; i += NT) {
                const int row = i / a.W, x = i - row * a.W;
                const int c = row / NR, r = row - c * NR;
                const int y = y0 + r;
                if ((unsigned)y < (unsigned)a.H) tile[c * CST + r * WP + a.P + x] = src[((size_t)c * a.H + y) * a.W + x];
            }
        }
    } else {
        xload(0);
        xstore(tile);
        xrest(0, tile);
    }
    wstore(wst);
    wrest(0, wst);
    __syncthreads();

    // ---- lane geometry ----
    const int nl = tid % a.NL, ml = tid / a.NL;
    const int hr = ml / a.SEG, w0 = (ml - hr * a.SEG) * kTM;
    const int xlane_off = (hr * S) * WP + w0 * S;              // + (c*NR + i)*WP: 16-byte aligned (WP % 4 == 0)
    const float* xlane = tile + xlane_off;

    float acc[kTM][kTN], cm[kTM][kTN];   // running maxima; the units alternate between them
    int unit[kTM][kTN];
#pragma unroll
    for (int e = 0; e < kTM; e++)
#pragma unroll
        for (int t = 0; t < kTN; t++) { acc[e][t] = 0.f; cm[e][t] = 0.f; unit[e][t] = 0; }

    const int nstage = a.CGP / kCC;
    const float* xch = xlane;
    for (int ch = 0; ch < nstage; ch++) {
        if (ch + 1 < nstage) {
            wload(ch + 1);
            if constexpr (!RESIDENT) xload(ch + 1);
        }
        const float* wrow = wst + (ch & 1) * kKC * BNP + kTN * nl;   // walks down the 9*kCC rows of the stage
        // walks down the window rows of the stage's channels
        const float* xrow = RESIDENT ? xch : tile + (ch & 1) * xhalf + xlane_off;
        static_assert(kTrack == 1 && kCC % 2 == 0, "a unit is a channel; units in pairs");
        if constexpr (RESIDENT) {
            // A unit (one channel: nine differences per position and output) continues the running maximum: cur
            // starts from prev, which is left alone, so the unit raised the maximum iff cur > prev afterwards, and the
            // two arrays swap roles from unit to unit (no copy, one compare and one select per unit and output).
            // The loop over pairs of units stays rolled.
            auto unit_pass = [&](const float (&prev)[kTM][kTN], float (&cur)[kTM][kTN], int un) {
                // The three window rows of the unit, unrolled, with the reads of a row issued before the arithmetic
                // of the row before it.
                struct Row { float x[NXR * 4]; float w[3][kTN]; };
                auto fetch = [&](Row& f, int r) {
                    const float* xp = xrow + r * WP;
#pragma unroll
                    for (int q = 0; q < NXR; q++) {
                        const float4 v = *reinterpret_cast<const float4*>(xp + 4 * q);
                        f.x[4 * q] = v.x; f.x[4 * q + 1] = v.y; f.x[4 * q + 2] = v.z; f.x[4 * q + 3] = v.w;
                    }
#pragma unroll
                    for (int j = 0; j < 3; j++) {
                        const float4 w4 = *reinterpret_cast<const float4*>(wrow + (3 * r + j) * BNP);
                        f.w[j][0] = w4.x; f.w[j][1] = w4.y; f.w[j][2] = w4.z; f.w[j][3] = w4.w;
                    }
                };
                Row fa, fb;
                fetch(fa, 0);
#pragma unroll
                for (int r = 0; r < 3; r++) {
                    Row& now = (r & 1) ? fb : fa;
                    Row& nxt = (r & 1) ? fa : fb;
                    if (r + 1 < 3) fetch(nxt, r + 1);
#pragma unroll
                    for (int j = 0; j < 3; j++)
#pragma unroll
                        for (int e = 0; e < kTM; e++)
#pragma unroll
                            for (int t = 0; t < kTN; t++)
                                cur[e][t] = __builtin_fmaxf(r == 0 && j == 0 ? prev[e][t] : cur[e][t],
                                                            __builtin_fabsf(now.x[e * S + j] - now.w[j][t]));
                }
                xrow += CST;
                wrow += 9 * BNP;
                if constexpr (POS) {
                    // Eight compares into their own scalar register pairs, then their selects: a select straight
                    // after its compare waits two cycles for the lane mask.  The empty asm statements keep their
                    // order: the first kind keeps a mask from being folded back into the plain form, the second
                    // ends a group.
                    static_assert(kTM % 2 == 0, "rows in pairs");
#pragma unroll
                    for (int e = 0; e < kTM; e += 2) {
                        unsigned long long raised[2][kTN];
#pragma unroll
                        for (int a2 = 0; a2 < 2; a2++)
#pragma unroll
                            for (int t = 0; t < kTN; t++) {
                                raised[a2][t] = __builtin_amdgcn_fcmpf(cur[e + a2][t], prev[e + a2][t], 2 /* ordered > */);
                                asm volatile("" : "+s"(raised[a2][t]));
                            }
#pragma unroll
                        for (int a2 = 0; a2 < 2; a2++)
#pragma unroll
                            for (int t = 0; t < kTN; t++) {
                                if (__builtin_amdgcn_inverse_ballot_w64(raised[a2][t])) unit[e + a2][t] = un;
                                asm volatile("" : "+v"(unit[e + a2][t]));
                            }
                    }
                }
            };
#pragma unroll 1
            for (int u = 0; u < kCC; u += 2) {
                const int un = ch * kCC + u;
                unit_pass(acc, cm, un);
                unit_pass(cm, acc, un + 1);
            }
        } else {
            // The staged variant has no registers to spare for that (it also carries the parked image words of the
            // next stage; any other arrangement of this loop that was tried spilled): one unit per trip, its maximum
            // taken from zero and then compared with the running one (compare and two selects per unit and output).
#pragma unroll 1
            for (int u = 0; u < kCC / kTrack; u++) {
                float cm[kTM][kTN];   // the unit's maximum; without pos, the running maximum itself
#pragma unroll
                for (int e = 0; e < kTM; e++)
#pragma unroll
                    for (int t = 0; t < kTN; t++) cm[e][t] = POS ? 0.f : acc[e][t];
                // The 3*kTrack window rows of the unit, unrolled, with the reads of a row issued before the
                // arithmetic of the row before it.
                struct Row { float x[NXR * 4]; float w[3][kTN]; };
                auto fetch = [&](Row& f, int r) {     // r = cc*3 + i: window row i of the unit's channel cc
                    const float* xp = xrow + ((r / 3) * NR + r % 3) * WP;
#pragma unroll
                    for (int q = 0; q < NXR; q++) {
                        const float4 v = *reinterpret_cast<const float4*>(xp + 4 * q);
                        f.x[4 * q] = v.x; f.x[4 * q + 1] = v.y; f.x[4 * q + 2] = v.z; f.x[4 * q + 3] = v.w;
                    }
#pragma unroll
                    for (int j = 0; j < 3; j++) {
                        const float4 w4 = *reinterpret_cast<const float4*>(wrow + (3 * r + j) * BNP);
                        f.w[j][0] = w4.x; f.w[j][1] = w4.y; f.w[j][2] = w4.z; f.w[j][3] = w4.w;
                    }
                };
                Row fa, fb;
                fetch(fa, 0);
#pragma unroll
                for (int r = 0; r < 3 * kTrack; r++) {
                    Row& cur = (r & 1) ? fb : fa;
                    Row& nxt = (r & 1) ? fa : fb;
                    if (r + 1 < 3 * kTrack) fetch(nxt, r + 1);
#pragma unroll
                    for (int j = 0; j < 3; j++)
#pragma unroll
                        for (int e = 0; e < kTM; e++)
#pragma unroll
                            for (int t = 0; t < kTN; t++)
                                cm[e][t] = __builtin_fmaxf(cm[e][t], __builtin_fabsf(cur.x[e * S + j] - cur.w[j][t]));
                }
                xrow += kTrack * CST;
                wrow += 9 * kTrack * BNP;
                const int un = ch * (kCC / kTrack) + u;
#pragma unroll
                for (int e = 0; e < kTM; e++)
#pragma unroll
                    for (int t = 0; t < kTN; t++)
                        if constexpr (POS) {
                            if (cm[e][t] > acc[e][t]) { acc[e][t] = cm[e][t]; unit[e][t] = un; }
                        } else {
                            acc[e][t] = cm[e][t];
                        }
            }
        }
        xch += kCC * CST;
        if (ch + 1 < nstage) {
            wstore(wst + ((ch + 1) & 1) * kKC * BNP);
            wrest(ch + 1, wst + ((ch + 1) & 1) * kKC * BNP);
            if constexpr (!RESIDENT) {
                xstore(tile + ((ch + 1) & 1) * xhalf);
                xrest(ch + 1, tile + ((ch + 1) & 1) * xhalf);
            }
        }
        __syncthreads();
    }

    const int h = h0 + hr;
    if (h >= a.HO) return;
    const int L = a.HO * a.WO;
    if constexpr (!POS) {
#pragma unroll
        for (int t = 0; t < kTN; t++) {
            const int n = n0 + kTN * nl + t;
            if (n >= a.NG) break;
            const size_t at = (((size_t)b * a.G + g) * a.NG + n) * L + (size_t)h * a.WO + w0;
            if (a.vec_out) {
                *reinterpret_cast<float4*>(out + at) = make_float4(acc[0][t], acc[1][t], acc[2][t], acc[3][t]);
                *reinterpret_cast<float4*>(out + at + 4) = make_float4(acc[4][t], acc[5][t], acc[6][t], acc[7][t]);
            } else {
#pragma unroll
                for (int e = 0; e < kTM; e++)
                    if (w0 + e < a.WO) out[at + e] = acc[e][t];
            }
        }
        return;
    }
    // ---- the lowest k of the recorded unit, from the image rows in LDS and the weight rows in cache ----
    // Per output the recorded channel's nine weights are contiguous: two 16-byte loads at 4-byte alignment
    // and one word instead of one load per candidate, issued for the lane's eight positions together.
    typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
    static_assert(kTrack == 1, "a unit is one channel: nine candidates");
    // EB positions of one output at a time, in steps (output t, positions e0 .. e0 + EB - 1).  The weight loads of a
    // step are issued one step ahead (two register sets that take turns), so that the cache latency of a step's
    // weights passes while the step before it is searched; the pixels come from LDS (RESIDENT) or from the image.
    constexpr int EB = kTM / 2, STEPS = kTN * (kTM / EB);
    float wq[2][EB][9];
    auto issue = [&](int step, float (&wb)[EB][9]) {
        const int t = step / (kTM / EB), e0 = (step % (kTM / EB)) * EB;
        const int n = min(n0 + kTN * nl + t, a.NG - 1);     // an output past the layer's last reads that one's weights
        const float* wn = weight + ((size_t)g * a.NG + n) * K;
#pragma unroll
        for (int eb = 0; eb < EB; eb++) {
            const float* wp = wn + unit[e0 + eb][t] * 9;    // a recorded unit is a real channel: inside the row
            const f4u q0 = *reinterpret_cast<const f4u*>(wp), q1 = *reinterpret_cast<const f4u*>(wp + 4);
            wb[eb][0] = q0.x; wb[eb][1] = q0.y; wb[eb][2] = q0.z; wb[eb][3] = q0.w;
            wb[eb][4] = q1.x; wb[eb][5] = q1.y; wb[eb][6] = q1.z; wb[eb][7] = q1.w;
            wb[eb][8] = wp[8];
        }
    };
    int ps[kTM];
    issue(0, wq[0]);
#pragma unroll
    for (int step = 0; step < STEPS; step++) {
        const int t = step / (kTM / EB), e0 = (step % (kTM / EB)) * EB;
        if (step + 1 < STEPS) issue(step + 1, wq[(step + 1) & 1]);
        float xq[EB][9];
#pragma unroll
        for (int eb = 0; eb < EB; eb++) {
            const int e = e0 + eb;
            if constexpr (RESIDENT) {
                const float* xe = xlane + e * S + unit[e][t] * CST;
#pragma unroll
                for (int r = 0; r < 9; r++) xq[eb][r] = xe[(r / 3) * WP + r % 3];
            } else {
                // the window of position (h, w0 + e) in the recorded channel; outside the image it reads 0
                const unsigned plane = (unsigned)unit[e][t] * (unsigned)(a.H * a.W);
                const int yy = h * S - a.P, xx = (w0 + e) * S - a.P;
#pragma unroll
                for (int r = 0; r < 9; r++) {
                    const int y = yy + r / 3, x = xx + r % 3;
                    const bool real = (unsigned)y < (unsigned)a.H && (unsigned)x < (unsigned)a.W;
                    const float v = src[real ? plane + (unsigned)(y * a.W + x) : 0u];
                    xq[eb][r] = real ? v : 0.f;
                }
            }
        }
        const float (&wb)[EB][9] = wq[step & 1];
#pragma unroll
        for (int eb = 0; eb < EB; eb++) {
            const int e = e0 + eb;
            const float target = acc[e][t];
            int q = 0;
            float dq = 0.f;
#pragma unroll
            for (int r = 8; r >= 0; r--) {                // descending: the lowest match is the one kept
                const float df = xq[eb][r] - wb[eb][r];
                if (__builtin_fabsf(df) == target) { q = r; dq = df; }
            }
            ps[e] = target > 0.f ? ((unit[e][t] * 9 + q) | (__float_as_int(dq) & 0x80000000)) : 0;
        }
        if (e0 + EB < kTM) continue;                      // the output's other positions come with the next step
        const int n = n0 + kTN * nl + t;
        if (n >= a.NG) continue;
        const size_t at = (((size_t)b * a.G + g) * a.NG + n) * L + (size_t)h * a.WO + w0;
        if (a.vec_out) {
            *reinterpret_cast<float4*>(out + at) = make_float4(acc[0][t], acc[1][t], acc[2][t], acc[3][t]);
            *reinterpret_cast<float4*>(out + at + 4) = make_float4(acc[4][t], acc[5][t], acc[6][t], acc[7][t]);
            *reinterpret_cast<int4*>(pos + at) = make_int4(ps[0], ps[1], ps[2], ps[3]);
            *reinterpret_cast<int4*>(pos + at + 4) = make_int4(ps[4], ps[5], ps[6], ps[7]);
        } else {
#pragma unroll
            for (int e = 0; e < kTM; e++)
                if (w0 + e < a.WO) { out[at + e] = acc[e][t]; pos[at + e] = ps[e]; }
        }
    }
}

}  // namespace

bool inf_conv_forward_supported(const ConvGeom& q, int G, int CO) {
    ConvFwd a{};
    return plan(q, G, CO, a);
}

// pos == nullptr: values only (the kernel without the argmax).
hipError_t inf_conv_forward(const float* img, const float* weight, float* out, int32_t* pos, const ConvGeom& q, int G,
                            int CO, int device, hipStream_t stream) {
    ConvFwd a{};
    if (!plan(q, G, CO, a)) return hipErrorInvalidValue;   // the API layer asks inf_conv_forward_supported first
    const bool with_pos = pos != nullptr;
    a.vec_in = q.W % 4 == 0 && aligned16(img);
    a.vec_out = q.WO % kTM == 0 && aligned16(out) && aligned16(pos);   // every run of 8 positions whole and aligned
    const size_t lds = ((size_t)a.xwords + 2 * (size_t)kKC * kBNP) * sizeof(float);
    static std::atomic<bool> raised[64][8] = {};   // callers may come from several threads
    const int ki = ((q.S - 1) * 2 + a.resident) * 2 + (with_pos ? 1 : 0);
    using Kern = void (*)(const float*, const float*, float*, int32_t*, ConvFwd);
    const Kern table[8] = {inf_conv_forward_kernel<1, false, false>, inf_conv_forward_kernel<1, false, true>,
                           inf_conv_forward_kernel<1, true, false>,  inf_conv_forward_kernel<1, true, true>,
                           inf_conv_forward_kernel<2, false, false>, inf_conv_forward_kernel<2, false, true>,
                           inf_conv_forward_kernel<2, true, false>,  inf_conv_forward_kernel<2, true, true>};
    const Kern kern = table[ki];
    if (!(device >= 0 && device < 64 && raised[device][ki].load(std::memory_order_acquire))) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)kLdsLimit);
        if (e != hipSuccess) return e;
        if (device >= 0 && device < 64) raised[device][ki].store(true, std::memory_order_release);
    }
    const unsigned grid = (unsigned)((long long)q.B * G * a.tiles_h * a.tiles_n);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(a.ML * a.NL), lds, stream, img, weight, out, pos, a);
    return hipGetLastError();
}

}  // namespace ldist

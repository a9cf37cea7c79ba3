// L_inf distance forward with argmax for the unfolded-conv layout (HW > 1) when the reduction is short:
// the whole K of a 32-row x 32-output tile stays in LDS.  Same results, bit for bit, as inf_forward.hip;
// semantics of the reference kernel model/inf_dist_cuda.cu:10-68.
//
// In this layout a recorded 32-wide chunk cannot be read again cheaply at the end (k has stride HW in the
// input: a strided gather per output), and tracking k itself in the loop costs four instructions per
// (row, output, k).  Here the loop keeps the running maximum only (one v_sub_f32 and half a v_max3_f32)
// and asks once per window of eight k whether the maximum moved (a compare and a select per output and
// window: 1.75 instructions per (row, output, k) in all).  Because both panels are still in LDS when the
// loop ends, the lowest k inside the recorded window is then found from LDS: eight differences per output,
// once per output instead of once per output and stage.
//
// Workgroup: 256 lanes = four waves that split K in four contiguous ranges (a range is a whole number of
// windows); a wave covers the whole 32 x 32 tile with a 4 x 4 register patch per lane.  The four partial
// results meet in LDS in ascending order of k ("strictly larger wins"), which keeps the lowest k on ties.
// LDS: X[k][32 rows] and W[k][32 outputs] (k-major), plus 6 KB for the merge.  The input is row-contiguous in
// memory and goes in with 128-bit stores.  The weights are read along k with coalesced 32-bit loads, four
// neighbouring outputs per lane, and stored as one 128-bit word whose place in row k is XORed with k % 8
// (in units of four outputs): the 64 lanes of a store, which differ in k, then cover all banks instead of
// four.  K = 288 (a 3x3 window over 32 channels) takes 78 KB: two workgroups per CU, whose load and compute
// phases overlap each other.
#include "fwd_engine.hpp"

namespace ldist {

namespace shortk {
constexpr int BM = 32, BN = 32, NT = 256, NGROUP = 4, WIN = 8;
constexpr int KQ = NGROUP * WIN;                  // K is padded to a multiple of this
constexpr int MAX_KP_TWO_PER_CU = 288;            // (2*Kp*32 + 1024)*4 + 2048 bytes <= 80 KB
// float offset inside row k of W of the group of four outputs nq (0..7)
__device__ __forceinline__ constexpr int wslot(int k, int nq) { return ((nq ^ (k & 7)) << 2); }
inline int padded_k(int K) { return (K + KQ - 1) / KQ * KQ; }
inline size_t lds_bytes(int Kp) { return ((size_t)2 * Kp * BM + BM * BN) * sizeof(float) + BM * BN * sizeof(uint16_t); }
}  // namespace shortk

__global__ void __launch_bounds__(shortk::NT, 2)
inf_forward_shortk_kernel(const float* __restrict__ input, const float* __restrict__ weight,
                          float* __restrict__ output, int32_t* __restrict__ pos, Dims d, int Kp) {
    using namespace shortk;
    extern __shared__ __align__(16) float lds[];
    float* X = lds;                         // [Kp][BM]
    float* W = lds + (size_t)Kp * BM;       // [Kp][BN]
    float* cand_v = W + (size_t)Kp * BN;    // [BN][BM]: the row index is innermost, like the output tensor
    uint16_t* cand_w = reinterpret_cast<uint16_t*>(cand_v + BM * BN);

    const int tid = threadIdx.x;
    int id = blockIdx.x;
    const int tm = id % d.tiles_m;
    id /= d.tiles_m;
    const int tn = id % d.tiles_n, g = id / d.tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;
    const int K = d.K, HW = d.HW;

    // ---- global -> LDS, the whole reduction axis at once -------------------------------------------
    {
        // input: a lane keeps its four rows (consecutive positions of one image: HW % 4 == 0) and walks k
        const int mq = tid % (BM / 4), kx = tid / (BM / 4);
        const int m = m0 + mq * 4;
        const bool row_ok = m < d.M;
        const int b = row_ok ? m / HW : 0, hw = row_ok ? m % HW : 0;
        const float* xin = input + ((size_t)(b * d.G + g) * K) * HW + hw;
        // weights: lanes run along k (coalesced 32-bit loads), a lane takes four neighbouring outputs
        const int npass = Kp / (NT / (BM / 4));   // = Kp / 32 for both panels
        constexpr int BATCH = 3;
#pragma unroll 1
        for (int p0 = 0; p0 < npass; p0 += BATCH) {
            float4 xv[BATCH], wv[BATCH];
#pragma unroll
            for (int e = 0; e < BATCH; e++) {
                const int p = p0 + e;
                xv[e] = make_float4(0.f, 0.f, 0.f, 0.f);
                wv[e] = xv[e];
                if (p < npass) {
                    const int k = kx + p * (NT / (BM / 4));
                    if (row_ok && k < K) xv[e] = *reinterpret_cast<const float4*>(xin + (size_t)k * HW);
                    const int wid = tid + p * NT;            // < Kp * 8
                    const int kw = wid % Kp, nq = wid / Kp;
                    const int n = n0 + nq * 4;
                    if (kw < K) {
                        const float* wr = weight + ((size_t)g * d.NG + n) * K + kw;
                        if (n + 0 < d.NG) wv[e].x = wr[0];
                        if (n + 1 < d.NG) wv[e].y = wr[(size_t)K];
                        if (n + 2 < d.NG) wv[e].z = wr[(size_t)2 * K];
                        if (n + 3 < d.NG) wv[e].w = wr[(size_t)3 * K];
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < BATCH; e++) {
                const int p = p0 + e;
                if (p < npass) {
                    const int k = kx + p * (NT / (BM / 4));
                    *reinterpret_cast<float4*>(X + k * BM + mq * 4) = xv[e];
                    const int wid = tid + p * NT;
                    const int kw = wid % Kp, nq = wid / Kp;
                    *reinterpret_cast<float4*>(W + kw * BN + wslot(kw, nq)) = wv[e];
                }
            }
        }
    }
    __syncthreads();

    // ---- the reduction: wave q takes k in [q*Kg, (q+1)*Kg) -----------------------------------------
    const int lane = tid & 63, grp = tid >> 6;
    const int tx = lane % 8, ty = lane / 8;
    const int Kg = Kp / NGROUP, nwin = Kg / WIN;
    float accA[4][4], accB[4][4];
    int widx[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) { accA[i][j] = 0.f; accB[i][j] = 0.f; widx[i][j] = 0; }

    // Operand addresses: row kb + e of a window (kb a multiple of 8) keeps the lane's four outputs at group tx ^ e,
    // so eight lane constants, added to a pointer that moves by a window at a time, serve the whole loop.
    const float* xp = X + (size_t)grp * Kg * BM + ty * 4;
    const float* wp = W + (size_t)grp * Kg * BN;
    int woff[WIN];
#pragma unroll
    for (int e = 0; e < WIN; e++) woff[e] = e * BN + ((tx ^ e) << 2);
    float4 xa[2], wa[2], xb[2], wb[2];
    auto fetch = [&](float4 (&xf)[2], float4 (&wf)[2], int kk) {   // rows kk, kk + 1 of the current window
#pragma unroll
        for (int e = 0; e < 2; e++) {
            xf[e] = *reinterpret_cast<const float4*>(xp + (kk + e) * BM);
            wf[e] = *reinterpret_cast<const float4*>(wp + woff[kk + e]);
        }
    };
    // One window: cur continues the running maximum from prev (prev is left alone), so the window raised the
    // maximum iff cur > prev afterwards.  The arrays swap roles from window to window: nothing is copied.
    // Four pairs of k; the next pair's operands are fetched while the current pair is reduced, the first pair
    // of the next window during the last reduction (after the last window that reads rows which belong to the
    // next range or lie just behind the panel, inside the allocation; they are never used).
    auto window = [&](const float (&prev)[4][4], float (&cur)[4][4], int wid) {
        auto reduce = [&](const float4 (&xf)[2], const float4 (&wf)[2], const float (&from)[4][4]) {
            const float x0[4] = {xf[0].x, xf[0].y, xf[0].z, xf[0].w}, x1[4] = {xf[1].x, xf[1].y, xf[1].z, xf[1].w};
            const float w0[4] = {wf[0].x, wf[0].y, wf[0].z, wf[0].w}, w1[4] = {wf[1].x, wf[1].y, wf[1].z, wf[1].w};
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    cur[i][j] = __builtin_fmaxf(__builtin_fmaxf(from[i][j], __builtin_fabsf(x0[i] - w0[j])),
                                                __builtin_fabsf(x1[i] - w1[j]));
        };
        fetch(xb, wb, 2);
        __builtin_amdgcn_sched_barrier(0);
        reduce(xa, wa, prev);
        fetch(xa, wa, 4);
        __builtin_amdgcn_sched_barrier(0);
        reduce(xb, wb, cur);
        fetch(xb, wb, 6);
        __builtin_amdgcn_sched_barrier(0);
        reduce(xa, wa, cur);
        xp += WIN * BM;
        wp += WIN * BN;
        fetch(xa, wa, 0);
        __builtin_amdgcn_sched_barrier(0);
        reduce(xb, wb, cur);
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (cur[i][j] > prev[i][j]) widx[i][j] = wid;
    };
    fetch(xa, wa, 0);
    const int wid0 = grp * nwin;
#pragma unroll 1
    for (int w = 0; w < nwin; w += 2) {
        window(accA, accB, wid0 + w);
        if (w + 1 < nwin) {
            window(accB, accA, wid0 + w + 1);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) accA[i][j] = accB[i][j];
        }
    }

    // ---- the four k ranges meet in LDS, ascending k: a later range wins only with a strictly larger value
#pragma unroll 1
    for (int turn = 0; turn < NGROUP; turn++) {
        if (grp == turn) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int o = (tx * 4 + j) * BM + ty * 4;
                float4 v = make_float4(accA[0][j], accA[1][j], accA[2][j], accA[3][j]);
                int wsel[4] = {widx[0][j], widx[1][j], widx[2][j], widx[3][j]};
                if (turn > 0) {
                    const float4 old = *reinterpret_cast<const float4*>(cand_v + o);
                    const ushort4 ow = *reinterpret_cast<const ushort4*>(cand_w + o);
                    if (!(v.x > old.x)) { v.x = old.x; wsel[0] = ow.x; }
                    if (!(v.y > old.y)) { v.y = old.y; wsel[1] = ow.y; }
                    if (!(v.z > old.z)) { v.z = old.z; wsel[2] = ow.z; }
                    if (!(v.w > old.w)) { v.w = old.w; wsel[3] = ow.w; }
                }
                *reinterpret_cast<float4*>(cand_v + o) = v;
                *reinterpret_cast<ushort4*>(cand_w + o) =
                    make_ushort4((unsigned short)wsel[0], (unsigned short)wsel[1], (unsigned short)wsel[2], (unsigned short)wsel[3]);
            }
        }
        __syncthreads();
    }

    // ---- lowest k inside the recorded window, from the panels; a lane takes four neighbouring rows of one output
    {
        const int nl = tid / (BM / 4), mq = tid % (BM / 4);
        const int o = nl * BM + mq * 4;
        const float4 v4 = *reinterpret_cast<const float4*>(cand_v + o);
        const ushort4 w4 = *reinterpret_cast<const ushort4*>(cand_w + o);
        const float vs[4] = {v4.x, v4.y, v4.z, v4.w};
        const int ws[4] = {w4.x, w4.y, w4.z, w4.w};
        int ps[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int kb = ws[i] * WIN;
            const float* xr = X + kb * BM + mq * 4 + i;
            const float* wr = W + kb * BN + (nl & 3);
            float xv[WIN], wv[WIN];
#pragma unroll
            for (int e = 0; e < WIN; e++) { xv[e] = xr[e * BM]; wv[e] = wr[e * BN + wslot(e, nl >> 2)]; }   // kb % 8 == 0
            int p = 0;
#pragma unroll
            for (int e = WIN - 1; e >= 0; e--) {   // descending: the lowest match is written last
                const float df = xv[e] - wv[e];
                if (__builtin_fabsf(df) == vs[i]) p = (kb + e) | (__float_as_int(df) & 0x80000000);
            }
            ps[i] = vs[i] > 0.f ? p : 0;           // nothing exceeded the initial 0: the reference leaves pos = 0
        }
        const int m = m0 + mq * 4, n = n0 + nl;
        if (m < d.M && n < d.NG) {                 // HW % 4 == 0: the four rows lie inside the tensor and one image
            const int b = m / HW, hw = m % HW;
            const size_t at = ((size_t)(b * d.G + g) * d.NG + n) * HW + hw;
            *reinterpret_cast<float4*>(output + at) = v4;
            *reinterpret_cast<int4*>(pos + at) = make_int4(ps[0], ps[1], ps[2], ps[3]);
        }
    }
}

// Whether the kernel above serves the problem: conv layout with rows in aligned groups of four, and a K whose
// panels leave room for two workgroups per CU (`any_k`: for one as well -- tests and tuning).
bool inf_forward_shortk_applicable(const Problem& pr, const void* input, const void* output, const void* pos, bool any_k) {
    if (pr.HW == 1 || pr.HW % 4 != 0) return false;
    if (!aligned16(input) || !aligned16(output) || !aligned16(pos)) return false;
    const int Kp = shortk::padded_k(pr.K);
    if (Kp / shortk::WIN > 65535) return false;                         // window ids are parked as 16-bit
    if (shortk::lds_bytes(Kp) > 160 * 1024) return false;
    return any_k || Kp <= shortk::MAX_KP_TWO_PER_CU;
}

hipError_t inf_forward_shortk(const float* input, const float* weight, float* output, int32_t* pos, const Problem& pr,
                              hipStream_t stream) {
    Dims d = make_dims(pr);
    d.tiles_m = (d.M + shortk::BM - 1) / shortk::BM;
    d.tiles_n = (d.NG + shortk::BN - 1) / shortk::BN;
    const int Kp = shortk::padded_k(pr.K);
    const size_t lds = shortk::lds_bytes(Kp);
    static bool lds_allowed[64] = {};
    if (hipError_t e = allow_lds(inf_forward_shortk_kernel, 160 * 1024, pr.device, lds_allowed); e != hipSuccess) return e;
    const unsigned grid = (unsigned)d.tiles_m * d.tiles_n * d.G;
    hipLaunchKernelGGL(inf_forward_shortk_kernel, dim3(grid), dim3(shortk::NT), lds, stream, input, weight, output, pos,
                       d, Kp);
    return hipGetLastError();
}

}  // namespace ldist

// L_inf distance forward with argmax for the unfolded-conv layout (HW > 1) when the reduction is short:
// the whole K of a 64-row x 32-output tile stays in LDS.  Same results, bit for bit, as inf_forward.hip;
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
// Workgroup: 512 lanes = eight waves, one workgroup per CU, which walks every grid-th tile.  Waves
// 0..3 take the upper 32 rows of the tile, waves 4..7 the lower 32; the four waves of a half split K in four
// contiguous ranges (a range is a whole number of windows) and each covers its 32 x 32 half tile with a 4 x 4
// register patch per lane.  Every wave parks its (value, window) pairs in a slab of its own; after one barrier
// the lane that finishes an output reads the four pairs in ascending order of k ("strictly larger wins",
// which keeps the lowest k on ties).
// LDS: X[k][64 rows] and W[k][32 outputs] (k-major), plus 40 KB of slabs; K = 288 (a 3x3 window over 32
// channels) takes 148 KB.  The weight panel is loaded once per run of tiles that share it.
// During the reduction nobody but the wave itself reads its block of the input panel (its 32 rows, its k range),
// so every wave brings in its own block: a window of the block (8 k x 32 rows) is one 128-bit load per lane.  The
// loads of the next tile's block stay parked in registers for a whole tile; the wave writes a window to LDS one
// window ahead of reducing it and at once reuses the registers for the same window of the tile after that.  So
// the panel is written and the loads are issued a few instructions at a time, in the shadow of the arithmetic,
// and no barrier stands between them and the reduction.  The weights are read along k with coalesced 32-bit
// loads, four neighbouring outputs per lane, and stored as one 128-bit word (the lanes of such a store differ in
// k and meet in few banks; it happens once per run of tiles, and plain rows let every later read of the panel use
// one address register and constant offsets).
#include "fwd_engine.hpp"

namespace ldist {

namespace shortk {
constexpr int BM = 64, BN = 32, NT = 512, NGROUP = 4, WIN = 8;
constexpr int KQ = NGROUP * WIN;                  // K is padded to a multiple of this
constexpr int MAXWIN = 10;                        // windows per k range the kernel is built for: K <= 320
inline int padded_k(int K) { return (K + KQ - 1) / KQ * KQ; }
// panels, four value slabs (float) and four window slabs (one byte per output: at most 40 windows)
inline size_t lds_bytes(int Kp) { return ((size_t)Kp * (BM + BN) + NGROUP * BM * BN) * sizeof(float) + NGROUP * BM * BN; }
// Place of (output n, row m) in the merge area: row-contiguous like the output tensor, with m XORed by a
// constant of n's group of four, so that the 64 lanes of a wave (8 groups of outputs x 8 groups of rows, 16 bytes
// each) spread over all banks when they park their patch, instead of over eight 16-byte slots.
__device__ __forceinline__ constexpr int cslot(int n, int m) {
    return n * BM + (m ^ ((((n >> 2) & 7) << 2) | (((n >> 2) & 1) << 5)));
}
// Byte offset of (output n, row m) in a window slab: four neighbouring rows share a 32-bit word, words are laid
// out rows-of-four major with n XORed by two bits of the row group, which spreads a wave's 64 word stores (and
// the finishing lanes' byte reads) over the banks.
__device__ __forceinline__ constexpr int bslot(int n, int m) { return (((m >> 2) * BN + (n ^ ((m >> 3) & 3))) << 2) | (m & 3); }
// The output that lane l (= row l of the tile) of wave v finishes in round r, see the finish phase of the kernel.
__device__ __forceinline__ constexpr int finish_output(int l, int v, int r) {
    return ((((l & 3) | ((l >> 5) << 2)) ^ v) << 2) | (((l >> 2) & 3) ^ r);
}
static_assert(BN == 32 && NT == 512, "finish_output: eight waves x four rounds cover 32 outputs");
}  // namespace shortk

// NW = windows per k range = padded K / 32; the window loop is unrolled over it, so that the parked loads are
// named registers and no branch stands between a load and the write that waits for it.
template <int NW>
__global__ void __launch_bounds__(shortk::NT, 2)
inf_forward_shortk_kernel(const float* __restrict__ input, const float* __restrict__ weight,
                          float* __restrict__ output, int32_t* __restrict__ pos, Dims d, int tiles_total) {
    using namespace shortk;
    constexpr int Kp = NW * KQ, nwin = NW, Kg = NW * WIN;
    extern __shared__ __align__(16) float lds[];
    float* X = lds;                         // [Kp][BM]
    float* W = lds + (size_t)Kp * BM;       // [Kp][BN]
    float* slab_v = W + (size_t)Kp * BN;    // [NGROUP][BN][BM] values per k range, see cslot(); slab 0 then holds the
    int* out_p = reinterpret_cast<int*>(slab_v + BM * BN);      // finished values and slab 1 (as integers) the finished pos
    unsigned char* slab_w = reinterpret_cast<unsigned char*>(slab_v + NGROUP * BM * BN);   // [NGROUP][..] windows, see bslot()

    const int tid = threadIdx.x;
    const int K = d.K, HW = d.HW;
    // Workgroup w takes tiles w, w + grid, w + 2 grid, ...: at any time the workgroups then read neighbouring
    // pieces of the input (with a contiguous run per workgroup they would all sit at the same offset inside
    // their images, i.e. on the same few memory channels).  Tiles are ordered rows first, so the weight panel
    // changes only when a workgroup's walk crosses into the next output tile or group.
    const int t_begin = blockIdx.x, t_step = gridDim.x, t_end = tiles_total;
    if (t_begin >= t_end) return;           // the whole workgroup leaves together

    const int lane = tid & 63, wave = tid >> 6;
    const int half = wave / NGROUP, grp = wave % NGROUP;
    const int tx = lane % 8, ty = lane / 8;

    // The wave's block of the input panel: rows half*32.. of the tile, k in [grp*Kg, (grp+1)*Kg).  In pass p a lane
    // takes four rows (consecutive positions of one image: HW % 4 == 0) at k = grp*Kg + 8 p + lane / 8.
    const int lrow = half * 32 + (lane % 8) * 4, lk = grp * Kg + lane / 8;
    typedef float F4 __attribute__((ext_vector_type(4)));
    typedef int I4 __attribute__((ext_vector_type(4)));
    F4 park[NW];
    // Buffer loads: the descriptor of the whole input in scalar registers, the lane's byte offset of (its four rows,
    // k = lk) of the tile in one register, the pass's k rows as the scalar offset.  An offset of all ones lies outside
    // the descriptor's 2 GB range and reads as zeros: that is how rows past M, k past K and the tile after the last
    // come out as zeros, without a branch or a predicate (the host checks that the input is smaller than 2 GB).
    // The loads and the waits for them are written out (inline assembly): the compiler's own wait in front of the
    // first panel write of a tile was for all outstanding loads, the youngest of which is two windows old, and
    // the tail of the memory latency showed (0.29 ms against 0.27 ms with the same loads served from L2).  Written
    // out, every panel write waits for its own load only: when pass p of a tile is written, the passes behind it, the
    // next tile's pass 0 and that tile's passes up to p have been issued since -- NW - 1 loads, at every p and for
    // the first tile too (its loads go out in one run before the loop), plus at most the two stores of a flush.  So
    // "at most NW - 1 memory operations outstanding" means the load has returned; the loads of load_w() are issued and
    // waited for while all of these are older, which keeps the compiler's own counts for them on the safe side.
    const unsigned long long xbase = reinterpret_cast<unsigned long long>(input);
    const I4 xrs = {(int)(unsigned)xbase, (int)(unsigned)((xbase >> 32) & 0xffffu), (int)0x80000000u, 0x00020000};
    // k of this range that exist: whole passes below p_full, lanes with lane / 8 < rem in pass p_full, none above
    const int k_valid = min(max(K - grp * Kg, 0), Kg), p_full = k_valid / WIN, rem = k_valid % WIN;
    struct Offsets { unsigned all, edge; };
    auto x_offsets = [&](int t) -> Offsets {
        Offsets o = {~0u, ~0u};
        if (t < t_end) {
            const int tm = t % d.tiles_m, g = (t / d.tiles_m) / d.tiles_n;
            const int m = tm * BM + lrow;
            if (m < d.M) {                       // HW % 4 == 0: four rows are inside the tensor together
                const int b = m / HW, hw = m % HW;
                o.all = (unsigned)((((size_t)(b * d.G + g) * K + lk) * HW + hw) * sizeof(float));
                if (lane / 8 < rem) o.edge = o.all;
            }
        }
        return o;
    };
    auto issue_pass = [&](int p, const Offsets& o) {
        const unsigned off = p < p_full ? o.all : (p == p_full ? o.edge : ~0u);
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"
                     : "=v"(park[p])
                     : "v"(off), "s"(xrs), "s"(p * WIN * HW * (int)sizeof(float)));
    };
    float* const xblock = X + (size_t)lk * BM + lrow;
    auto store_pass = [&](int p) {
        asm volatile("s_waitcnt vmcnt(%1)" : "+v"(park[p]) : "n"(NW - 1));
        *reinterpret_cast<F4*>(xblock + p * WIN * BM) = park[p];
    };
    // weight panel of (group g, output tile tn): lanes run along k, a lane takes four neighbouring outputs
    auto load_w = [&](int g, int tn) {
        const int n0 = tn * BN;
        const int items = Kp * (BN / 4);
#pragma unroll 1
        for (int i0 = tid; i0 < items; i0 += 2 * NT) {
            float4 wv[2];
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int i = i0 + e * NT;
                wv[e] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (i < items) {
                    const int kw = i % Kp, n = n0 + (i / Kp) * 4;
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
            for (int e = 0; e < 2; e++) {
                const int i = i0 + e * NT;
                if (i < items) {
                    const int kw = i % Kp;
                    *reinterpret_cast<float4*>(W + kw * BN + (i / Kp) * 4) = wv[e];
                }
            }
        }
    };

    // Tile -> global, from slabs 0 and 1: a lane stores four neighbouring rows of one output with 128-bit stores.
    // A tile's results go out at the start of the next tile.
    auto flush = [&](int t) {
        const int tm = t % d.tiles_m, wkey = t / d.tiles_m;
        const int tn = wkey % d.tiles_n, g = wkey / d.tiles_n;
        const int nl = tid / (BM / 4), mq = tid % (BM / 4);
        const int o = cslot(nl, mq * 4);
        const int m = tm * BM + mq * 4, n = tn * BN + nl;
        if (m < d.M && n < d.NG) {                     // HW % 4 == 0: the four rows lie inside the tensor and one image
            const int b = m / HW, hw = m % HW;
            const size_t at = ((size_t)(b * d.G + g) * d.NG + n) * HW + hw;
            *reinterpret_cast<float4*>(output + at) = *reinterpret_cast<const float4*>(slab_v + o);
            *reinterpret_cast<int4*>(pos + at) = *reinterpret_cast<const int4*>(out_p + o);
        }
    };

    int w_loaded = -1;
    {
        const Offsets first = x_offsets(t_begin);
#pragma unroll
        for (int p = 0; p < NW; p++) issue_pass(p, first);
    }
#pragma unroll 1
    for (int t = t_begin; t < t_end; t += t_step) {
        const int wkey = t / d.tiles_m;
        if (wkey != w_loaded) {   // every lane of the previous tile is past its epilogue
            load_w(wkey / d.tiles_n, wkey % d.tiles_n);
            w_loaded = wkey;
            __syncthreads();
        }
        const Offsets next = x_offsets(t + t_step);      // all ones behind the last tile: those loads read zeros
        // The first window's write waits for this tile's parked loads, all of them a window old or older.  The flush
        // comes after it: the wait counts stores too, and behind the flush it would wait for those.
        store_pass(0);
        issue_pass(0, next);
        if (t > t_begin) flush(t - t_step);

        // ---- the reduction: the wave takes rows half*32.. of the tile and k in [grp*Kg, (grp+1)*Kg) --------
        float accA[4][4], accB[4][4];
        int widx[4][4];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) { accA[i][j] = 0.f; accB[i][j] = 0.f; widx[i][j] = 0; }
        const float* xp = X + (size_t)grp * Kg * BM + half * 32 + ty * 4;
        const float* wp = W + (size_t)grp * Kg * BN + tx * 4;
        float4 xa[2], wa[2], xb[2], wb[2];
        auto fetch = [&](float4 (&xf)[2], float4 (&wf)[2], int kk) {   // rows kk, kk + 1 of the current window
#pragma unroll
            for (int e = 0; e < 2; e++) {
                xf[e] = *reinterpret_cast<const float4*>(xp + (kk + e) * BM);
                wf[e] = *reinterpret_cast<const float4*>(wp + (kk + e) * BN);
            }
        };
        // One window: cur continues the running maximum from prev (prev is left alone), so the window raised the
        // maximum iff cur > prev afterwards.  The arrays swap roles from window to window: nothing is copied.
        // Four pairs of k; the next pair's operands are fetched while the current pair is reduced, the first pair
        // of the next window during the last reduction (after the last window that reads rows of the next range
        // or just behind the panel, inside the allocation; they are never used).
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
            // Eight compares into their own scalar register pairs, then their selects: a select straight after its
            // compare (what the compiler makes of the plain form) waits two cycles for the lane mask.  The empty asm
            // statements keep their order: the first kind keeps a mask from being folded back into the plain form,
            // the second ends a group of eight.
#pragma unroll
            for (int i = 0; i < 4; i += 2) {
                unsigned long long raised[2][4];
#pragma unroll
                for (int a = 0; a < 2; a++)
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        raised[a][j] = __builtin_amdgcn_fcmpf(cur[i + a][j], prev[i + a][j], 2 /* ordered > */);
                        asm volatile("" : "+s"(raised[a][j]));
                    }
#pragma unroll
                for (int a = 0; a < 2; a++)
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        if (__builtin_amdgcn_inverse_ballot_w64(raised[a][j])) widx[i + a][j] = wid;
                        asm volatile("" : "+v"(widx[i + a][j]));
                    }
            }
        };
        fetch(xa, wa, 0);
        // Window w + 1 of the block goes to LDS, and its registers take the same window of the next tile, before
        // window w is reduced: the reads of window w + 1 start in the last quarter of window w.
#pragma unroll
        for (int w = 0; w < NW; w++) {
            if (w + 1 < NW) {
                store_pass(w + 1);
                issue_pass(w + 1, next);
            }
            if (w % 2 == 0) window(accA, accB, w); else window(accB, accA, w);
        }
        float (&acc)[4][4] = NW % 2 == 1 ? accB : accA;   // where the last window left the maxima
        __syncthreads();      // every lane has read the previous tile's results (flush) out of slabs 0 and 1

        // ---- every wave parks its patch in the slab of its k range: values as 128-bit words of four rows, windows
        // (counted inside the range: they fit a byte) as one word of four rows
        {
            float* sv = slab_v + grp * (BM * BN);
            unsigned* sw = reinterpret_cast<unsigned*>(slab_w + grp * (BM * BN));
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int n = tx * 4 + j, m = half * 32 + ty * 4;
                *reinterpret_cast<float4*>(sv + cslot(n, m)) = make_float4(acc[0][j], acc[1][j], acc[2][j], acc[3][j]);
                sw[bslot(n, m) >> 2] = (unsigned)widx[0][j] | ((unsigned)widx[1][j] << 8) | ((unsigned)widx[2][j] << 16) |
                                       ((unsigned)widx[3][j] << 24);
            }
        }
        __syncthreads();

        // ---- an output is finished by one lane: the four ranges in ascending k (a later range wins only with a
        // strictly larger value), then the lowest k inside the winner's window, from the panels.  Every lane reads a
        // different window, i.e. other rows of the panels, so lanes must differ in the column they read or they meet
        // in one bank: lane l of a wave takes row l of the tile (64 different columns of X) and, in round r of wave v,
        // output finish_output(l, v, r): over the eight waves and four rounds every output of the row once, every
        // output twice per wave instruction (32 columns of W), and -- what the choice of lane bits is for -- the 64
        // value words cslot() and the 64 window bytes bslot() of a wave instruction in 64 different banks: the group
        // of four outputs, which both slots XOR into the row's place, comes from lane bits 0, 1 and 5, which the row's
        // own bits 2..4 do not cancel (with output (l + r) % 32 the slabs were read through eight banks).
        {
            constexpr int ROUNDS = BN / (NT / 64);
            const int ml = lane;
            int o[ROUNDS], kb[ROUNDS], pfound[ROUNDS];
            float v[ROUNDS];
            // all slab reads first, then all panel reads, then all writes: a write to the merge area between two
            // rounds would order the next round's reads behind it
            float vq[ROUNDS][NGROUP];
            int wq[ROUNDS][NGROUP];
#pragma unroll
            for (int rr = 0; rr < ROUNDS; rr++) {
                const int nl = finish_output(lane, wave, rr);
                const int ob = bslot(nl, ml);
                o[rr] = cslot(nl, ml);
#pragma unroll
                for (int q = 0; q < NGROUP; q++) {
                    vq[rr][q] = slab_v[q * (BM * BN) + o[rr]];
                    wq[rr][q] = slab_w[q * (BM * BN) + ob];
                }
            }
            // The values exist here, whatever the comparisons below say: otherwise the compiler moves each read behind
            // the comparison that needs it, and the reads wait for one another.
#pragma unroll
            for (int rr = 0; rr < ROUNDS; rr++)
                asm volatile("" : "+v"(vq[rr][0]), "+v"(vq[rr][1]), "+v"(vq[rr][2]), "+v"(vq[rr][3]), "+v"(wq[rr][0]),
                             "+v"(wq[rr][1]), "+v"(wq[rr][2]), "+v"(wq[rr][3]));
            static_assert(NGROUP == 4, "the statement above names four ranges");
#pragma unroll
            for (int rr = 0; rr < ROUNDS; rr++) {
                v[rr] = vq[rr][0];
                int wsel = wq[rr][0];
#pragma unroll
                for (int q = 1; q < NGROUP; q++) {
                    const bool gt = vq[rr][q] > v[rr];
                    v[rr] = gt ? vq[rr][q] : v[rr];
                    wsel = gt ? wq[rr][q] + q * nwin : wsel;
                }
                kb[rr] = wsel * WIN;
            }
#pragma unroll
            for (int rr = 0; rr < ROUNDS; rr++) {
                const int nl = finish_output(lane, wave, rr);
                const float* xr = X + kb[rr] * BM + ml;
                const float* wr = W + kb[rr] * BN + nl;
                float xv[WIN], wv[WIN];
#pragma unroll
                for (int e = 0; e < WIN; e++) { xv[e] = xr[e * BM]; wv[e] = wr[e * BN]; }
                int p = 0;
#pragma unroll
                for (int e = WIN - 1; e >= 0; e--) {   // descending: the lowest match is written last
                    const float df = xv[e] - wv[e];
                    if (__builtin_fabsf(df) == v[rr]) p = (kb[rr] + e) | (__float_as_int(df) & 0x80000000);
                }
                pfound[rr] = v[rr] > 0.f ? p : 0;      // v == 0: the reference leaves pos = 0
            }
#pragma unroll
            for (int rr = 0; rr < ROUNDS; rr++) {      // slabs 0 and 1 now carry the tile's results; nobody else
                slab_v[o[rr]] = v[rr];                 // reads these two words
                out_p[o[rr]] = pfound[rr];
            }
        }
        __syncthreads();   // the panels are free for the next tile; its results wait in the merge area
    }
    asm volatile("s_waitcnt vmcnt(0)");   // the loads issued for the tile after the last (zeros) have landed before the wave ends
    flush(t_begin + (t_end - 1 - t_begin) / t_step * t_step);
}

// Whether the kernel above serves the problem: conv layout with rows in aligned groups of four, and a K whose
// panels fit LDS.
bool inf_forward_shortk_applicable(const Problem& pr, const void* input, const void* output, const void* pos) {
    if (pr.HW == 1 || pr.HW % 4 != 0) return false;
    if (!aligned16(input) || !aligned16(output) || !aligned16(pos)) return false;
    if ((size_t)pr.B * pr.G * pr.K * pr.HW * sizeof(float) >= (size_t)1 << 31) return false;   // 32-bit buffer offsets
    const int Kp = shortk::padded_k(pr.K);
    return Kp / shortk::KQ <= shortk::MAXWIN && shortk::lds_bytes(Kp) <= 160 * 1024;
}

template <int NW>
static hipError_t launch_shortk(unsigned grid, size_t lds, int device, hipStream_t stream, const float* input,
                                const float* weight, float* output, int32_t* pos, const Dims& d, int tiles) {
    static LdsRecord lds_allowed = {};
    if (hipError_t e = allow_lds(inf_forward_shortk_kernel<NW>, 160 * 1024, device, lds_allowed); e != hipSuccess) return e;
    hipLaunchKernelGGL(inf_forward_shortk_kernel<NW>, dim3(grid), dim3(shortk::NT), lds, stream, input, weight, output,
                       pos, d, tiles);
    return hipGetLastError();
}

hipError_t inf_forward_shortk(const float* input, const float* weight, float* output, int32_t* pos, const Problem& pr,
                              hipStream_t stream) {
    Dims d = make_dims(pr);
    d.tiles_m = (d.M + shortk::BM - 1) / shortk::BM;
    d.tiles_n = (d.NG + shortk::BN - 1) / shortk::BN;
    const int Kp = shortk::padded_k(pr.K);
    const size_t lds = shortk::lds_bytes(Kp);
    // one workgroup per CU
    const long tiles = (long)d.tiles_m * d.tiles_n * d.G;
    const unsigned grid = (unsigned)(tiles < pr.num_cu ? tiles : pr.num_cu);
#define LDIST_SHORTK(NW) \
    case NW: return launch_shortk<NW>(grid, lds, pr.device, stream, input, weight, output, pos, d, (int)tiles)
    switch (Kp / shortk::KQ) {
        LDIST_SHORTK(1); LDIST_SHORTK(2); LDIST_SHORTK(3); LDIST_SHORTK(4); LDIST_SHORTK(5);
        LDIST_SHORTK(6); LDIST_SHORTK(7); LDIST_SHORTK(8); LDIST_SHORTK(9); LDIST_SHORTK(10);
    }
#undef LDIST_SHORTK
    static_assert(shortk::MAXWIN == 10, "one case per window count");
    return hipErrorInvalidValue;   // not reached: inf_forward_shortk_applicable() admits ten windows at most
}

}  // namespace ldist

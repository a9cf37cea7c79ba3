// Both p-norm gradients of a convolution-shaped layer in one pass over the terms (reference
// model/norm_dist_cuda.cu:294-425 computes them in two kernels that each evaluate every term, on the unfolded
// input of model/norm_dist.py:132):
//   t[m,n,k]          = g[m,n] * (|x[m,k] - w[n,k]| / out[m,n])^(p-1) * sign(x - w)
//   grad_input [m,k]  = sum_n t[m,n,k]          grad_weight[n,k] += -sum_m t[m,n,k]
// with m = (image, output position), n the outputs of one group, k = (channel, tap) of the group's window.
//
// A layer of this shape has few outputs per group and very many rows, so a workgroup keeps the weights of its
// columns k for ALL outputs of the group in LDS, next to a tile of grad_weight sums of the same shape, and walks
// tiles of 64 rows.  Per tile it stages g and 1/out (NG x 64 each), and every lane reduces an 8 x 2 patch of
// (row, column) over n: a term is evaluated once, added to the lane's grad_input sum and to the column's partial sum
// over the lane's eight rows; the eight lanes that share the columns (half a DPP row) add those with three row
// shifts and the last of them, the only lane that ever touches these two words, adds the total onto the LDS tile of
// grad_weight.  (A DPP addition costs 4.4 clocks against 2.5 for a plain one: with a 4 x 4 patch the sixteen of them
// per output were 10 % of the loop's instructions and 15 % of its time.)  After its last tile the workgroup adds the
// LDS tile onto grad_weight with float atomics (one addend per workgroup and element).
//
// grad_input.  From the unfolded tensor (IMG = false) a tile is 64 columns wide and every element is written once.
// From the image (IMG = true, 3x3 windows) a pixel collects up to nine columns.  Float atomics for that, in memory
// or in LDS, cost as much as the arithmetic (151 M of them for 128 images of 128 x 32 x 32: 1.2 -> 2.0 ms), so the
// work is cut such that every pixel has one owner: a tile is 63 columns wide, i.e. seven whole channels, a
// workgroup takes whole images, and it keeps the image rows of its seven channel planes that its windows are
// still adding to in LDS (a ring of rows: a tile of 64 positions covers a few output rows, and everything above
// the next tile's first window is final).  A tile's sums are parked in LDS by (column, position), over the g and
// 1/out panels, which are free by then; then every pixel of the ring rows that the tile's windows reach fetches
// its up to nine (position, tap) entries -- two small tables give, per image row and tap row, the output row whose
// window has that tap there, and the same per column -- and adds them to its ring word in a fixed order.  Final
// rows are written to memory with plain stores and their ring rows cleared: grad_img needs no zero fill, and the
// result does not depend on the order in which workgroups run.  (Before the parked tile the sums joined the ring in
// nine rounds, one per tap, with a barrier between them: 1.57 against 1.38 ms on 128 x 128 x 32 x 32, p = 8.)
//
// IE = p - 1 for the multiply-only exponents (1, 2, 3, 7): the power is taken of the raw difference and the
// coefficient g / out^(p-1) is staged instead of g, unless a tile holds an output outside [2^-12, 2^12], which then
// takes the normalised difference like IE = 0 (any p > 1, through v_log_f32 / v_exp_f32).
#include "kernels.hpp"
#include "pow.hpp"
#include "tile.hpp"
#include "wave_reduce.hpp"

#include <algorithm>

namespace ldist {

namespace {

constexpr int TR = 64;              // rows of a tile
constexpr int TCP = 64;             // columns a tile has lanes for
constexpr int WLD = TCP + 4;        // row length of the weight and grad_weight tiles (rows 16-byte aligned)
constexpr int TI = 8, TJ = 2;       // a lane's patch: rows x columns; 64 / TI lanes share a column pair, inside one DPP row
constexpr int kPlanes = 7;          // IMG: channels per tile (63 columns)
constexpr size_t kMaxLds = 159 * 1024;   // all of LDS less the kernel's own static words

struct ConvBwd {
    int B, G, K, NG, HW, M;          // the unfolded problem: K = 9 channels per group (image) or CI / G
    int tiles_k;                     // column tiles per group
    int units, units_per_wg;         // what a workgroup walks: tiles of 64 rows (columns), whole images (image)
    int ring_rows;                   // IMG: image rows per channel plane held in LDS, a power of two
    int park_extra;                  // IMG: floats between the 1/out panel and the ring that the parked tile runs into
    int slices;                      // workgroups per (group, column tile): units / units_per_wg, rounded up
};

inline size_t lds_bytes(int NG, size_t plane_floats) {
    return ((size_t)2 * NG * WLD + (size_t)2 * NG * TR + plane_floats) * sizeof(float);
}

// IMG: a tile's grad_input sums are parked as [64 columns][64 positions] over the g and 1/out panels; what that
// takes beyond the panels' 2 * NG * 64 floats
inline int park_extra(int NG) { return std::max(0, TCP * TR - 2 * NG * TR); }

// IMG: the floats behind the panels: the parked tile's overhang, the ring of image rows, a word that stays zero,
// and the two tables (image row, tap row) -> output row and (image column, tap column) -> output column
inline size_t image_floats(int NG, int ring_rows, int H, int W) {
    return (size_t)park_extra(NG) + (size_t)kPlanes * ring_rows * W + 4 + 3 * (size_t)(H + W);
}

}  // namespace

template <bool IMG, int IE>
__global__ void __launch_bounds__(256, 4)   // four workgroups per CU is what LDS allows at 32 outputs per group: 128 registers
norm_conv_backward_kernel(const float* __restrict__ grad_output, const float* __restrict__ input,
                          const float* __restrict__ weight, const float* __restrict__ output,
                          float* __restrict__ grad_input, float* __restrict__ grad_weight, float e, ConvBwd d,
                          ImgWin win) {
    constexpr int TC = IMG ? 9 * kPlanes : TCP;   // columns per tile
    extern __shared__ __align__(16) float lds[];
    const int NG = d.NG, K = d.K;
    float* Ws = lds;                     // [NG][WLD]  w[n][k0 + c]
    float* Gw = Ws + NG * WLD;           // [NG][WLD]  sums for grad_weight[n][k0 + c]
    float* Cs = Gw + NG * WLD;           // [NG][TR]   g, or g / out^IE
    float* Rs = Cs + NG * TR;            // [NG][TR]   1 / out
    float* Fp = Rs + NG * TR + (IMG ? d.park_extra : 0);   // IMG: [kPlanes][ring_rows][W] gradient of the image rows still being added to
    const int tid = threadIdx.x;
    constexpr int TYN = TR / TI;             // lanes along the rows
    const int ty = tid % TYN, tx = tid / TYN;   // rows first: the lanes of a column group are neighbours in a DPP row
    // Consecutive workgroup ids go to different XCDs (8 per device, each with its own L2).  The grid is padded to a
    // multiple of 8 and remapped so that every XCD gets one contiguous run of (slice, group, column tile) with the
    // column tile fastest: the workgroups of one (slice, group) stage the same g and out, walk their units in step,
    // and now find each other's fetches in their L2 (config 4: five column tiles; 771 MB fetched per launch before).
    const int remapped = (int)(blockIdx.x % 8u) * (int)(gridDim.x / 8u) + (int)(blockIdx.x / 8u);
    const int pairs = d.tiles_k * d.G;
    if (remapped >= pairs * d.slices) return;   // padding
    const int slice = remapped / pairs, pair = remapped - slice * pairs;
    const int tk = pair % d.tiles_k, g = pair / d.tiles_k;
    const int k0 = tk * TC;
    const int u_begin = slice * d.units_per_wg, u_end = min(d.units, u_begin + d.units_per_wg);

    auto spower = [&](float u) {   // sign(u) * |u|^(p-1); by reference: the integer-exponent instantiations do not use e
        if constexpr (IE == 0) return __builtin_copysignf(pow_pos(__builtin_fabsf(u), e), u);   // u == 0: 0 either way
        else if constexpr (IE == 1) return u;
        else if constexpr (IE == 2) return u * __builtin_fabsf(u);
        else return pow_int<IE>(u);
    };

    for (int i = tid; i < NG * TCP; i += 256) {
        const int n = i / TCP, c = i % TCP;
        Ws[n * WLD + c] = (c < TC && k0 + c < K) ? weight[((size_t)g * NG + n) * K + k0 + c] : 0.f;
        Gw[n * WLD + c] = 0.f;
    }
    // General exponent (IE == 0): the term g * u * |u|^(p-2), u = (x - w) / out, is taken as
    //   g * (x - w) * exp2((p - 2) * log2|x - w| + log2(out^-(p-1)))
    // wherever that is accurate enough (the second summand staged per (row, output) in place of 1/out, so that the
    // division rides in the exponent's fused multiply-add: one plain instruction less per term, and no copy of the
    // sign).  The exponent is a difference of two numbers of the size of (p - 1) * |log2 out| for the terms that count,
    // each off by what the hardware logarithm is off by (one unit in the last place of |log2 out|), which the term
    // carries (p - 1) times as large: inside the tolerance of a gradient whose terms cancel (1e-6 * p / 8 of the sum
    // of their magnitudes) only while |log2 out| < 1.  So everything is taken in units of a power of two read off the
    // outputs of the workgroup's first tile (exact scalings of x, the weights and the outputs; the one nearest to the
    // geometric mean of the largest and the smallest of them), and a tile takes the form only if all its outputs lie within [1/2, 2] units
    // (voted on the barrier that follows the staging); other tiles divide first.
    float unit_inv = 1.0f;   // 1 / unit
    const float em1 = e - 1.0f;   // p - 2
    if constexpr (IE == 0) {
        float top = 0.f, nbot = -__builtin_inff();   // the largest and minus the smallest output of the first tile
        if (u_begin < u_end) {
            const int rows = IMG ? min(TR, d.HW) : min(TR, d.M - u_begin * TR);
            for (int i = tid; i < NG * TR; i += 256) {
                const int n = i / TR, r = i % TR;
                if (r < rows) {
                    size_t o;
                    if constexpr (IMG) {
                        o = ((size_t)(u_begin * d.G + g) * NG + n) * d.HW + r;
                    } else {
                        const int m = u_begin * TR + r, bi = m / d.HW;
                        o = ((size_t)(bi * d.G + g) * NG + n) * d.HW + (m - bi * d.HW);
                    }
                    const float ov = output[o];
                    if (ov > 0.f && ov < __builtin_inff()) {   // a NaN is not taken either
                        top = __builtin_fmaxf(top, ov);
                        nbot = __builtin_fmaxf(nbot, -ov);
                    }
                }
            }
        }
        top = wave_max(top);
        nbot = wave_max(nbot);
        __syncthreads();                       // Gw's zero fill above is complete
        if ((tid & 63) == 63) { Gw[tid >> 6] = top; Gw[4 + (tid >> 6)] = nbot; }
        __syncthreads();
        top = __builtin_fmaxf(__builtin_fmaxf(Gw[0], Gw[1]), __builtin_fmaxf(Gw[2], Gw[3]));
        nbot = __builtin_fmaxf(__builtin_fmaxf(Gw[4], Gw[5]), __builtin_fmaxf(Gw[6], Gw[7]));
        __syncthreads();
        if ((tid & 63) == 63) { Gw[tid >> 6] = 0.f; Gw[4 + (tid >> 6)] = 0.f; }
        // the power of two nearest (as a ratio) to the geometric mean of the two
        const float mid = __builtin_sqrtf(top) * __builtin_sqrtf(-nbot) * 1.41421356f;
        const int ex = min(100, max(-100, (int)((__float_as_uint(mid) >> 23) & 0xff) - 127));
        unit_inv = top > 0.f ? __uint_as_float((unsigned)(127 - ex) << 23) : 1.0f;
        for (int i = tid; i < NG * TCP; i += 256) Ws[(i / TCP) * WLD + i % TCP] *= unit_inv;   // each lane the words it wrote
    }
    // the lane's four columns: whether they exist, and for the image their channel plane and tap
    bool col_ok[TJ];
    int col_plane[TJ], col_tap[TJ], col_dh[TJ], col_dw[TJ];   // IMG: the column's channel plane inside the tile, its tap and the tap's offsets
    int col_off[TJ];                                      // IMG: where the tap lies from the window's corner, in the tile's planes of one image
#pragma unroll
    for (int j = 0; j < TJ; j++) {
        const int c = tx * TJ + j;
        col_ok[j] = c < TC && k0 + c < K;
        col_plane[j] = c / 9;
        col_tap[j] = c - col_plane[j] * 9;
        col_dh[j] = (col_tap[j] / 3) * win.D;
        col_dw[j] = (col_tap[j] - (col_tap[j] / 3) * 3) * win.D;
        col_off[j] = (col_plane[j] * win.H + col_dh[j]) * win.W + col_dw[j];
    }
    // IMG: the current image's planes of this tile, and its g and out rows of this group, behind buffer descriptors:
    // 32-bit offsets from a uniform base, and an offset of all ones (outside the 2 GB range: reads as zero) for
    // everything that is not there -- padding taps, rows past the image's last position, columns past K.
    __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(input), 0, (int)0x80000000u, 0x00020000);
    __amdgpu_buffer_rsrc_t g_rsrc = x_rsrc, o_rsrc = x_rsrc;

    // One tile: rows first_row .. first_row + 63 of the unfolded matrix, of which `rows` exist (IMG: rows of image b
    // from position pos0).  Leaves the grad_input sums of the lane's patch in acc.
    auto tile = [&](int first_row, int rows, int b, int pos0, float (&acc)[TI][TJ], WinRow (&wrow)[TI], size_t (&xoff)[TI]) {
        float q[TI][TJ];
        if constexpr (!IMG) {
#pragma unroll
            for (int i = 0; i < TI; i++) {
                const int r = min(ty * TI + i, rows - 1);
                const int m = first_row + r, bi = m / d.HW;
                xoff[i] = ((size_t)(bi * d.G + g) * K) * d.HW + (m - bi * d.HW);
            }
        }
#pragma unroll
        for (int i = 0; i < TI; i++) {
            const int corner = IMG ? wrow[i].h0 * win.W + wrow[i].w0 : 0;   // IMG: the window's corner in a plane (may lie in the padding)
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                acc[i][j] = 0.f;
                const bool ok = ty * TI + i < rows && col_ok[j];
                if constexpr (IMG) {   // the window's tap of column j: channel and offsets are the lane's constants
                    const int h = wrow[i].h0 + col_dh[j], w = wrow[i].w0 + col_dw[j];
                    // one select, no branches: the tests are combined bitwise
                    const bool in = ok & ((unsigned)h < (unsigned)win.H) & ((unsigned)w < (unsigned)win.W);
                    const unsigned o = in ? 4u * (unsigned)(corner + col_off[j]) : ~0u;
                    q[i][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(x_rsrc, o, 0, 0)) * unit_inv;
                } else {
                    q[i][j] = ok ? input[xoff[i] + (size_t)(k0 + tx * TJ + j) * d.HW] * unit_inv : 0.f;   // unit_inv: 1 unless IE == 0
                }
            }
        }
        // g and out of the tile's rows for every output of the group; rows are contiguous in memory
        bool unsafe = false;
        if constexpr (IMG) {
            // A lane takes row r = tid % 64 of outputs tid / 64, + 4, + 8, ...: four outputs per pass, their eight
            // loads in flight together (one output at a time, every load is waited for on its own).  Rows and outputs
            // that do not exist load nothing (all-ones offset) and stage 0.
            const int r = tid & (TR - 1);
            const unsigned row_off = 4u * (unsigned)(pos0 + r), out_stride = 4u * (unsigned)d.HW;
#pragma unroll 1
            for (int n0 = tid / TR; n0 < NG; n0 += 16) {
                float gv[4], ov[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int n = n0 + 4 * u;
                    const unsigned o = ((r < rows) & (n < NG)) ? row_off + (unsigned)n * out_stride : ~0u;
                    gv[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(g_rsrc, o, 0, 0));
                    ov[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(o_rsrc, o, 0, 0));
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int n = n0 + 4 * u;
                    if (n < NG) {
                        const float out = ov[u] * unit_inv;
                        float ri = 0.f;   // IE == 0: ri holds the output itself until the vote is in
                        if (r < rows) {
                            ri = IE > 0 ? __builtin_amdgcn_rcpf(out) : out;
                            // IE > 0: the factored form needs out^(p-1) inside the float range; IE == 0: the logarithmic form's range
                            unsafe |= IE > 0 ? !(out >= 0x1p-12f && out <= 0x1p12f) : !(out >= 0.5f && out <= 2.0f);
                        }
                        Cs[n * TR + r] = gv[u];
                        Rs[n * TR + r] = ri;
                    }
                }
            }
        } else {
            // the same walk from the unfolded layout: a tile's rows may belong to two images, so a lane keeps the
            // element offset of its row in output 0 and steps by HW per output
            const int r = tid & (TR - 1);
            const int m = first_row + min(r, rows - 1), bi = m / d.HW;
            const size_t row0 = ((size_t)(bi * d.G + g) * NG) * d.HW + (m - bi * d.HW);
#pragma unroll 1
            for (int n0 = tid / TR; n0 < NG; n0 += 16) {
                float gv[4], ov[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int n = min(n0 + 4 * u, NG - 1);   // past the last output: a valid address, the value is not used
                    gv[u] = grad_output[row0 + (size_t)n * d.HW];
                    ov[u] = output[row0 + (size_t)n * d.HW];
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int n = n0 + 4 * u;
                    if (n < NG) {
                        const float out = ov[u] * unit_inv;
                        float c = 0.f, ri = 0.f;   // IE == 0: ri holds the output itself until the vote is in
                        if (r < rows) {
                            c = gv[u];
                            ri = IE > 0 ? __builtin_amdgcn_rcpf(out) : out;
                            unsafe |= IE > 0 ? !(out >= 0x1p-12f && out <= 0x1p12f) : !(out >= 0.5f && out <= 2.0f);
                        }
                        Cs[n * TR + r] = c;
                        Rs[n * TR + r] = ri;
                    }
                }
            }
        }
        const bool factored = !__syncthreads_or(unsafe);   // also: the panels are written
        if (IE > 0 && factored) {
            for (int i = tid; i < NG * TR; i += 256) Cs[i] *= pow_int<(IE > 0 ? IE : 1)>(Rs[i]);   // each lane its own elements
            __syncthreads();
        }
        if constexpr (IE == 0) {   // each lane its own elements: out -> 1/out, or the logarithmic form's summand
            for (int i = tid; i < NG * TR; i += 256) {
                const float out = Rs[i];
                if (i % TR >= rows) {
                    Rs[i] = factored ? -__builtin_inff() : 0.f;   // rows that do not exist: a power of 0, a factor 0
                } else if (factored) {
                    // log2 of out^-(p-1) from the output itself; what the product loses when it is rounded to a
                    // float goes into g as a factor
                    const float lo = __builtin_amdgcn_logf(out), hi = -e * lo;
                    Cs[i] *= __builtin_amdgcn_exp2f(__builtin_fmaf(-e, lo, -hi));
                    Rs[i] = hi;
                } else {
                    Rs[i] = __builtin_amdgcn_rcpf(out);
                }
            }
            __syncthreads();
        }
        auto reduce = [&](auto term) {   // term(x - w, 1/out): the power that g (or g / out^IE) multiplies
            for (int n = 0; n < NG; n++) {
                float cv[TI], rv[TI], wv[TJ];
#pragma unroll
                for (int i = 0; i < TI; i += 4) {
                    const float4 c4 = *reinterpret_cast<const float4*>(Cs + n * TR + ty * TI + i);
                    const float4 r4 = *reinterpret_cast<const float4*>(Rs + n * TR + ty * TI + i);
                    cv[i] = c4.x; cv[i + 1] = c4.y; cv[i + 2] = c4.z; cv[i + 3] = c4.w;
                    rv[i] = r4.x; rv[i + 1] = r4.y; rv[i + 2] = r4.z; rv[i + 3] = r4.w;
                }
                if constexpr (TJ == 4) {
                    const float4 w4 = *reinterpret_cast<const float4*>(Ws + n * WLD + tx * 4);
                    wv[0] = w4.x; wv[1] = w4.y; wv[2] = w4.z; wv[3] = w4.w;
                } else {
                    const float2 w2 = *reinterpret_cast<const float2*>(Ws + n * WLD + tx * 2);
                    wv[0] = w2.x; wv[1] = w2.y;
                }
                float s[TJ];
#pragma unroll
                for (int j = 0; j < TJ; j++) s[j] = 0.f;
#pragma unroll
                for (int i = 0; i < TI; i++)
#pragma unroll
                    for (int j = 0; j < TJ; j++) {
                        const float sp = term(q[i][j] - wv[j], rv[i]);
                        acc[i][j] = __builtin_fmaf(cv[i], sp, acc[i][j]);   // two fused multiply-adds, not a shared
                        s[j] = __builtin_fmaf(cv[i], sp, s[j]);             // product and two additions
                    }
                float tot[TJ];
#pragma unroll
                for (int j = 0; j < TJ; j++) tot[j] = dpp_lanes_total<TYN>(s[j]);
                if (ty == TYN - 1) {   // d/dw of |x - w| is minus d/dx
                    float* gp = Gw + n * WLD + tx * TJ;
                    if constexpr (TJ == 4) {
                        float4 v = *reinterpret_cast<float4*>(gp);
                        v.x -= tot[0]; v.y -= tot[1]; v.z -= tot[2]; v.w -= tot[3];
                        *reinterpret_cast<float4*>(gp) = v;
                    } else {
                        float2 v = *reinterpret_cast<float2*>(gp);
                        v.x -= tot[0]; v.y -= tot[1];
                        *reinterpret_cast<float2*>(gp) = v;
                    }
                }
            }
        };
        if (IE > 0 && factored) reduce([&](float df, float) { return spower(df); });
        else if (IE == 0 && factored)
            reduce([&](float df, float c4) { return df * __builtin_amdgcn_exp2f(__builtin_fmaf(__builtin_amdgcn_logf(__builtin_fabsf(df)), em1, c4)); });
        else reduce([&](float df, float ri) { return spower(df * ri); });
    };

    float acc[TI][TJ];
    WinRow wrow[TI];
    size_t xoff[TI];
    if constexpr (IMG) {
        const int H = win.H, W = win.W, R = d.ring_rows, first_ch = tk * kPlanes;
        const int planes = min(kPlanes, win.CG - first_ch);
        // behind the ring: a word that stays zero (what a pixel reads for a tap that has no position in the tile), and
        // the tables that turn (image row, tap row) and (image column, tap column) into the output row (times WO) and
        // the output column whose window has that tap there; a large negative number where there is none
        float* const zero_word = Fp + kPlanes * R * W;
        int* const HT = reinterpret_cast<int*>(zero_word + 4);
        int* const WT = HT + 3 * H;
        float* const Pk = Cs;   // [64][64]: the tile's grad_input sums by (column, position), over the two panels
        constexpr int kNone = -(1 << 20);
        if (tid < 4) zero_word[tid] = 0.f;
        for (int i = tid; i < 3 * (H + W); i += 256) {
            const bool row = i < 3 * H;
            const int e = row ? i : i - 3 * H, at = e / 3, t = e - at * 3;
            const int lim = row ? win.HO : win.WO;
            const int hh = at + win.P - t * win.D, o = hh / win.S;
            const bool ok = hh >= 0 && o * win.S == hh && o < lim;
            HT[i] = ok ? (row ? o * win.WO : o) : kNone;   // WT follows HT
        }
        const float inv_w = 1.0f / (float)W;
        for (int b = u_begin; b < u_end; b++) {
            float* dst = grad_input + ((size_t)b * win.C + g * win.CG + first_ch) * H * W;
            // Writes image rows h_from .. h_to - 1 of the planes to memory and clears their ring rows.  Rows more than
            // a ring away from h_from have never been touched (the windows reach less far): they are zero.
            auto flush_rows = [&](int h_from, int h_to) {
                const int nrow = h_to - h_from;
                for (int i = tid; i < planes * nrow * W; i += 256) {
                    const int w = i % W, rest = i / W, hr = rest % nrow, c = rest / nrow, h = h_from + hr;
                    float v = 0.f;
                    if (hr < R) {
                        float* cell = Fp + (c * R + (h & (R - 1))) * W + w;
                        v = *cell;
                        *cell = 0.f;
                    }
                    dst[(c * H + h) * W + w] = v;
                }
            };
            for (int i = tid; i < kPlanes * R * W; i += 256) Fp[i] = 0.f;   // the first tile's barriers come before its use
            x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<float*>(input + ((size_t)b * win.C + g * win.CG + first_ch) * H * W), 0, (int)0x80000000u, 0x00020000);
            g_rsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<float*>(grad_output + (size_t)(b * d.G + g) * NG * d.HW), 0, (int)0x80000000u, 0x00020000);
            o_rsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<float*>(output + (size_t)(b * d.G + g) * NG * d.HW), 0, (int)0x80000000u, 0x00020000);
            // the corners of the windows of the lane's positions, moved on by 64 positions per tile (positions past
            // the image's last one are never used: every use asks for i < rows)
#pragma unroll
            for (int i = 0; i < TI; i++) {
                const int ho = (ty * TI + i) / win.WO, wo = (ty * TI + i) - ho * win.WO;
                wrow[i].b = b;
                wrow[i].h0 = ho * win.S - win.P;
                wrow[i].w0 = wo * win.S - win.P;
            }
            const int step_rows = TR / win.WO;
            const int step_h = step_rows * win.S, step_w = (TR - step_rows * win.WO) * win.S;
            const int wrap_w = win.WO * win.S, end_w = wrap_w - win.P;   // a corner's column stays below end_w
            int flushed = 0;   // image rows below this one are in memory
            for (int pos0 = 0; pos0 < d.HW; pos0 += TR) {
                const int rows = min(TR, d.HW - pos0);
                if (pos0 > 0) {
#pragma unroll
                    for (int i = 0; i < TI; i++) {
                        wrow[i].h0 += step_h;
                        wrow[i].w0 += step_w;
                        if (wrow[i].w0 >= end_w) { wrow[i].w0 -= wrap_w; wrow[i].h0 += win.S; }
                    }
                }
                tile(0, rows, b, pos0, acc, wrow, xoff);
                // rows above this tile's first window are final (the last tile's rounds ended with a barrier)
                const int h_lo = min(H, max(flushed, (pos0 / win.WO) * win.S - win.P));
                if (h_lo > flushed) flush_rows(flushed, h_lo);
                flushed = h_lo;
                __syncthreads();   // ring rows cleared above may be this tile's; every lane is done with the panels
                // The tile's sums join the planes.  They are parked by (column, position) over the two panels, and
                // every pixel that a window of this tile can reach fetches its up to nine (position, tap) entries
                // and adds them to its ring word: one owner per pixel, a fixed order of the nine, no rounds.
#pragma unroll
                for (int j = 0; j < TJ; j++)
#pragma unroll
                    for (int i = 0; i < TI; i += 4)
                        *reinterpret_cast<float4*>(Pk + (tx * TJ + j) * TR + ty * TI + i) =
                            make_float4(acc[i][j], acc[i + 1][j], acc[i + 2][j], acc[i + 3][j]);
                __syncthreads();
                const int last = pos0 + rows - 1;
                const int h_first = max(0, (pos0 / win.WO) * win.S - win.P);
                const int h_last = min(H - 1, (last / win.WO) * win.S - win.P + 2 * win.D);
                const int nrow = h_last - h_first + 1;
                const float inv_nrow = 1.0f / (float)nrow;
                for (int i = tid; i < planes * nrow * W; i += 256) {
                    // i = (c * nrow + hr) * W + w; quotients of small numbers through the reciprocal
                    const int rest = (int)(((float)i + 0.5f) * inv_w), w = i - rest * W;
                    const int c = (int)(((float)rest + 0.5f) * inv_nrow), h = h_first + (rest - c * nrow);
                    const float* col = Pk + c * 9 * TR - pos0;
                    int hb[3], wb[3];
#pragma unroll
                    for (int t = 0; t < 3; t++) {
                        hb[t] = HT[h * 3 + t];
                        wb[t] = WT[w * 3 + t];
                    }
                    float sum = 0.f;
#pragma unroll
                    for (int th = 0; th < 3; th++)
#pragma unroll
                        for (int tw = 0; tw < 3; tw++) {
                            const int pos = hb[th] + wb[tw];   // negative when either has no window
                            const bool in = (unsigned)(pos - pos0) < (unsigned)rows;
                            sum += *(in ? col + (th * 3 + tw) * TR + pos : zero_word);
                        }
                    Fp[(c * R + (h & (R - 1))) * W + w] += sum;
                }
                __syncthreads();   // the next tile stages over the parked sums; its flush reads the ring
            }
            flush_rows(flushed, H);
            __syncthreads();       // before the ring is used for the next image
        }
    } else {
        for (int t = u_begin; t < u_end; t++) {
            const int m0 = t * TR, rows = min(TR, d.M - m0);
            tile(m0, rows, 0, 0, acc, wrow, xoff);
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++)
                    if (ty * TI + i < rows && col_ok[j]) grad_input[xoff[i] + (size_t)(k0 + tx * TJ + j) * d.HW] = acc[i][j];
            __syncthreads();   // the next tile overwrites the panels
        }
    }
    __syncthreads();
    for (int i = tid; i < NG * TCP; i += 256) {
        const int n = i / TCP, c = i % TCP;
        if (c < TC && k0 + c < K) atomicAdd(grad_weight + ((size_t)g * NG + n) * K + k0 + c, Gw[n * WLD + c]);
    }
}

namespace {

// Image rows per plane the ring must hold: the most that the windows of one tile of 64 positions cover (tiles start
// at multiples of 64 inside an image), rounded up to a power of two.
int ring_rows_for(const ImgWin& win, int HW) {
    int out_rows = 1;
    for (int pos0 = 0; pos0 < HW; pos0 += TR) {
        const int last = std::min(HW, pos0 + TR) - 1;
        out_rows = std::max(out_rows, last / win.WO - pos0 / win.WO + 1);
        if (pos0 / TR >= win.WO) break;   // the pattern of starts inside an output row repeats by then
    }
    const int rows = (out_rows - 1) * win.S + 2 * win.D + 1;
    int ring = 1;
    while (ring < rows) ring *= 2;
    return ring;
}

template <bool IMG, int IE>
hipError_t launch_conv_backward(const float* grad_output, const float* input, const float* weight, const float* output,
                                float* grad_input, float* grad_weight, float p, const Problem& pr, const ImgWin& win,
                                hipStream_t stream) {
    ConvBwd d{pr.B, pr.G, pr.K, pr.NG, pr.HW, pr.B * pr.HW, 0, 0, 0, 0, 0, 0};
    d.tiles_k = IMG ? (win.CG + kPlanes - 1) / kPlanes : (d.K + TCP - 1) / TCP;
    d.units = IMG ? pr.B : (d.M + TR - 1) / TR;
    const long pairs = (long)d.tiles_k * d.G;
    if constexpr (IMG) {
        d.ring_rows = ring_rows_for(win, pr.HW);
        d.park_extra = park_extra(d.NG);
    }
    const size_t lds = lds_bytes(d.NG, IMG ? image_floats(d.NG, d.ring_rows, win.H, win.W) : 0);
    // Units per workgroup.  A CU issues at the same rate whether two, three or four workgroups share it, so what a
    // launch takes is what the busiest CU has to work through: workgroups per CU (dealt round robin) times units per
    // workgroup.  With few long workgroups that is uneven -- 860 workgroups of three images on 256 CUs leave twelve
    // images on some CUs and nine on the others, a fifth above the mean -- so the choice minimises it, charging every
    // workgroup a fixed cost (its weight tile and the flush of its grad_weight tile at the end: about a third of a
    // 64-row tile) and the last one on a CU half its length (it runs partly alone, at half the CU's rate).  The number
    // of workgroups stays within sixteen times what the device holds at once.
    long per_cu = (long)(160 * 1024 / lds);
    if (per_cu > 8) per_cu = 8;
    if (per_cu < 1) per_cu = 1;
    const long resident = per_cu * pr.num_cu;
    long best = -1;
    double best_cost = 0;
    const double fixed = IMG ? 0.3 / std::max(1, (pr.HW + TR - 1) / TR) : 0.3;   // in units: an image is HW / 64 tiles
    const long lo = std::max(1L, ((long)d.units * pairs + 16 * resident - 1) / (16 * resident));
    for (long upw = lo; upw <= d.units && upw < lo + 4096; upw++) {
        const long wgs = pairs * ((d.units + upw - 1) / upw);
        const double cost = (double)((wgs + pr.num_cu - 1) / pr.num_cu) * ((double)upw + fixed) + 0.5 * (double)upw;
        if (best < 0 || cost < best_cost) { best = upw; best_cost = cost; }
    }
    d.units_per_wg = (int)best;
    const long slices = (d.units + d.units_per_wg - 1) / d.units_per_wg;
    d.slices = (int)slices;
    const long grid = (pairs * slices + 7) / 8 * 8;   // whole rounds of the eight XCDs; the padding exits at once
    auto kern = norm_conv_backward_kernel<IMG, IE>;
    static LdsRecord lds_allowed = {};
    // the limit is raised once, to the most any layer may ask for
    if (hipError_t e = allow_lds(kern, kMaxLds, pr.device, lds_allowed); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, stream, grad_output, input, weight,
                       output, grad_input, grad_weight, p - 1.0f, d, win);
    return hipGetLastError();
}

template <bool IMG>
hipError_t dispatch_conv_backward(const float* grad_output, const float* input, const float* weight, const float* output,
                                  float* grad_input, float* grad_weight, float p, const Problem& pr, const ImgWin& win,
                                  hipStream_t stream) {
    switch (small_int_power(p - 1.0f)) {
        case 1: return launch_conv_backward<IMG, 1>(grad_output, input, weight, output, grad_input, grad_weight, p, pr, win, stream);
        case 2: return launch_conv_backward<IMG, 2>(grad_output, input, weight, output, grad_input, grad_weight, p, pr, win, stream);
        case 3: return launch_conv_backward<IMG, 3>(grad_output, input, weight, output, grad_input, grad_weight, p, pr, win, stream);
        case 7: return launch_conv_backward<IMG, 7>(grad_output, input, weight, output, grad_input, grad_weight, p, pr, win, stream);
        default: return launch_conv_backward<IMG, 0>(grad_output, input, weight, output, grad_input, grad_weight, p, pr, win, stream);
    }
}

bool forced_on() { return g_tile_override == 0 || g_tile_override == 1; }   // tests and tuning

}  // namespace

// Whether the one-pass kernel takes a layer given as unfolded columns: the conv layout with enough rows to give
// every CU work, and few enough outputs per group for the four LDS tiles (NG KB).
bool norm_conv_backward_fused_applicable(const Problem& pr) {
    if (pr.HW == 1 || g_tile_override >= 2) return false;
    if (lds_bytes(pr.NG, 0) > kMaxLds) return false;
    return forced_on() || (long)pr.B * pr.HW >= 64L * pr.num_cu;
}

// The same for a layer given as an image: also the ring of image rows of seven channel planes must fit LDS.
bool norm_conv_backward_fused_image_applicable(const ConvGeom& q, int G, int CO, int num_cu) {
    if (g_tile_override >= 2 || (long)q.HO * q.WO <= 1) return false;
    const ImgWin win{q.C, q.C / G, q.H, q.W, q.HO, q.WO, q.S, q.P, q.D};
    if (lds_bytes(CO / G, image_floats(CO / G, ring_rows_for(win, q.HO * q.WO), q.H, q.W)) > kMaxLds) return false;
    // the kernel's 32-bit byte offsets: a tile's planes of one image, one image's outputs of a group
    if (4L * kPlanes * q.H * q.W >= (1L << 31) || 4L * (CO / G) * q.HO * q.WO >= (1L << 31)) return false;
    return forced_on() || (long)q.B * q.HO * q.WO >= 64L * num_cu;
}

// From the unfolded input (B, CI, HW): every element of grad_input is written, grad_weight is added to.
hipError_t norm_conv_backward_fused_columns(const float* grad_output, const float* input, const float* weight,
                                            const float* output, float* grad_input, float* grad_weight, float p,
                                            const Problem& pr, hipStream_t stream) {
    return dispatch_conv_backward<false>(grad_output, input, weight, output, grad_input, grad_weight, p, pr, ImgWin{}, stream);
}

// From the image (3x3 window): every element of grad_img is written, grad_weight is added to.
hipError_t norm_conv_backward_fused_image(const float* grad_output, const float* img, const float* weight,
                                          const float* output, float* grad_img, float* grad_weight, float p,
                                          const ConvGeom& q, int G, int CO, int num_cu, int device, hipStream_t stream) {
    const Problem pr{q.B, G, q.C / G * 9, CO / G, q.HO * q.WO, num_cu, device};
    const ImgWin win{q.C, q.C / G, q.H, q.W, q.HO, q.WO, q.S, q.P, q.D};
    return dispatch_conv_backward<true>(grad_output, img, weight, output, grad_img, grad_weight, p, pr, win, stream);
}

}  // namespace ldist

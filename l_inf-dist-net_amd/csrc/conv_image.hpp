// Launch shape shared by the kernels that run the 3x3 distance layer straight from images
// (inf_conv_forward.hip: values and argmax; bound_conv_forward.hip: interval bounds).
#pragma once
#include "kernels.hpp"

namespace ldist {
namespace convimg {

constexpr int kTM = 8, kTN = 4;   // positions x outputs per lane
constexpr int kCC = 4;            // channels per weight stage
constexpr int kTrack = 1;         // channels per recorded unit
constexpr int kKC = kCC * 9;      // k values per weight stage
constexpr int kMaxThreads = 256;
constexpr int kBNP = 68;          // row length of the weight stage: 64 outputs + 4, a constant so that reads take immediate offsets
constexpr int kWRegs = 9;         // weight words a lane carries from global to LDS per stage (64 outputs x 36 / 256)
// image words a lane carries per stage when the channels are staged (4 channels x rows held x padded width / lanes)
__host__ __device__ constexpr int x_regs(int S) { return S == 1 ? 7 : 10; }

struct ConvFwd {
    int B, G, CG, NG, K;         // images, groups, channels and outputs per group, K = 9*CG
    int H, W, HO, WO, P;         // image, output positions, padding
    int R, NR, WP, CGP;          // output rows per workgroup, image rows held, padded row length, CG rounded up to kCC
    int SEG, ML, NL, BN;         // 8-position segments per output row, lanes along positions / outputs, outputs per
                                 // workgroup
    int tiles_h, tiles_n;
    int vec_in, vec_out;         // 128-bit global loads of image rows / stores of results allowed
    int resident;                // 1: all channels of the image rows stay in LDS; 0: staged kCC channels at a time
    int xwords;                  // floats of the image area in LDS
    int cstride;                 // resident: floats between channels (NR*WP padded to 4 mod 8); staged: unused
};

constexpr size_t kLdsLimit = 160 * 1024;

// Fills the launch shape; false when this kernel does not cover the geometry.
// Channel stride of the resident image area: rows stay 16-byte aligned (a multiple of 4) and consecutive
// channels start 4 banks apart modulo 8, so that channel c begins at bank 4c mod 64.
inline int channel_stride(int plane) { return plane % 8 == 4 ? plane : plane + (4 - plane % 8 + 8) % 8; }

// nx: images staged side by side (1: the input; 2: lower and upper interval ends, which are always staged and may
// have any number of channels: that kernel masks the channels a last stage does not have).
inline bool plan(const ConvGeom& q, int G, int CO, ConvFwd& a, int nx = 1) {
    if (q.KH != 3 || q.KW != 3 || q.D != 1 || (q.S != 1 && q.S != 2)) return false;
    if (G <= 0 || q.C % G != 0 || CO % G != 0) return false;
    if ((long long)kCC * q.H * q.W >= (1LL << 28)) return false;   // staged loads pack the channel above 28 offset bits
    const int S = q.S, NXR = (7 * S + 2) / 4 + 1;
    a.B = q.B; a.G = G; a.CG = q.C / G; a.NG = CO / G; a.K = a.CG * 9;
    a.H = q.H; a.W = q.W; a.HO = q.HO; a.WO = q.WO; a.P = q.P;
    a.CGP = (a.CG + kCC - 1) / kCC * kCC;
    a.SEG = (q.WO + kTM - 1) / kTM;                  // a last segment may reach past the row: those positions are not stored
    // the last lane of a row reads NXR*4 words from column (SEG-1)*8*S; the image with its padding is W + 2P wide
    int wp = (a.SEG - 1) * kTM * S + NXR * 4;
    if (q.W + 2 * q.P > wp) wp = q.W + 2 * q.P;
    a.WP = (wp + 3) / 4 * 4;
    if (a.WP % 32 == 0) a.WP += 4;                     // rows of one lane's window in different banks
    // Outputs per workgroup: at most 64, split evenly over the tiles; more tiles when a workgroup of that
    // width would have too many lanes (wide images).
    const int quads = (a.NG + kTN - 1) / kTN;
    for (int pass = 0; pass < 2; pass++) {
        // pass 0: all channels resident in LDS; pass 1: channels staged (needs CG % kCC == 0, so that no
        // stage holds a channel that does not exist)
        const bool resident = pass == 0;
        if (resident && nx > 1) continue;
        if (g_conv_staging_override == 3) continue;
        if (g_conv_staging_override == 1 && !resident) continue;
        if (g_conv_staging_override == 2 && resident) continue;
        if (!resident && nx == 1 && a.CG % kCC != 0) continue;
        // Candidates: the fewest output tiles that fit and up to three more (a narrower workgroup may take more
        // rows, or rows that divide the image evenly); each further tile re-reads the image rows once more,
        // priced at 3 %.  Past those, more tiles are only tried until something fits at all.
        const int first_tiles = (quads + 15) / 16;
        bool have = false;
        double haveScore = -1.0;
        ConvFwd pick = a;
        for (int tiles_n = first_tiles; tiles_n <= quads; tiles_n++) {
            if (have && tiles_n > first_tiles + 3) break;
            const int NL = (quads + tiles_n - 1) / tiles_n;
            if (a.SEG * NL > kMaxThreads) continue;
            const int BN = NL * kTN;
            // rows per workgroup: the choice that keeps most lanes busy on a CU (LDS limit, 8 waves of this
            // register footprint, rows computed past the image bottom count as idle); ties take more rows
            int bestR = 0, bestWords = 0;
            double bestScore = -1.0;
            const int maxR = kMaxThreads / (a.SEG * NL);
            int forced = g_conv_rows_override;
            if (forced > maxR) forced = maxR;
            if (forced > q.HO) forced = q.HO;
            for (int R = 1; R <= maxR && R <= q.HO; R++) {
                if (forced > 0 && R != forced) continue;
                const int NR = (R - 1) * S + 3;
                const int NT = R * a.SEG * NL;
                int xwords;
                if (resident) {
                    xwords = a.CGP * channel_stride(NR * a.WP);
                } else {
                    // a lane carries kXRegs image words per stage in registers; what a small workgroup cannot
                    // carry that way it copies directly, which is slow: only taken when forced
                    const int kXRegs = x_regs(S);
                    const int stage = kCC * NR * a.WP;
                    if (stage > kXRegs * NT && forced <= 0) continue;
                    const int half = stage > kXRegs * NT ? stage : kXRegs * NT;
                    xwords = 2 * ((half + 3) / 4 * 4);
                }
                const size_t lds = ((size_t)nx * xwords + 2 * (size_t)kKC * kBNP) * sizeof(float);
                if (lds > kLdsLimit - (nx > 1 ? 1024 : 0)) { if (resident) break; else continue; }   // nx > 1: room for the kernel's static LDS
                const long waves_wg = (NT + 63) / 64;
                long wgs = (long)(kLdsLimit / lds);
                if (wgs * waves_wg > 8) wgs = 8 / waves_wg;
                const int tiles_h = (q.HO + R - 1) / R;
                const double score = (double)wgs * NT * q.HO / ((double)tiles_h * R);
                if (score >= bestScore) { bestScore = score; bestR = R; bestWords = xwords; }
            }
            // below six resident waves per CU this variant does badly: try the other, or leave the layer to
            // the column kernels
            if (bestR == 0 || (bestScore < 384.0 && forced <= 0)) continue;
            const int real_tiles = (quads + NL - 1) / NL;
            const double priced = bestScore * (1.0 - 0.03 * (real_tiles - first_tiles));
            if (have && priced <= haveScore) continue;
            have = true;
            haveScore = priced;
            pick = a;
            pick.NL = NL; pick.BN = BN; pick.tiles_n = real_tiles;
            pick.R = bestR; pick.NR = (bestR - 1) * S + 3; pick.ML = bestR * a.SEG;
            pick.tiles_h = (q.HO + bestR - 1) / bestR;
            pick.resident = resident ? 1 : 0;
            pick.xwords = bestWords;
            pick.cstride = channel_stride(pick.NR * a.WP);
        }
        if (have) {
            a = pick;
            return (long long)q.B * G * a.tiles_h * a.tiles_n < (1LL << 31);
        }
    }
    return false;
}

}  // namespace convimg
}  // namespace ldist

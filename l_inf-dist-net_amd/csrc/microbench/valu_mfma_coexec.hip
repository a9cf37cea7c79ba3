// Micro-benchmark behind one design decision of the L_inf forward: can the matrix cores take the subtraction?
// v_mfma_f32_32x32x2_f32 with A = (x, -1) and B = (1, w) yields exact fp32 differences x - w, which would leave
// the vector ALU with half a v_max3_f32 per difference -- if matrix and vector instructions ran side by side.
// This program times long streams of one instruction kind, alone and together, on every SIMD of the device:
// a workgroup is 512 lanes = 8 waves, two per SIMD; waves 0..3 run stream A, waves 4..7 stream B, so each SIMD
// holds one wave of either kind (the program prints the SIMD of every wave from its HW_ID register), plus the
// same pair of streams interleaved inside one wave.  If the streams overlapped, a pair would take about as long
// as its longer member; on gfx950 every pair takes the sum (and the counter SQ_VALU_MFMA_COEXEC_CYCLES stays 0).
// Usage: valu_mfma_coexec [case]   (no argument: all cases; one case number: that case only, for counter runs)
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
#define CK(e) do { hipError_t _e = (e); if (_e != hipSuccess) { printf("HIP error %s line %d\n", hipGetErrorString(_e), __LINE__); exit(1);} } while (0)

enum { NONE = 0, MFMA32 = 1, MAX3 = 2, SUB = 3, MIX = 4, MFMA16 = 5, BOTH_SAME = 6 };

template <int S>
__device__ __forceinline__ float stream(const float* x, int iters) {
    const int l = threadIdx.x & 63;
    float s = 0.f;
    if constexpr (S == MFMA32) {
        float a = x[l & 31], b = x[(l + 3) & 31];
        f16v acc[4];
        for (int q = 0; q < 4; q++) for (int r = 0; r < 16; r++) acc[q][r] = 0.f;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int q = 0; q < 4; q++) acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[q], 0, 0, 0);
        }
        for (int q = 0; q < 4; q++) for (int r = 0; r < 16; r++) s += acc[q][r];
    } else if constexpr (S == MFMA16) {
        float a = x[l & 31], b = x[(l + 3) & 31];
        f4v acc[8];
        for (int q = 0; q < 8; q++) for (int r = 0; r < 4; r++) acc[q][r] = 0.f;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int q = 0; q < 8; q++) acc[q] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[q], 0, 0, 0);
        }
        for (int q = 0; q < 8; q++) for (int r = 0; r < 4; r++) s += acc[q][r];
    } else if constexpr (S == MAX3) {
        float v[16];
        for (int i = 0; i < 16; i++) v[i] = x[(l + i) & 31];
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int i = 0; i < 32; i++)
                v[i % 16] = __builtin_fmaxf(__builtin_fmaxf(v[i % 16], __builtin_fabsf(v[(i + 1) % 16])), __builtin_fabsf(v[(i + 5) % 16]));
        }
        for (int r = 0; r < 16; r++) s += v[r];
    } else if constexpr (S == SUB) {
        float v[16];
        for (int i = 0; i < 16; i++) v[i] = x[(l + i) & 31];
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int i = 0; i < 32; i++) v[i % 16] = v[(i + 3) % 16] - v[(i + 7) % 16];
        }
        for (int r = 0; r < 16; r++) s += v[r];
    } else if constexpr (S == MIX) {   // the L_inf forward's own mix: 2 sub + 1 max3 (the operands move, so nothing hoists)
        float v[16], d[16];
        for (int i = 0; i < 16; i++) { v[i] = x[(l + i) & 31]; d[i] = 0.f; }
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float d0 = v[(i + 3) % 16] - v[(i + 7) % 16];
                const float d1 = v[(i + 4) % 16] - d[(i + 9) % 16];
                d[i] = __builtin_fmaxf(__builtin_fmaxf(d[i], __builtin_fabsf(d0)), __builtin_fabsf(d1));
                v[i] = d0;
            }
        }
        for (int r = 0; r < 16; r++) s += d[r];
    } else if constexpr (S == BOTH_SAME) {   // one wave: MFMA (4 independent accumulators) with max3 work in its shadow
        float a = x[l & 31], b = x[(l + 3) & 31];
        f16v acc[4];
        float v[16];
        for (int q = 0; q < 4; q++) for (int r = 0; r < 16; r++) acc[q][r] = 0.f;
        for (int i = 0; i < 16; i++) v[i] = x[(l + i) & 31];
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[q], 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 8; i++)
                    v[(i + 8 * q) % 16] = __builtin_fmaxf(__builtin_fmaxf(v[(i + 8 * q) % 16], __builtin_fabsf(v[(i + 1) % 16])), __builtin_fabsf(v[(i + 5) % 16]));
            }
        }
        for (int q = 0; q < 4; q++) for (int r = 0; r < 16; r++) s += acc[q][r];
        for (int r = 0; r < 16; r++) s += v[r];
    }
    return s;
}

template <int A, int B>
__global__ void __launch_bounds__(512) k(const float* x, float* out, int itA, int itB, int* simd) {
    const int wave = threadIdx.x >> 6;
    float s = 0.f;
    if (wave < 4) s = stream<A>(x, itA); else s = stream<B>(x, itB);
    out[blockIdx.x * 512 + threadIdx.x] = s;
    if (blockIdx.x == 0 && (threadIdx.x & 63) == 0) simd[wave] = __builtin_amdgcn_s_getreg((4 /*HW_ID*/) | (0 << 6) | (31 << 11));
}

template <int A, int B>
float run(const float* dx, float* dout, int* dsimd, int itA, int itB) {
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    hipLaunchKernelGGL((k<A, B>), dim3(256), dim3(512), 0, 0, dx, dout, 50, 50, dsimd);
    CK(hipDeviceSynchronize());
    float best = 1e30f;
    for (int rep = 0; rep < 3; rep++) {
        CK(hipEventRecord(e0));
        hipLaunchKernelGGL((k<A, B>), dim3(256), dim3(512), 0, 0, dx, dout, itA, itB, dsimd);
        CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        if (ms < best) best = ms;
    }
    return best;
}

int main(int argc, char** argv) {
    float hx[32]; for (int i = 0; i < 32; i++) hx[i] = 0.001f * i;
    float *dx, *dout; int* dsimd;
    CK(hipMalloc(&dx, 128)); CK(hipMalloc(&dout, 256 * 512 * 4)); CK(hipMalloc(&dsimd, 64));
    CK(hipMemcpy(dx, hx, 128, hipMemcpyHostToDevice));
    const int only = argc > 1 ? atoi(argv[1]) : -1;   // run a single pair (for the counter runs)
    // iteration counts chosen so each stream alone takes a similar time:
    // MFMA32: 4 mfma x 64 clk = 256 clk / iter; MAX3: 32 x ~4.6 = 147; SUB: 32 x ~2.6..5 = 83..160; MIX: 48 instr
    const int IM = 20000, IV = 35000, IS = 35000, IX = 25000, IM16 = 20000;
#define R(idx, A, B, ia, ib, name)                                                        \
    if (only < 0 || only == idx) {                                                        \
        float ms = run<A, B>(dx, dout, dsimd, ia, ib);                                    \
        printf("%2d %-34s %8.3f ms\n", idx, name, ms); fflush(stdout);                    \
    }
    R(0, MFMA32, NONE, IM, 0, "mfma32 alone (1 wave/SIMD)")
    R(1, NONE, MAX3, 0, IV, "max3 alone (1 wave/SIMD)")
    R(2, MFMA32, MAX3, IM, IV, "mfma32 | max3 (co-resident)")
    R(3, NONE, SUB, 0, IS, "sub alone")
    R(4, MFMA32, SUB, IM, IS, "mfma32 | sub")
    R(5, NONE, MIX, 0, IX, "mix(2sub+max3) alone")
    R(6, MFMA32, MIX, IM, IX, "mfma32 | mix")
    R(7, MFMA16, NONE, IM16, 0, "mfma16x16x4 alone")
    R(8, MFMA16, MAX3, IM16, IV, "mfma16 | max3")
    R(9, MAX3, MAX3, IV, IV, "max3 | max3")
    R(10, MFMA32, MFMA32, IM, IM, "mfma32 | mfma32")
    R(11, BOTH_SAME, NONE, IM, 0, "same wave: mfma32 + 8 max3 each")
    R(12, BOTH_SAME, BOTH_SAME, IM, IM, "same wave x2 waves/SIMD")
    R(13, MIX, MIX, IX, IX, "mix | mix")
    int hs[8]; CK(hipMemcpy(hs, dsimd, 32, hipMemcpyDeviceToHost));
    printf("HW_ID simd of waves 0..7:");
    for (int i = 0; i < 8; i++) printf(" %d", (hs[i] >> 4) & 3);
    printf("\n");
    return 0;
}

// Overlap of transcendental and plain vector instructions on a gfx950 SIMD, as a function of how many plain
// instructions follow each transcendental one in every wave's stream.
// Stream of a wave: NA groups per half trip; group i = one v_exp_f32 (first half) / v_log_f32 (second half) on a[i],
// then K plain instructions on accumulators nobody touched in the last 16 instructions.
// PLAIN 0: v_fmac_f32 (VOP2, 32-bit encoding); 1: v_fma_f32 (VOP3, 64-bit encoding); 2: v_sub_f32 (VOP2);
// 3: v_bfi_b32 (VOP3); 4: v_mul_f32 with an SGPR operand (VOP2)
#include <hip/hip_runtime.h>
#include <cstdio>
constexpr int NA = 16, NC = 32;
template <int PLAIN>
__device__ __forceinline__ void plain(float& c, float x, float y, float s) {
    if (PLAIN == 0) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(c) : "v"(x), "v"(y));
    if (PLAIN == 1) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(c) : "v"(x), "v"(y));
    if (PLAIN == 2) asm volatile("v_sub_f32 %0, %0, %1" : "+v"(c) : "v"(y));
    if (PLAIN == 3) asm volatile("v_bfi_b32 %0, %1, %0, %2" : "+v"(c) : "v"(x), "v"(y));
    if (PLAIN == 4) asm volatile("v_mul_f32 %0, %1, %0" : "+v"(c) : "s"(s));
}
template <int PLAIN, int K, bool TRANS>
__global__ void __launch_bounds__(1024) probe(float* out, int iters, float a0, float s0) {
    float a[NA], c[NC];
    const float x = 1.0f + a0, y = a0 * 0.5f;
    const float s = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(s0)));
#pragma unroll
    for (int i = 0; i < NA; i++) a[i] = 1.0f + a0 * (threadIdx.x + i);
#pragma unroll
    for (int i = 0; i < NC; i++) c[i] = a0 * i;
#pragma unroll 1
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int i = 0; i < NA; i++) {
                if (TRANS) {
                    if (h == 0) asm volatile("v_exp_f32 %0, %0" : "+v"(a[i]));
                    else asm volatile("v_log_f32 %0, %0" : "+v"(a[i]));
                }
#pragma unroll
                for (int q = 0; q < K; q++) plain<PLAIN>(c[((h * NA + i) * K + q) % NC], x, y, s);
            }
    }
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NA; i++) t += a[i];
#pragma unroll
    for (int i = 0; i < NC; i++) t += c[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = t;
}
template <int PLAIN, int K, bool TRANS>
void run(const char* name) {
    float* out; (void)hipMalloc(&out, 256 * 1024 * 4);
    printf("%-22s K=%2d %s:", name, K, TRANS ? "with trans" : "plain only");
    for (int nthr : {256, 512, 768, 1024}) {
        int iters = 2000; dim3 grid(256), block(nthr);
        hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
        hipLaunchKernelGGL((probe<PLAIN, K, TRANS>), grid, block, 0, 0, out, 10, 1e-3f, 1.0f);
        (void)hipEventRecord(e0); hipLaunchKernelGGL((probe<PLAIN, K, TRANS>), grid, block, 0, 0, out, iters, 1e-3f, 1.0f); (void)hipEventRecord(e1);
        (void)hipEventSynchronize(e1);
        float ms; (void)hipEventElapsedTime(&ms, e0, e1);
        // cycles per group (one trans + K plain) per SIMD, all waves of the SIMD together, at 2.4 GHz
        const int waves = nthr / 256;
        const double cyc = ms * 1e-3 * 2.4e9 / ((double)iters * 2 * NA * waves);
        printf("  %dw %6.2f", waves, cyc);
    }
    printf("   (cycles per group and wave, 2.4 GHz)\n");
    (void)hipFree(out);
}
int main() {
    run<0, 0, true>("trans alone");
    run<0, 4, false>("v_fmac VOP2"); run<1, 4, false>("v_fma VOP3"); run<2, 4, false>("v_sub VOP2"); run<3, 4, false>("v_bfi VOP3");
    run<4, 4, false>("v_mul sgpr");
    run<0, 2, true>("v_fmac VOP2"); run<0, 4, true>("v_fmac VOP2"); run<0, 5, true>("v_fmac VOP2"); run<0, 6, true>("v_fmac VOP2");
    run<0, 8, true>("v_fmac VOP2"); run<0, 12, true>("v_fmac VOP2");
    run<1, 2, true>("v_fma VOP3"); run<1, 3, true>("v_fma VOP3"); run<1, 4, true>("v_fma VOP3"); run<1, 6, true>("v_fma VOP3");
    return 0;
}

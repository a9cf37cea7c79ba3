// Does grouping help?  Stream of a wave: G transcendental instructions in a row, then G*K plain VOP2 instructions
// in a row (v_fmac_f32 on registers not touched for at least 16 instructions).  ABS: the log takes |x| (VOP3 encoding).
#include <hip/hip_runtime.h>
#include <cstdio>
constexpr int NA = 16, NC = 48;
template <int K, int G, bool ABS>
__global__ void __launch_bounds__(1024) probe(float* out, int iters, float a0) {
    float a[NA], c[NC];
    const float x = 1.0f + a0, y = a0 * 0.5f;
#pragma unroll
    for (int i = 0; i < NA; i++) a[i] = 1.0f + a0 * (threadIdx.x + i);
#pragma unroll
    for (int i = 0; i < NC; i++) c[i] = a0 * i;
#pragma unroll 1
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int i0 = 0; i0 < NA; i0 += G) {
#pragma unroll
                for (int i = i0; i < i0 + G; i++) {
                    if (h == 0) asm volatile("v_exp_f32 %0, %0" : "+v"(a[i]));
                    else if (ABS) asm volatile("v_log_f32_e64 %0, |%0|" : "+v"(a[i]));
                    else asm volatile("v_log_f32 %0, %0" : "+v"(a[i]));
                }
#pragma unroll
                for (int q = 0; q < K * G; q++)
                    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(c[((h * NA + i0) * K + q) % NC]) : "v"(x), "v"(y));
            }
    }
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NA; i++) t += a[i];
#pragma unroll
    for (int i = 0; i < NC; i++) t += c[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = t;
}
template <int K, int G, bool ABS>
void run() {
    float* out; (void)hipMalloc(&out, 256 * 1024 * 4);
    printf("K=%d plain per trans, groups of %2d trans%s:", K, G, ABS ? ", log |x|" : "");
    for (int nthr : {256, 512, 1024}) {
        int iters = 2000; dim3 grid(256), block(nthr);
        hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
        hipLaunchKernelGGL((probe<K, G, ABS>), grid, block, 0, 0, out, 10, 1e-3f);
        (void)hipEventRecord(e0); hipLaunchKernelGGL((probe<K, G, ABS>), grid, block, 0, 0, out, iters, 1e-3f); (void)hipEventRecord(e1);
        (void)hipEventSynchronize(e1);
        float ms; (void)hipEventElapsedTime(&ms, e0, e1);
        const int waves = nthr / 256;
        printf("  %dw %6.2f", waves, ms * 1e-3 * 2.4e9 / ((double)iters * 2 * NA * waves));
    }
    printf("   cycles per (trans + K plain) and wave\n");
    (void)hipFree(out);
}
int main() {
    run<3, 1, false>(); run<3, 2, false>(); run<3, 4, false>(); run<3, 8, false>(); run<3, 16, false>();
    run<3, 1, true>(); run<3, 8, true>();
    run<6, 1, false>(); run<6, 4, false>(); run<6, 8, false>();
    return 0;
}

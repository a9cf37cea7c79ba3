// How many lanes per clock a CU retires for LDS atomics of different types (and plain reads and writes for scale).
// 256 workgroups of 512 lanes; every lane makes 2000 operations on pseudo-random words among 5120 (the bins of one
// row of a 5120-wide layer).  The scatter kernels of inf_backward.hip keep their bins in the type this program shows
// to be fast.  Prints one line per operation; the sum check shows that no addition was lost.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(e) do { hipError_t e_ = (e); if (e_ != hipSuccess) { printf("HIP error %s, line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

constexpr int kWords = 5120, kLanes = 512, kGroups = 256, kIters = 2000;

template <int MODE>
__global__ void __launch_bounds__(kLanes) probe(float* out, int iters) {
    __shared__ float bins[kWords];
    __shared__ double dbins[kWords];
    unsigned* ubins = reinterpret_cast<unsigned*>(bins);
    for (int i = threadIdx.x; i < kWords; i += kLanes) { bins[i] = 0.f; dbins[i] = 0.0; }
    __syncthreads();
    unsigned s = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
    unsigned seen = 0;
    for (int it = 0; it < iters; it++) {
        s = s * 1664525u + 1013904223u;
        const unsigned a = (s >> 8) % kWords;
        if (MODE == 0) atomicAdd(&bins[a], 1.0f);          // ds_add_f32
        if (MODE == 1) atomicAdd(&dbins[a], 1.0);          // ds_add_f64
        if (MODE == 2) atomicAdd(&ubins[a], 1u);           // ds_add_u32
        if (MODE == 3) seen += atomicAdd(&ubins[a], 1u);   // ds_add_rtn_u32
        if (MODE == 4) bins[a] = 1.0f;                     // ds_write_b32
        if (MODE == 5) seen += ubins[a];                   // ds_read_b32
    }
    __syncthreads();
    float total = 0.f;
    for (int i = threadIdx.x; i < kWords; i += kLanes)
        total += (MODE == 2 || MODE == 3) ? (float)ubins[i] : bins[i] + (float)dbins[i];
    out[blockIdx.x * kLanes + threadIdx.x] = total + (float)(seen & 1u) * 1e-30f;
}

template <int MODE>
void run(const char* name, bool sums) {
    float* out;
    CK(hipMalloc(&out, kGroups * kLanes * sizeof(float)));
    hipEvent_t a, b;
    CK(hipEventCreate(&a));
    CK(hipEventCreate(&b));
    hipLaunchKernelGGL(probe<MODE>, dim3(kGroups), dim3(kLanes), 0, 0, out, 10);
    CK(hipEventRecord(a));
    hipLaunchKernelGGL(probe<MODE>, dim3(kGroups), dim3(kLanes), 0, 0, out, kIters);
    CK(hipEventRecord(b));
    CK(hipEventSynchronize(b));
    float ms;
    CK(hipEventElapsedTime(&ms, a, b));
    static float host[kLanes];
    CK(hipMemcpy(host, out, sizeof(host), hipMemcpyDeviceToHost));
    double sum = 0;
    for (int i = 0; i < kLanes; i++) sum += host[i];
    printf("%-16s %7.3f ms  %5.2f lanes per clock and CU at 2.4 GHz", name, ms, (double)kLanes * kIters / (ms * 1e-3 * 2.4e9));
    if (sums) printf("  (workgroup 0 holds %.0f of %d additions)", sum, kLanes * kIters);
    printf("\n");
    CK(hipFree(out));
}

int main() {
    run<0>("ds_add_f32", true);
    run<1>("ds_add_f64", true);
    run<2>("ds_add_u32", true);
    run<3>("ds_add_rtn_u32", true);
    run<4>("ds_write_b32", false);
    run<5>("ds_read_b32", false);
    return 0;
}

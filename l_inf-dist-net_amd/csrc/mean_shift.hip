// Per-channel mean shift of a (B, C, L) tensor: y[b,c,l] = x[b,c,l] - mean_c, mean_c the mean of
// x over b and l, in one kernel; optionally moves a running mean.  This is the training-mode
// arithmetic of the reference's MeanNorm (model/norm_dist.py:85-96), which runs it as five
// small torch kernels per layer and direction; the same kernel serves the backward pass
// (gx = gy - mean(gy)).  HBM-bound: a workgroup owns a slab small enough that its second read
// comes from cache, so the tensor is fetched once and written once.
#include "kernels.hpp"
#include "wave_reduce.hpp"

namespace ldist {

constexpr int kMsCols = 32;      // channels per workgroup, L == 1
constexpr int kMsThreads = 256;
constexpr int kMsChanThreads = 1024;   // the channel kernel: one workgroup per channel

__device__ __forceinline__ void move_running_mean(float* running_mean, int c, float mean, float momentum) {
    // (1 - momentum) * running + momentum * mean, rounded after each step as two torch ops would
    const float kept = running_mean[c] * (1.0f - momentum);
    running_mean[c] = kept + momentum * mean;
}

// L == 1: channels are contiguous.  Workgroup = kMsCols channels x all B rows.  A lane owns four
// neighbouring channels (one 128-bit access per row) and the rows ty, ty + 32, ...; eight lanes
// cover a 128-byte row segment.  Sixteen rows per lane are loaded before the first is used, which
// keeps 64 KB in flight per workgroup; up to 512 rows stay in registers for the subtraction, so
// the tensor is read exactly once.  VEC4 needs C % 4 == 0 and 16-byte aligned bases.
template <bool VEC4>
__global__ void __launch_bounds__(kMsThreads)
mean_shift_rows_kernel(const float* __restrict__ x, float* __restrict__ y, float* __restrict__ mean_out,
                       float* __restrict__ running_mean, float momentum, int B, int C) {
    constexpr int TX = kMsCols / 4, RY = kMsThreads / TX, HOLD = 16;   // 8 lanes across, 32 down
    __shared__ float part[RY][kMsCols];
    __shared__ float mean_s[kMsCols];
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int c = blockIdx.x * kMsCols + tx * 4;
    auto load4 = [&](int r) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (r < B) {
            const float* p = x + (size_t)r * C + c;
            if constexpr (VEC4) {
                if (c < C) v = *reinterpret_cast<const float4*>(p);
            } else {
                if (c < C) v.x = p[0];
                if (c + 1 < C) v.y = p[1];
                if (c + 2 < C) v.z = p[2];
                if (c + 3 < C) v.w = p[3];
            }
        }
        return v;
    };
    auto store4 = [&](int r, float4 v) {
        if (r >= B) return;
        float* p = y + (size_t)r * C + c;
        if constexpr (VEC4) {
            if (c < C) *reinterpret_cast<float4*>(p) = v;
        } else {
            if (c < C) p[0] = v.x;
            if (c + 1 < C) p[1] = v.y;
            if (c + 2 < C) p[2] = v.z;
            if (c + 3 < C) p[3] = v.w;
        }
    };
    float4 held[HOLD];
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int r0 = 0; r0 < B; r0 += HOLD * RY) {
#pragma unroll
        for (int i = 0; i < HOLD; i++) held[i] = load4(r0 + ty + i * RY);
#pragma unroll
        for (int i = 0; i < HOLD; i++) { s.x += held[i].x; s.y += held[i].y; s.z += held[i].z; s.w += held[i].w; }
    }
    part[ty][tx * 4 + 0] = s.x; part[ty][tx * 4 + 1] = s.y; part[ty][tx * 4 + 2] = s.z; part[ty][tx * 4 + 3] = s.w;
    __syncthreads();
    if (threadIdx.x < kMsCols) {
        float t = 0.f;
#pragma unroll
        for (int q = 0; q < RY; q++) t += part[q][threadIdx.x];
        const float mean = t / (float)B;
        mean_s[threadIdx.x] = mean;
        const int cc = blockIdx.x * kMsCols + threadIdx.x;
        if (cc < C) {
            if (mean_out) mean_out[cc] = mean;
            if (running_mean) move_running_mean(running_mean, cc, mean, momentum);
        }
    }
    __syncthreads();
    const float4 m = make_float4(mean_s[tx * 4], mean_s[tx * 4 + 1], mean_s[tx * 4 + 2], mean_s[tx * 4 + 3]);
    auto shifted = [&](float4 v) { return make_float4(v.x - m.x, v.y - m.y, v.z - m.z, v.w - m.w); };
    if (B <= HOLD * RY) {   // everything is still in registers
#pragma unroll
        for (int i = 0; i < HOLD; i++) store4(ty + i * RY, shifted(held[i]));
    } else {
        for (int r0 = 0; r0 < B; r0 += HOLD * RY) {
#pragma unroll
            for (int i = 0; i < HOLD; i++) held[i] = load4(r0 + ty + i * RY);
#pragma unroll
            for (int i = 0; i < HOLD; i++) store4(r0 + ty + i * RY, shifted(held[i]));
        }
    }
}

// L > 1: for a fixed (b, c) the L values are contiguous.  Workgroup = one channel; lanes run along l
// (128-bit accesses when VEC == 4: L % 4 == 0 and 16-byte aligned bases).  A channel is one workgroup's work and
// there are often fewer channels than CUs, so the workgroup is as large as it can be: what limits this kernel is
// how many loads one CU keeps in flight.
template <int VEC>
__global__ void __launch_bounds__(kMsChanThreads)
mean_shift_channel_kernel(const float* __restrict__ x, float* __restrict__ y, float* __restrict__ mean_out,
                          float* __restrict__ running_mean, float momentum, int B, int C, int L) {
    __shared__ float part[kMsChanThreads / 64];
    __shared__ float mean_s;
    const int c = blockIdx.x;
    const int per_b = L / VEC;                    // vectors per (b, c) run
    const int total = B * per_b;
    // four independent loads in flight per lane: a channel is one workgroup's work, and with one load per trip
    // the workgroup waits out a memory latency per 4 KB (8 KB with 128-bit loads)
    constexpr int UN = 4;
    auto at_of = [&](int i) {
        const int b = i / per_b, q = i - b * per_b;
        return ((size_t)b * C + c) * L + (size_t)q * VEC;
    };
    float s = 0.f;
    for (int i0 = threadIdx.x; i0 < total; i0 += UN * kMsChanThreads) {
        if constexpr (VEC == 4) {
            float4 v[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const int i = i0 + u * kMsChanThreads;
                v[u] = i < total ? *reinterpret_cast<const float4*>(x + at_of(i)) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int u = 0; u < UN; u++) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
        } else {
            float v[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const int i = i0 + u * kMsChanThreads;
                v[u] = i < total ? x[at_of(i)] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < UN; u++) s += v[u];
        }
    }
    s = wave_sum(s);                // lane 63 holds the wave's sum
    if ((threadIdx.x & 63) == 63) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
#pragma unroll
        for (int q = 0; q < kMsChanThreads / 64; q++) t += part[q];
        const float mean = t / ((float)B * (float)L);
        mean_s = mean;
        if (mean_out) mean_out[c] = mean;
        if (running_mean) move_running_mean(running_mean, c, mean, momentum);
    }
    __syncthreads();
    const float mean = mean_s;
    for (int i0 = threadIdx.x; i0 < total; i0 += UN * kMsChanThreads) {
        size_t at[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) at[u] = at_of(min(i0 + u * kMsChanThreads, total - 1));
        if constexpr (VEC == 4) {
            float4 v[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) v[u] = *reinterpret_cast<const float4*>(x + at[u]);
#pragma unroll
            for (int u = 0; u < UN; u++)
                if (i0 + u * kMsChanThreads < total)
                    *reinterpret_cast<float4*>(y + at[u]) = make_float4(v[u].x - mean, v[u].y - mean, v[u].z - mean, v[u].w - mean);
        } else {
            float v[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) v[u] = x[at[u]];
#pragma unroll
            for (int u = 0; u < UN; u++)
                if (i0 + u * kMsChanThreads < total) y[at[u]] = v[u] - mean;
        }
    }
}

hipError_t mean_shift(const float* x, float* y, float* mean_out, float* running_mean, float momentum, int B, int C,
                      int L, hipStream_t stream) {
    if (L == 1) {
        const unsigned grid = (unsigned)((C + kMsCols - 1) / kMsCols);
        if (C % 4 == 0 && aligned16(x) && aligned16(y))
            hipLaunchKernelGGL(mean_shift_rows_kernel<true>, dim3(grid), dim3(kMsThreads), 0, stream, x, y, mean_out,
                               running_mean, momentum, B, C);
        else
            hipLaunchKernelGGL(mean_shift_rows_kernel<false>, dim3(grid), dim3(kMsThreads), 0, stream, x, y,
                               mean_out, running_mean, momentum, B, C);
    } else if (L % 4 == 0 && aligned16(x) && aligned16(y)) {
        hipLaunchKernelGGL(mean_shift_channel_kernel<4>, dim3((unsigned)C), dim3(kMsChanThreads), 0, stream, x, y,
                           mean_out, running_mean, momentum, B, C, L);
    } else {
        hipLaunchKernelGGL(mean_shift_channel_kernel<1>, dim3((unsigned)C), dim3(kMsChanThreads), 0, stream, x, y,
                           mean_out, running_mean, momentum, B, C, L);
    }
    return hipGetLastError();
}

}  // namespace ldist

// Micro-benchmarks that measure what this GPU gives: streaming reads and copies from HBM, and the
// matrix cores' rate on a loop of independent MFMA instructions. The benchmark prints a step's
// achieved bandwidth and flops against these beside the published peaks.
//
// The reference measures its own device the same way: a streaming-copy kernel
// (/root/reference/benchmarks/roofline/memory_peak.cu) and an FMA loop
// (/root/reference/benchmarks/roofline/fp32_peak.cu), whose results feed its roofline plot
// (/root/reference/benchmarks/roofline/plot_roofline_only.py:9-10).
#include "common.h"

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Every thread reads 16 bytes per iteration, consecutive threads consecutive addresses; the
// grid strides over the buffer. The xor of everything read is stored only if it has an unlikely
// value, so that the loads cannot be dropped.
__global__ void __launch_bounds__(256)
stream_read_kernel(const u32x4* __restrict__ src, size_t n_vec, unsigned* __restrict__ sink) {
    u32x4 acc = {0u, 0u, 0u, 0u};
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    for (; i + 3 * stride < n_vec; i += 4 * stride) {
        const u32x4 a = __builtin_nontemporal_load(src + i);
        const u32x4 b = __builtin_nontemporal_load(src + i + stride);
        const u32x4 c = __builtin_nontemporal_load(src + i + 2 * stride);
        const u32x4 d = __builtin_nontemporal_load(src + i + 3 * stride);
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < n_vec; i += stride) acc ^= __builtin_nontemporal_load(src + i);
    const unsigned x = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (x == 0x9E3779B9u) sink[0] = x;
}

__global__ void __launch_bounds__(256)
stream_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t n_vec) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    for (; i + stride < n_vec; i += 2 * stride) {
        const u32x4 a = __builtin_nontemporal_load(src + i);
        const u32x4 b = __builtin_nontemporal_load(src + i + stride);
        __builtin_nontemporal_store(a, dst + i);
        __builtin_nontemporal_store(b, dst + i + stride);
    }
    for (; i < n_vec; i += stride) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Four independent accumulators per wavefront, operands that never change: nothing but the matrix
// cores' issue rate limits the loop. 32x32x16 bf16: 2*32*32*16 flops per instruction.
__global__ void __launch_bounds__(256)
mfma_bf16_loop_kernel(int iters, float* __restrict__ sink) {
    bf16x8 a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = static_cast<__bf16>(0.001f * static_cast<float>((threadIdx.x + e) % 7));
        b[e] = static_cast<__bf16>(0.002f * static_cast<float>((threadIdx.x + 3 * e) % 5));
    }
    f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
    for (int i = 0; i < iters; ++i) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
    }
    const f32x16 s = c0 + c1 + c2 + c3;
    float t = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) t += s[e];
    if (t == 12345.678f) sink[0] = t;
}

// The same with true 32-bit operands: 32x32x2 f32, 2*32*32*2 flops per instruction.
__global__ void __launch_bounds__(256)
mfma_f32_loop_kernel(int iters, float* __restrict__ sink) {
    const float a = 0.001f * static_cast<float>(threadIdx.x % 7), b = 0.002f * static_cast<float>(threadIdx.x % 5);
    f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
    for (int i = 0; i < iters; ++i) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c3, 0, 0, 0);
    }
    const f32x16 s = c0 + c1 + c2 + c3;
    float t = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) t += s[e];
    if (t == 12345.678f) sink[0] = t;
}

// Plain vector FMAs, eight independent chains per lane: what a kernel without matrix instructions
// (the 32-bit products of this engine) can reach.
__global__ void __launch_bounds__(256)
fma_f32_loop_kernel(int iters, float* __restrict__ sink) {
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.001f * static_cast<float>(threadIdx.x + e);
    const float m = 1.0000001f, c = 1e-9f;
    for (int i = 0; i < iters; ++i) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = fmaf(v[e], m, c);
    }
    float t = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) t += v[e];
    if (t == 12345.678f) sink[0] = t;
}

extern "C" {

// Each launcher queues `reps` launches on the stream; the caller times them with events.
// Bytes moved per launch: n_bytes (read) or 2 * n_bytes (copy). n_bytes must be a multiple of 16.
int mllm_peak_stream_read(const void* src, size_t n_bytes, void* sink, int workgroups, int reps, hipStream_t stream) {
    if (n_bytes % 16 != 0 || workgroups < 1 || reps < 1) return -1;
    for (int r = 0; r < reps; ++r)
        stream_read_kernel<<<workgroups, 256, 0, stream>>>(static_cast<const u32x4*>(src), n_bytes / 16,
                                                           static_cast<unsigned*>(sink));
    MLLM_LAUNCH_CHECK();
    return 0;
}

int mllm_peak_stream_copy(const void* src, void* dst, size_t n_bytes, int workgroups, int reps, hipStream_t stream) {
    if (n_bytes % 16 != 0 || workgroups < 1 || reps < 1) return -1;
    for (int r = 0; r < reps; ++r)
        stream_copy_kernel<<<workgroups, 256, 0, stream>>>(static_cast<const u32x4*>(src), static_cast<u32x4*>(dst),
                                                           n_bytes / 16);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// kind 0: bf16 MFMA 32x32x16; 1: f32 MFMA 32x32x2; 2: f32 vector FMA. Returns the flops of ONE launch
// through *flops (workgroups of 4 wavefronts, `iters` loop iterations).
int mllm_peak_math_loop(int kind, int workgroups, int iters, void* sink, int reps, double* flops,
                        hipStream_t stream) {
    if (workgroups < 1 || iters < 1 || reps < 1) return -1;
    const double waves = 4.0 * workgroups;
    for (int r = 0; r < reps; ++r) {
        if (kind == 0) mfma_bf16_loop_kernel<<<workgroups, 256, 0, stream>>>(iters, static_cast<float*>(sink));
        else if (kind == 1) mfma_f32_loop_kernel<<<workgroups, 256, 0, stream>>>(iters, static_cast<float*>(sink));
        else if (kind == 2) fma_f32_loop_kernel<<<workgroups, 256, 0, stream>>>(iters, static_cast<float*>(sink));
        else return -1;
    }
    if (kind == 0) *flops = waves * iters * 4.0 * 2.0 * 32 * 32 * 16;
    else if (kind == 1) *flops = waves * iters * 4.0 * 2.0 * 32 * 32 * 2;
    else *flops = waves * 64.0 * iters * 8.0 * 2.0;
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

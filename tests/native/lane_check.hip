// A test-only kernel: what the lane exchanges of the kernels' common.h give, for a test of them
// (tests/test_kernels_gpu.py). Not part of the engine.
#include "common.h"

// out[lane] = maximum, out[64 + lane] = sum over lanes l, l ^ 16, l ^ 32, l ^ 48 of in[lane] (one wavefront),
// then in[lane ^ 8], in[lane ^ 16], in[lane ^ 32], in[lane ^ 4]: what rows_max, rows_sum and lane_xor give.
// out: 384 floats.
__global__ void rows_check_kernel(const float* __restrict__ in, float* __restrict__ out) {
    const float v = in[threadIdx.x];
    out[threadIdx.x] = rows_max(v);
    out[64 + threadIdx.x] = rows_sum(v);
    out[128 + threadIdx.x] = lane_xor(v, 8);
    out[192 + threadIdx.x] = lane_xor(v, 16);
    out[256 + threadIdx.x] = lane_xor(v, 32);
    out[320 + threadIdx.x] = lane_xor(v, 4);
}

extern "C" int mllm_rows_check(const float* in, float* out, hipStream_t stream) {
    rows_check_kernel<<<1, 64, 0, stream>>>(in, out);
    MLLM_LAUNCH_CHECK();
    return 0;
}

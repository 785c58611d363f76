// Token choice on the device: greedy argmax and temperature sampling, fp32 logits.
#include "common.h"

#define SAMPLE_THREADS 256

// ---------------------------------------------------------------------------
// Row argmax, ties to the lowest index: /root/reference/src/kernels/argmax.cu:12-20,22-75.
// ---------------------------------------------------------------------------
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
    return (v > bv) || (v == bv && i < bi);
}

#define ARGMAX_CHUNK 2048      // elements per workgroup in the first stage (8 per thread)

// Stage 1: the best (value, index) of one chunk of one row. Stage 2 (n_chunks == 1 input
// chunks of pairs) reduces the chunks' results. Both keep the lowest index on ties.
__global__ void argmax_stage1(const float* __restrict__ logits, int ld, int V, int n_chunks,
                              float* __restrict__ part_val, int* __restrict__ part_idx, int* __restrict__ out) {
    __shared__ float sv[SAMPLE_THREADS / MLLM_WAVE];
    __shared__ int si[SAMPLE_THREADS / MLLM_WAVE];
    const int row_id = blockIdx.y, chunk = blockIdx.x;
    const float* row = logits + static_cast<size_t>(row_id) * ld;
    const int base = chunk * ARGMAX_CHUNK;
    float v[ARGMAX_CHUNK / SAMPLE_THREADS];
#pragma unroll
    for (int u = 0; u < ARGMAX_CHUNK / SAMPLE_THREADS; ++u) {
        const int i = base + u * SAMPLE_THREADS + threadIdx.x;
        v[u] = i < V ? row[i] : -INFINITY;
    }
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int u = 0; u < ARGMAX_CHUNK / SAMPLE_THREADS; ++u) {
        const int i = base + u * SAMPLE_THREADS + threadIdx.x;
        if (i < V && better(v[u], i, bv, bi)) { bv = v[u]; bi = i; }
    }
#pragma unroll
    for (int off = MLLM_WAVE / 2; off > 0; off >>= 1) {
        float ov = __shfl_xor(bv, off, MLLM_WAVE);
        int oi = __shfl_xor(bi, off, MLLM_WAVE);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    const int wave = threadIdx.x / MLLM_WAVE, lane = threadIdx.x % MLLM_WAVE;
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < SAMPLE_THREADS / MLLM_WAVE; ++w)
            if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        if (n_chunks == 1) {
            out[row_id] = (bi == 0x7fffffff) ? 0 : bi;       // a row of NaNs yields 0
        } else {
            part_val[static_cast<size_t>(row_id) * n_chunks + chunk] = bv;
            part_idx[static_cast<size_t>(row_id) * n_chunks + chunk] = bi;
        }
    }
}

__global__ void argmax_stage2(const float* __restrict__ part_val, const int* __restrict__ part_idx,
                              int n_chunks, int* __restrict__ out) {
    const int row_id = blockIdx.x, lane = threadIdx.x;      // one wavefront per row
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int c = lane; c < n_chunks; c += MLLM_WAVE) {
        const float v = part_val[static_cast<size_t>(row_id) * n_chunks + c];
        const int i = part_idx[static_cast<size_t>(row_id) * n_chunks + c];
        if (better(v, i, bv, bi)) { bv = v; bi = i; }
    }
#pragma unroll
    for (int off = MLLM_WAVE / 2; off > 0; off >>= 1) {
        float ov = __shfl_xor(bv, off, MLLM_WAVE);
        int oi = __shfl_xor(bi, off, MLLM_WAVE);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if (lane == 0) out[row_id] = (bi == 0x7fffffff) ? 0 : bi;
}

// ---------------------------------------------------------------------------
// Temperature sampling: p = softmax(logits / temperature) in fp32, then the
// inverse CDF at u in [0,1): the first index whose cumulative mass exceeds u * total.
// Rows with temperature <= 0 take the argmax. One block per row; every thread owns a
// contiguous chunk of the vocabulary so that the cumulative order is the index order.
// ---------------------------------------------------------------------------
__global__ void sample_kernel(const float* __restrict__ logits, int ld, int V,
                              const float* __restrict__ temperature, const float* __restrict__ u,
                              int* __restrict__ out) {
    __shared__ float scratch[16];
    __shared__ float part[SAMPLE_THREADS];
    __shared__ int chosen_thread;
    __shared__ float chosen_before;
    const int r = blockIdx.x;
    const float* row = logits + static_cast<size_t>(r) * ld;
    const float temp = temperature[r];
    const int chunk = (V + blockDim.x - 1) / blockDim.x;
    const int lo = min(V, static_cast<int>(threadIdx.x) * chunk), hi = min(V, lo + chunk);

    float m = -INFINITY;
    int mi = 0x7fffffff;
    for (int i = lo; i < hi; ++i) {
        float v = row[i];
        if (better(v, i, m, mi)) { m = v; mi = i; }
    }
    if (temp <= 0.f) {
        // greedy: reduce (value, index) pairs
        __shared__ float gv[SAMPLE_THREADS];
        __shared__ int gi[SAMPLE_THREADS];
        gv[threadIdx.x] = m;
        gi[threadIdx.x] = mi;
        __syncthreads();
        if (threadIdx.x == 0) {
            float bv = gv[0];
            int bi = gi[0];
            for (int t = 1; t < blockDim.x; ++t)
                if (better(gv[t], gi[t], bv, bi)) { bv = gv[t]; bi = gi[t]; }
            out[r] = (bi == 0x7fffffff) ? 0 : bi;
        }
        return;
    }
    const float row_max = block_max(m, scratch);
    const float inv_t = 1.0f / temp;
    float s = 0.f;
    for (int i = lo; i < hi; ++i) s += expf((row[i] - row_max) * inv_t);
    part[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int t = 0; t < blockDim.x; ++t) total += part[t];
        const float target = u[r] * total;
        float before = 0.f;
        int pick = -1;
        float pick_before = 0.f;
        int last_nonempty = 0;
        float last_before = 0.f;
        for (int t = 0; t < blockDim.x; ++t) {
            if (part[t] > 0.f) { last_nonempty = t; last_before = before; }
            if (pick < 0 && target < before + part[t]) { pick = t; pick_before = before; }
            before += part[t];
        }
        if (pick < 0) { pick = last_nonempty; pick_before = last_before; }   // rounding at the top end
        chosen_thread = pick;
        chosen_before = pick_before;
        part[0] = target;   // thread 0's own sum is no longer needed
    }
    __syncthreads();
    if (static_cast<int>(threadIdx.x) == chosen_thread) {
        const float target = part[0];
        float c = chosen_before;
        int pick = -1, last = lo;
        for (int i = lo; i < hi; ++i) {
            float p = expf((row[i] - row_max) * inv_t);
            if (p > 0.f) last = i;
            c += p;
            if (target < c) { pick = i; break; }
        }
        out[r] = pick >= 0 ? pick : last;
    }
}

extern "C" {

// Chunks of the first stage for a row of V values: the scratch holds n * chunks floats and ints.
int mllm_argmax_chunks(int V) { return (V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK; }

int mllm_argmax(const float* logits, int ld, int n, int V, int* out, float* part_val, int* part_idx,
                hipStream_t stream) {
    if (n <= 0) return 0;
    if (V <= 0) return -1;
    const int n_chunks = (V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
    argmax_stage1<<<dim3(n_chunks, n), SAMPLE_THREADS, 0, stream>>>(logits, ld, V, n_chunks, part_val, part_idx, out);
    MLLM_LAUNCH_CHECK();
    if (n_chunks > 1) {
        argmax_stage2<<<n, MLLM_WAVE, 0, stream>>>(part_val, part_idx, n_chunks, out);
        MLLM_LAUNCH_CHECK();
    }
    return 0;
}

int mllm_sample(const float* logits, int ld, int n, int V, const float* temperature, const float* u, int* out,
                hipStream_t stream) {
    if (n <= 0) return 0;
    sample_kernel<<<n, SAMPLE_THREADS, 0, stream>>>(logits, ld, V, temperature, u, out);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

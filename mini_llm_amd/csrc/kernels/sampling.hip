// Token choice on the device: greedy argmax and temperature sampling, fp32 logits.
#include <mutex>

#include "common.h"
#include "noalloc.h"

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
// `mirror` (in all kernels here; may be null): a second place for the tokens, which may be pinned host memory:
// the kernel that chooses a token hands it to the host itself, where a copy would be one more launch.
__global__ void argmax_stage1(const float* __restrict__ logits, int ld, int V, int n_chunks,
                              float* __restrict__ part_val, int* __restrict__ part_idx, int* __restrict__ out,
                              int* __restrict__ mirror) {
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
            const int tok = (bi == 0x7fffffff) ? 0 : bi;     // a row of NaNs yields 0
            out[row_id] = tok;
            if (mirror != nullptr) mirror[row_id] = tok;
        } else {
            part_val[static_cast<size_t>(row_id) * n_chunks + chunk] = bv;
            part_idx[static_cast<size_t>(row_id) * n_chunks + chunk] = bi;
        }
    }
}

__global__ void argmax_stage2(const float* __restrict__ part_val, const int* __restrict__ part_idx,
                              int n_chunks, int* __restrict__ out, int* __restrict__ mirror) {
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
    if (lane == 0) {
        const int tok = (bi == 0x7fffffff) ? 0 : bi;
        out[row_id] = tok;
        if (mirror != nullptr) mirror[row_id] = tok;
    }
}

// ---------------------------------------------------------------------------
// Temperature sampling: p = softmax(logits / temperature) in fp32, then the inverse CDF at
// u in [0,1): the first index whose cumulative mass exceeds u * total. Rows with
// temperature <= 0 take the argmax (lowest index on ties). One workgroup per row:
//   1. row maximum (and its lowest index), coalesced strided loads;
//   2. the mass of every tile of SAMPLE_TILE consecutive entries, one wavefront per tile;
//   3. a scan over the few tile masses finds the tile that holds u * total;
//   4. inside that tile every thread owns 8 consecutive entries; a workgroup scan finds the thread
//      and it walks its 8 entries.
// The cumulative order is the index order and every sum has a fixed order, so a draw depends on
// (logits, temperature, u) only.
// ---------------------------------------------------------------------------
#define SAMPLE_TILE 2048
#define SAMPLE_MAX_TILES 1024      // vocabularies up to 2M entries
#define SAMPLE_BLOCK 1024          // threads of the sampling workgroup

__global__ void __launch_bounds__(SAMPLE_BLOCK)
sample_kernel(const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
              const float* __restrict__ u, int* __restrict__ out, int* __restrict__ mirror) {
    __shared__ float sv[SAMPLE_BLOCK / MLLM_WAVE];
    __shared__ int si[SAMPLE_BLOCK / MLLM_WAVE];
    __shared__ float tile_mass[SAMPLE_MAX_TILES];
    __shared__ float wave_mass[SAMPLE_TILE / 8 / MLLM_WAVE];
    __shared__ int sh_tile;
    __shared__ float sh_rest;
    const int r = blockIdx.x, tid = threadIdx.x, wave = tid / MLLM_WAVE, lane = tid % MLLM_WAVE;
    const float* row = logits + static_cast<size_t>(r) * ld;
    const float temp = temperature[r];

    // 1. maximum and its lowest index
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i0 = 0; i0 < V; i0 += SAMPLE_BLOCK * 8) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int i = i0 + k * SAMPLE_BLOCK + tid;
            v[k] = row[min(i, V - 1)];           // unconditional (clamped) loads stay in flight together
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int i = i0 + k * SAMPLE_BLOCK + tid;
            if (i < V && better(v[k], i, bv, bi)) { bv = v[k]; bi = i; }
        }
    }
#pragma unroll
    for (int off = MLLM_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, MLLM_WAVE);
        const int oi = __shfl_xor(bi, off, MLLM_WAVE);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    bv = sv[0]; bi = si[0];
    for (int w = 1; w < SAMPLE_BLOCK / MLLM_WAVE; ++w)
        if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
    if (temp <= 0.f) {                       // greedy row (uniform over the workgroup)
        if (tid == 0) {
            const int tok = (bi == 0x7fffffff) ? 0 : bi;
            out[r] = tok;
            if (mirror != nullptr) mirror[r] = tok;
        }
        return;
    }
    // e^((x - max)/T) as 2^((x - max) * log2(e)/T)
    const float row_max = bv, inv_t = 1.44269504088896340736f / temp;

    // 2. mass of every tile; wavefront w takes tiles w, w+16, ...
    const int n_tiles = (V + SAMPLE_TILE - 1) / SAMPLE_TILE;
    for (int t = wave; t < n_tiles; t += SAMPLE_BLOCK / MLLM_WAVE) {
        float s = 0.f;
        const int base = t * SAMPLE_TILE;
        for (int k0 = 0; k0 < SAMPLE_TILE / MLLM_WAVE; k0 += 8) {
            float v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = row[min(base + (k0 + k) * MLLM_WAVE + lane, V - 1)];
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (base + (k0 + k) * MLLM_WAVE + lane < V) s += exp2f((v[k] - row_max) * inv_t);
        }
        s = wave_sum(s);
        if (lane == 0) tile_mass[t] = s;
    }
    __syncthreads();

    // 3. the tile that holds the target
    if (tid == 0) {
        float total = 0.f;
        for (int t = 0; t < n_tiles; ++t) total += tile_mass[t];
        const float target = u[r] * total;
        float before = 0.f;
        int pick = -1, last = 0;
        float rest = 0.f;
        for (int t = 0; t < n_tiles; ++t) {
            if (tile_mass[t] > 0.f) last = t;
            if (pick < 0 && target < before + tile_mass[t]) { pick = t; rest = target - before; }
            before += tile_mass[t];
        }
        if (pick < 0) { pick = last; rest = INFINITY; }      // rounding at the top end: last entry with mass
        sh_tile = pick;
        sh_rest = rest;
    }
    __syncthreads();

    // 4. inside the tile: 8 consecutive entries per thread; the first SAMPLE_TILE/8 threads suffice
    const bool worker = tid < SAMPLE_TILE / 8;
    const int base = sh_tile * SAMPLE_TILE + (worker ? tid : 0) * 8;
    const float rest = sh_rest;
    float p[8], local = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        p[k] = (worker && base + k < V) ? exp2f((row[min(base + k, V - 1)] - row_max) * inv_t) : 0.f;
        local += p[k];
    }
    // exclusive prefix of `local` over the workgroup, in thread order
    float incl = local;
#pragma unroll
    for (int off = 1; off < MLLM_WAVE; off <<= 1) {
        const float o = __shfl_up(incl, off, MLLM_WAVE);
        if (lane >= off) incl += o;
    }
    if (worker && lane == MLLM_WAVE - 1) wave_mass[wave] = incl;
    __syncthreads();
    float before = incl - local;
    for (int w = 0; w < wave && w < SAMPLE_TILE / 8 / MLLM_WAVE; ++w) before += wave_mass[w];
    // the first thread (in order) whose range reaches the target; if none does, the last with mass
    const bool hit = worker && rest < before + local && local > 0.f;
    const bool has_mass = worker && local > 0.f;
    // lowest hitting thread / highest thread with mass, through LDS atomics
    __shared__ int first_hit, last_mass;
    if (tid == 0) { first_hit = 0x7fffffff; last_mass = -1; }
    __syncthreads();
    if (hit) atomicMin(&first_hit, tid);
    if (has_mass) atomicMax(&last_mass, tid);
    __syncthreads();
    const int chosen = first_hit != 0x7fffffff ? first_hit : last_mass;
    if (tid == chosen) {
        float c = before;
        int pick = -1, last = base;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            if (p[k] > 0.f) last = base + k;
            c += p[k];
            if (pick < 0 && rest < c && p[k] > 0.f) pick = base + k;
        }
        const int tok = pick >= 0 ? pick : last;
        out[r] = tok;
        if (mirror != nullptr) mirror[r] = tok;
    }
}

extern "C" {

// Chunks of the first stage for a row of V values: the scratch holds n * chunks floats and ints.
int mllm_argmax_chunks(int V) { return (V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK; }

// out[r] = index of the largest of row r (the lowest on ties); `mirror`, if given, gets the same (see above).
int mllm_argmax_mirrored(const float* logits, int ld, int n, int V, int* out, int* mirror, float* part_val,
                         int* part_idx, hipStream_t stream) {
    if (n <= 0) return 0;
    if (V <= 0) return -1;
    const int n_chunks = (V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
    argmax_stage1<<<dim3(n_chunks, n), SAMPLE_THREADS, 0, stream>>>(logits, ld, V, n_chunks, part_val, part_idx, out, mirror);
    MLLM_LAUNCH_CHECK();
    if (n_chunks > 1) {
        argmax_stage2<<<n, MLLM_WAVE, 0, stream>>>(part_val, part_idx, n_chunks, out, mirror);
        MLLM_LAUNCH_CHECK();
    }
    return 0;
}

int mllm_argmax(const float* logits, int ld, int n, int V, int* out, float* part_val, int* part_idx,
                hipStream_t stream) {
    return mllm_argmax_mirrored(logits, ld, n, V, out, nullptr, part_val, part_idx, stream);
}

}  // extern "C"

// Scratch of the entry point that allocates nothing: the first stage's values, then its indices.
// In host code this name is only a handle for hipGetSymbolAddress; the array's address on a device is
// looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[MLLM_ARGMAX_NOALLOC_MAX_PAIRS * (sizeof(float) + sizeof(int))];

#define NOALLOC_MAX_DEVICES 64
static void* g_scratch_ptr[NOALLOC_MAX_DEVICES];     // per device; null until looked up
static std::mutex g_scratch_mutex;

// The address of `scratch` on the current device (looked up at the first call on that device).
static hipError_t scratch_on_current_device(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (p == nullptr) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return hipSuccess;
}

extern "C" {

int mllm_argmax_noalloc_max_pairs(void) { return MLLM_ARGMAX_NOALLOC_MAX_PAIRS; }

int mllm_argmax_noalloc(const float* logits, int ld, int n, int V, int* out, hipStream_t stream) {
    if (n <= 0) return 0;
    if (V <= 0) return -1;
    const int n_chunks = (V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
    if (static_cast<long long>(n) * n_chunks > MLLM_ARGMAX_NOALLOC_MAX_PAIRS) return -3;
    void* base = nullptr;
    const hipError_t e = scratch_on_current_device(&base);
    if (e != hipSuccess) return static_cast<int>(e);
    float* part_val = static_cast<float*>(base);
    int* part_idx = reinterpret_cast<int*>(static_cast<unsigned char*>(base) +
                                           MLLM_ARGMAX_NOALLOC_MAX_PAIRS * sizeof(float));
    return mllm_argmax(logits, ld, n, V, out, part_val, part_idx, stream);
}

int mllm_sample_mirrored(const float* logits, int ld, int n, int V, const float* temperature, const float* u,
                         int* out, int* mirror, hipStream_t stream) {
    if (n <= 0) return 0;
    if (V <= 0 || V > SAMPLE_TILE * SAMPLE_MAX_TILES) return -1;
    sample_kernel<<<n, SAMPLE_BLOCK, 0, stream>>>(logits, ld, V, temperature, u, out, mirror);
    MLLM_LAUNCH_CHECK();
    return 0;
}

int mllm_sample(const float* logits, int ld, int n, int V, const float* temperature, const float* u, int* out,
                hipStream_t stream) {
    return mllm_sample_mirrored(logits, ld, n, V, temperature, u, out, nullptr, stream);
}

}  // extern "C"

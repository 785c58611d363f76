// Embedding, LayerNorm and key/value page writes for gfx950.
#include <algorithm>

#include "common.h"

// ---------------------------------------------------------------------------
// Token + position embedding: x[t,:] = wte[ids[t],:] + wpe[pos[t],:]   (fp32 out)
// /root/reference/src/kernels/embedding.cu:23-43. wpe may be null (no learned positions).
// With `src` (optional): where src[t] >= 0, token t's id is prev[src[t]], a token that an earlier step
// sampled on the device and the host has not read yet; ids[t] is not read then.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const int* __restrict__ pos,
                             const T* __restrict__ wte, const T* __restrict__ wpe,
                             float* __restrict__ x, int D, const int* __restrict__ src,
                             const int* __restrict__ prev, int n_prev) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (src != nullptr) {
        const int s = src[t];
        if (s >= 0 && s < n_prev) id = prev[s];
    }
    const T* te = wte + static_cast<size_t>(id) * D;
    float* xr = x + static_cast<size_t>(t) * D;
    if (wpe != nullptr) {
        const T* pe = wpe + static_cast<size_t>(pos[t]) * D;
        for (int d = threadIdx.x; d < D; d += blockDim.x) xr[d] = to_float(te[d]) + to_float(pe[d]);
    } else {
        for (int d = threadIdx.x; d < D; d += blockDim.x) xr[d] = to_float(te[d]);
    }
}

// ---------------------------------------------------------------------------
// Token ids fed back on the device: ids[i] = prev[src[i]] where src[i] >= 0 (the request's
// newest token is the one an earlier step sampled into prev and the host has not read yet);
// other ids stay as the host wrote them.
// ---------------------------------------------------------------------------
__global__ void select_tokens_kernel(int* __restrict__ ids, const int* __restrict__ src,
                                     const int* __restrict__ prev, int n, int n_prev) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int s = src[i];
    if (s >= 0 && s < n_prev) ids[i] = prev[s];
}

// ---------------------------------------------------------------------------
// LayerNorm over the last dimension, statistics in fp32, two passes:
// mean, then biased variance of (x - mean); y = (x - mean) * rsqrt(var + eps) * g + b.
// /root/reference/src/kernels/layernorm.cu:32-49. `rows` (optional) selects input rows.
// ---------------------------------------------------------------------------
template <typename OutT>
__global__ void layernorm_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                 const float* __restrict__ gamma, const float* __restrict__ beta,
                                 OutT* __restrict__ y, int D, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    const float* xr = x + static_cast<size_t>(src) * D;
    OutT* yr = y + static_cast<size_t>(r) * D;
    // Up to LN_REGS elements per thread stay in registers (one pass over memory); rows longer
    // than blockDim * LN_REGS read the remainder again.
    constexpr int LN_REGS = 8;
    float v[LN_REGS];
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < LN_REGS; ++u) {
        const int d = threadIdx.x + u * blockDim.x;
        v[u] = d < D ? xr[d] : 0.f;
        s += v[u];
    }
    for (int d = threadIdx.x + LN_REGS * blockDim.x; d < D; d += blockDim.x) s += xr[d];
    const float mean = block_sum(s, scratch) / static_cast<float>(D);
    float q = 0.f;
#pragma unroll
    for (int u = 0; u < LN_REGS; ++u) {
        if (threadIdx.x + u * blockDim.x < D) { const float c = v[u] - mean; q += c * c; }
    }
    for (int d = threadIdx.x + LN_REGS * blockDim.x; d < D; d += blockDim.x) {
        const float c = xr[d] - mean;
        q += c * c;
    }
    const float var = block_sum(q, scratch) / static_cast<float>(D);
    const float inv = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int u = 0; u < LN_REGS; ++u) {
        const int d = threadIdx.x + u * blockDim.x;
        if (d < D) {
            float o = (v[u] - mean) * inv * gamma[d];
            if (beta) o += beta[d];
            yr[d] = from_float<OutT>(o);
        }
    }
    for (int d = threadIdx.x + LN_REGS * blockDim.x; d < D; d += blockDim.x) {
        float o = (xr[d] - mean) * inv * gamma[d];
        if (beta) o += beta[d];
        yr[d] = from_float<OutT>(o);
    }
}

// Same norm, one wavefront per row (WAVES rows per workgroup), the row in registers as float4:
// for D % 4 == 0 and D <= 2048. Fewer, fatter workgroups and 16-byte accesses.
template <typename OutT, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
layernorm_wave_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                      const float* __restrict__ gamma, const float* __restrict__ beta,
                      OutT* __restrict__ y, int n, int D, float eps) {
    // (the wavefront's index as a scalar, so that the exit below is a real branch; every load is
    // issued without a condition, from a clamped index, and all of them before the first use: a
    // load under a condition, or one left inside the last loop, starts only when the statistics
    // are done and adds its whole latency)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int r = blockIdx.x * WAVES + wave;
    if (r >= n) return;
    const int src = rows ? rows[r] : r;
    const float4* xr = reinterpret_cast<const float4*>(x + static_cast<size_t>(src) * D);
    const float4* g4 = reinterpret_cast<const float4*>(gamma);
    const float4* b4 = reinterpret_cast<const float4*>(beta ? beta : gamma);
    const int nq = D / 4, n_u = (nq + 63) / 64;
    float4 v[8], gg[8], bb[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < n_u) v[u] = xr[min(lane + 64 * u, nq - 1)];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        if (u < n_u) {
            const int i = min(lane + 64 * u, nq - 1);
            gg[u] = g4[i];
            bb[u] = b4[i];
        }
    }
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < n_u && lane + 64 * u < nq) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
    const float mean = wave_sum(s) / static_cast<float>(D);
    float q = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        if (u < n_u && lane + 64 * u < nq) {
            const float a = v[u].x - mean, b = v[u].y - mean, c = v[u].z - mean, d = v[u].w - mean;
            q += (a * a + b * b) + (c * c + d * d);
        }
    }
    const float inv = 1.0f / sqrtf(wave_sum(q) / static_cast<float>(D) + eps);
    OutT* yr = y + static_cast<size_t>(r) * D;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int i = lane + 64 * u;
        if (u < n_u && i < nq) {
            const float4 g = gg[u];
            const float4 b = beta ? bb[u] : make_float4(0.f, 0.f, 0.f, 0.f);
            const float o0 = (v[u].x - mean) * inv * g.x + b.x, o1 = (v[u].y - mean) * inv * g.y + b.y;
            const float o2 = (v[u].z - mean) * inv * g.z + b.z, o3 = (v[u].w - mean) * inv * g.w + b.w;
            if (sizeof(OutT) == 2) {
                uint2 pk;
                pk.x = pack_bf16x2(o0, o1);
                pk.y = pack_bf16x2(o2, o3);
                *reinterpret_cast<uint2*>(yr + 4 * i) = pk;
            } else {
                *reinterpret_cast<float4*>(yr + 4 * i) = make_float4(o0, o1, o2, o3);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Key/value write: copies the key and value columns of each token's row into the
// row `slots[t]` of the page pools (slot = page * page_size + offset; < 0: skip).
// /root/reference/src/kernels/prefill/append_kv.cu:28-46.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void kv_append_kernel(const T* __restrict__ src, int src_stride, int k_col, int v_col,
                                 T* __restrict__ k_pages, T* __restrict__ v_pages, int kv_dim,
                                 const int* __restrict__ slots) {
    const int t = blockIdx.x;
    const int slot = slots[t];
    if (slot < 0) return;
    const T* ks = src + static_cast<size_t>(t) * src_stride + k_col;
    const T* vs = src + static_cast<size_t>(t) * src_stride + v_col;
    T* kd = k_pages + static_cast<size_t>(slot) * kv_dim;
    T* vd = v_pages + static_cast<size_t>(slot) * kv_dim;
    for (int d = threadIdx.x; d < kv_dim; d += blockDim.x) {
        kd[d] = ks[d];
        vd[d] = vs[d];
    }
}

// ---------------------------------------------------------------------------
// Fixed-size per-request state: the slot of every request that starts at position 0 in this
// step (starts[b] == 0: nothing of it is cached yet) is cleared before the layers run, on the
// device, so that the step can be replayed as a graph. Slots < 0 (padding rows) are skipped.
// One workgroup column per request; `words` 4-byte words per slot.
// ---------------------------------------------------------------------------
__global__ void reset_state_kernel(uint32_t* __restrict__ state, size_t words, const int* __restrict__ slots,
                                   const int* __restrict__ starts) {
    const int b = blockIdx.y;
    const int slot = slots[b];
    if (slot < 0 || starts[b] != 0) return;
    uint32_t* row = state + static_cast<size_t>(slot) * words;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < words;
         i += static_cast<size_t>(gridDim.x) * blockDim.x)
        row[i] = 0u;
}

extern "C" {

int mllm_reset_state(void* state, size_t slot_bytes, int n_slots, const int* slots, const int* starts, int B,
                     hipStream_t stream) {
    if (B <= 0 || slot_bytes == 0) return 0;
    if (slot_bytes % 4 != 0 || (reinterpret_cast<uintptr_t>(state) & 3) != 0 || n_slots < 1) return -1;
    const size_t words = slot_bytes / 4;
    const unsigned gx = static_cast<unsigned>(std::min<size_t>((words + 255) / 256, 64));
    reset_state_kernel<<<dim3(gx, B), 256, 0, stream>>>(static_cast<uint32_t*>(state), words, slots, starts);
    MLLM_LAUNCH_CHECK();
    return 0;
}

int mllm_embed(const int* ids, const int* pos, const void* wte, const void* wpe, float* x, int T, int D,
               int dtype, const int* src, const int* prev, int n_prev, hipStream_t stream) {
    if (T <= 0) return 0;
    if (dtype == MLLM_F32)
        embed_kernel<float><<<T, 256, 0, stream>>>(ids, pos, (const float*)wte, (const float*)wpe, x, D, src, prev, n_prev);
    else
        embed_kernel<bf16_t><<<T, 256, 0, stream>>>(ids, pos, (const bf16_t*)wte, (const bf16_t*)wpe, x, D, src, prev, n_prev);
    MLLM_LAUNCH_CHECK();
    return 0;
}

int mllm_select_tokens(int* ids, const int* src, const int* prev, int n, int n_prev, hipStream_t stream) {
    if (n <= 0) return 0;
    select_tokens_kernel<<<(n + 255) / 256, 256, 0, stream>>>(ids, src, prev, n, n_prev);
    MLLM_LAUNCH_CHECK();
    return 0;
}

int mllm_layernorm(const float* x, const int* rows, const float* gamma, const float* beta, void* y, int n,
                   int D, float eps, int out_dtype, hipStream_t stream) {
    if (n <= 0) return 0;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gamma) |
                           reinterpret_cast<uintptr_t>(beta) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    if (D % 4 == 0 && D <= 2048 && aligned) {
        // Workgroups start at a limited rate (about 200 a microsecond over the chip): many rows go eight to a
        // workgroup instead of four (2,048 rows of 768: 6.9 us with 512 workgroups of four)
        if (n >= 512) {
            const int blocks = (n + 7) / 8;
            if (out_dtype == MLLM_F32)
                layernorm_wave_kernel<float, 8><<<blocks, 512, 0, stream>>>(x, rows, gamma, beta, (float*)y, n, D, eps);
            else
                layernorm_wave_kernel<bf16_t, 8><<<blocks, 512, 0, stream>>>(x, rows, gamma, beta, (bf16_t*)y, n, D, eps);
        } else {
            const int blocks = (n + 3) / 4;
            if (out_dtype == MLLM_F32)
                layernorm_wave_kernel<float, 4><<<blocks, 256, 0, stream>>>(x, rows, gamma, beta, (float*)y, n, D, eps);
            else
                layernorm_wave_kernel<bf16_t, 4><<<blocks, 256, 0, stream>>>(x, rows, gamma, beta, (bf16_t*)y, n, D, eps);
        }
        MLLM_LAUNCH_CHECK();
        return 0;
    }
    const int threads = D >= 1024 ? 512 : 256;
    if (out_dtype == MLLM_F32)
        layernorm_kernel<float><<<n, threads, 0, stream>>>(x, rows, gamma, beta, (float*)y, D, eps);
    else
        layernorm_kernel<bf16_t><<<n, threads, 0, stream>>>(x, rows, gamma, beta, (bf16_t*)y, D, eps);
    MLLM_LAUNCH_CHECK();
    return 0;
}

int mllm_kv_append(const void* src, int src_stride, int k_col, int v_col, void* k_pages, void* v_pages,
                   int kv_dim, const int* slots, int T, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    const int threads = kv_dim >= 512 ? 256 : 64;
    if (dtype == MLLM_F32)
        kv_append_kernel<float><<<T, threads, 0, stream>>>((const float*)src, src_stride, k_col, v_col,
                                                            (float*)k_pages, (float*)v_pages, kv_dim, slots);
    else
        kv_append_kernel<bf16_t><<<T, threads, 0, stream>>>((const bf16_t*)src, src_stride, k_col, v_col,
                                                             (bf16_t*)k_pages, (bf16_t*)v_pages, kv_dim, slots);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

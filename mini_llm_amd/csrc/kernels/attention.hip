// Causal attention over the paged cache, any dtype and head size: one wavefront
// per (query token, head). It serves prompt portions and decoded tokens alike: a
// query at position p of sequence b reads keys [lo, p] of b's pages, where
// lo = max(0, p - window + 1) for a windowed cache and 0 otherwise. The keys and
// values of the step's own tokens must already be in the pages.
//
// Scores, softmax and the value mix are fp32 with the running-maximum recurrence of
// /root/reference/src/kernels/prefill/flashattention.cu:129-178
// (m' = max(m, s); alpha = e^(m-m'); p = e^(s-m'); o = o*alpha + p*v; l = l*alpha + p; out = o/l),
// applied to 64 keys at a time. The reference's decode kernel adds 1e-6 to the
// denominator (/root/reference/src/kernels/decode/paged_attention.cu:97); this does not.
#include "common.h"

#define ATT_WAVES 4
#define ATT_MAX_ACC 4   // head_dim <= 64 * ATT_MAX_ACC

template <typename T>
__global__ void __launch_bounds__(ATT_WAVES * MLLM_WAVE)
paged_attention_generic(const T* __restrict__ q, int q_stride, int q_col,
                        const T* __restrict__ k_pages, const T* __restrict__ v_pages, int kv_dim,
                        const int* __restrict__ block_tables, int max_blocks,
                        const int* __restrict__ token_seq, const int* __restrict__ positions,
                        int n_tokens, int n_heads, int n_kv_heads, int head_dim, int page_size,
                        float scale, int window, T* __restrict__ out, int out_stride) {
    extern __shared__ float smem[];
    const int wave = threadIdx.x / MLLM_WAVE, lane = threadIdx.x % MLLM_WAVE;
    const int pair = blockIdx.x * ATT_WAVES + wave;
    if (pair >= n_tokens * n_heads) return;       // whole wave leaves; no block-wide sync below
    const int t = pair / n_heads, h = pair % n_heads;
    const int hk = h / (n_heads / n_kv_heads);
    const int b = token_seq[t];
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* table = block_tables + static_cast<size_t>(b) * max_blocks;

    float* q_s = smem + wave * (head_dim + 2 * MLLM_WAVE);
    float* p_s = q_s + head_dim;
    int* row_s = reinterpret_cast<int*>(p_s + MLLM_WAVE);

    const T* qp = q + static_cast<size_t>(t) * q_stride + q_col + h * head_dim;
    for (int d = lane; d < head_dim; d += MLLM_WAVE) q_s[d] = to_float(qp[d]) * scale;
    wave_lds_sync();

    float m = -INFINITY, l = 0.f;
    float acc[ATT_MAX_ACC] = {0.f, 0.f, 0.f, 0.f};
    const int kv_off = hk * head_dim;

    for (int j0 = lo; j0 <= p; j0 += MLLM_WAVE) {
        // phase A: one key per lane
        const int j = j0 + lane;
        const bool valid = j <= p;
        float s = -INFINITY;
        int row = 0;
        if (valid) {
            row = table[j / page_size] * page_size + j % page_size;
            const T* kp = k_pages + static_cast<size_t>(row) * kv_dim + kv_off;
            float dot = 0.f;
            for (int d = 0; d < head_dim; d += 8) {
                float kv[8];
                load8(kp + d, kv);
#pragma unroll
                for (int i = 0; i < 8; ++i) dot = fmaf(q_s[d + i], kv[i], dot);
            }
            s = dot;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        const float pj = valid ? expf(s - m_new) : 0.f;
        l = l * alpha + wave_sum(pj);
        m = m_new;
        wave_lds_sync();          // the previous round's readers are done
        p_s[lane] = pj;
        row_s[lane] = row;
        wave_lds_sync();
        // phase B: one (or a few) output dimensions per lane; p_s/row_s are read wave-wide
        const int n_keys = min(MLLM_WAVE, p - j0 + 1);
#pragma unroll
        for (int a = 0; a < ATT_MAX_ACC; ++a) {
            const int d = lane + a * MLLM_WAVE;
            if (d < head_dim) {
                float o = acc[a] * alpha;
                for (int jj = 0; jj < n_keys; ++jj) {
                    const T* vp = v_pages + static_cast<size_t>(row_s[jj]) * kv_dim + kv_off;
                    o = fmaf(p_s[jj], to_float(vp[d]), o);
                }
                acc[a] = o;
            }
        }
    }
    T* op = out + static_cast<size_t>(t) * out_stride + h * head_dim;
    const float inv_l = 1.0f / l;
#pragma unroll
    for (int a = 0; a < ATT_MAX_ACC; ++a) {
        const int d = lane + a * MLLM_WAVE;
        if (d < head_dim) op[d] = from_float<T>(acc[a] * inv_l);
    }
}

extern "C" {

// Returns 0, a HIP error code, or -1 for a head size the kernel refuses.
int mllm_paged_attention_generic(const void* q, int q_stride, int q_col, const void* k_pages,
                                 const void* v_pages, int kv_dim, const int* block_tables, int max_blocks,
                                 const int* token_seq, const int* positions, int n_tokens, int n_heads,
                                 int n_kv_heads, int head_dim, int page_size, float scale, int window,
                                 void* out, int out_stride, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (head_dim % 8 != 0 || head_dim > 64 * ATT_MAX_ACC || n_heads % n_kv_heads != 0) return -1;
    const int pairs = n_tokens * n_heads;
    const int blocks = (pairs + ATT_WAVES - 1) / ATT_WAVES;
    const size_t smem = static_cast<size_t>(ATT_WAVES) * (head_dim + 2 * MLLM_WAVE) * sizeof(float);
    if (dtype == MLLM_F32)
        paged_attention_generic<float><<<blocks, ATT_WAVES * MLLM_WAVE, smem, stream>>>(
            (const float*)q, q_stride, q_col, (const float*)k_pages, (const float*)v_pages, kv_dim,
            block_tables, max_blocks, token_seq, positions, n_tokens, n_heads, n_kv_heads, head_dim,
            page_size, scale, window, (float*)out, out_stride);
    else
        paged_attention_generic<bf16_t><<<blocks, ATT_WAVES * MLLM_WAVE, smem, stream>>>(
            (const bf16_t*)q, q_stride, q_col, (const bf16_t*)k_pages, (const bf16_t*)v_pages, kv_dim,
            block_tables, max_blocks, token_seq, positions, n_tokens, n_heads, n_kv_heads, head_dim,
            page_size, scale, window, (bf16_t*)out, out_stride);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

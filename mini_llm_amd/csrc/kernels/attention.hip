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

// ---------------------------------------------------------------------------------------------
// Prompt portions at any head size (multiples of 16 up to 256), any page size, float32 or bfloat16
// storage: 64 queries of one sequence and one head per workgroup share tiles of 64 keys and values
// that are gathered through the block table into LDS as float32, and the two products run on the
// matrix cores in TRUE 32-bit (v_mfma_f32_16x16x4_f32: float32 operands, no reduced-precision mode).
// This is the 32-bit path's prefill attention, and the bfloat16 path's where the bfloat16 matrix-core
// kernel refuses the sizes. (The one-wavefront-per-query kernel above re-reads every key from memory
// for every query: 5.6 TFLOP/s at 8 x 512 tokens.)
//
// As in the bfloat16 kernel everything is computed transposed, so that a lane owns ONE query:
//   S^T = K Q^T    A = 16 keys x 4 dims from LDS, B = the lane's query fragment (registers)
//   O^T = V^T P^T  A = 16 dims x 4 keys from the transposed values in LDS, B = P^T straight from the S^T
//                  accumulators (the k index of a product may be permuted as long as both operands agree)
// Lane l of a wavefront has query l % 16; its k index l / 16 stands, in product j of a group of four, for
// dim 16c + 4 (l / 16) + j (keys: for key 4 (l / 16) + j), so that one 16-byte LDS read feeds four products.
// Recurrence: /root/reference/src/kernels/prefill/flashattention.cu:129-178, in base 2.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
#define TL_BQ 64
#define TL_BK 64
#define TL_VSTRIDE (TL_BK + 4)      // floats per transposed value row: 17 x 16 bytes, odd, so 16-byte reads of 16 rows do not collide

template <typename T> __device__ __forceinline__ f32x4_t load4f(const T* p);
template <> __device__ __forceinline__ f32x4_t load4f<float>(const float* p) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    return f32x4_t{v.x, v.y, v.z, v.w};
}
template <> __device__ __forceinline__ f32x4_t load4f<bf16_t>(const bf16_t* p) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    return f32x4_t{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                   __uint_as_float(v.y & 0xffff0000u)};
}
template <typename T> __device__ __forceinline__ void store4f(T* p, f32x4_t v);
template <> __device__ __forceinline__ void store4f<float>(float* p, f32x4_t v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
template <> __device__ __forceinline__ void store4f<bf16_t>(bf16_t* p, f32x4_t v) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
}

// DC: the most 16-dim chunks of a head (head_dim <= 16 DC); loops over chunks are unrolled to DC and
// predicated, so that the register arrays are indexed by constants.
template <typename T, int DC>
__global__ void __launch_bounds__(256)
paged_attention_tiled(const T* __restrict__ q, int q_stride, int q_col, const T* __restrict__ k_pages,
                      const T* __restrict__ v_pages, int kv_dim, const int* __restrict__ block_tables, int max_blocks,
                      const int* __restrict__ cu_q, const int* __restrict__ ctx_len, int n_seqs, int n_heads,
                      int n_kv_heads, int head_dim, int page_size, float scale_log2e, int window,
                      T* __restrict__ out, int out_stride) {
    extern __shared__ __attribute__((aligned(16))) float tl_smem[];
    const int n_c = head_dim / 16;                 // 16-dim chunks
    const int ldk = head_dim + 4;                  // floats per key row: (head_dim / 4 + 1) x 16 bytes, odd
    float* Ks = tl_smem;                           // [TL_BK][ldk]
    float* Vt = tl_smem + TL_BK * ldk;             // [head_dim][TL_VSTRIDE]

    // which sequence and which of its 64-query tiles (the heaviest causal tiles first)
    int tile = gridDim.y - 1 - blockIdx.y, b = 0, q_begin = 0, q_len = 0;
    for (; b < n_seqs; ++b) {
        q_begin = cu_q[b];
        q_len = cu_q[b + 1] - q_begin;
        const int nt = (q_len + TL_BQ - 1) / TL_BQ;
        if (tile < nt) break;
        tile -= nt;
    }
    if (b >= n_seqs) return;                       // surplus workgroup; the whole workgroup leaves

    const int h = blockIdx.x, hk = h / (n_heads / n_kv_heads);
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int G = lane / 16, c16 = lane % 16;
    const int start = ctx_len[b] - q_len;          // position of the step's first query
    const int q0 = tile * TL_BQ;
    const int qi = q0 + wave * 16 + c16;           // this lane's query within the step's rows
    const bool q_ok = qi < q_len;
    const int p = start + min(qi, q_len - 1);      // its position (a lane beyond the last query repeats it; never stored)
    const int p_first = start + q0, p_last = start + min(q0 + TL_BQ, q_len) - 1;
    const int k_lo = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int my_lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    // the last position any of this wavefront's queries may see (uniform over the wavefront)
    const int wave_last = start + min(q0 + wave * 16 + 15, q_len - 1);
    const int* table = block_tables + static_cast<size_t>(b) * max_blocks;
    const size_t kv_off = static_cast<size_t>(hk) * head_dim;

    // the lane's query fragment, scaled: qf[c][j] = q[16c + 4G + j] * scale * log2(e)
    f32x4_t qf[DC];
    f32x4_t o[DC];
    const T* qp = q + static_cast<size_t>(q_begin + min(qi, q_len - 1)) * q_stride + q_col + h * head_dim + 4 * G;
#pragma unroll
    for (int c = 0; c < DC; ++c) {
        o[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        qf[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (c < n_c) qf[c] = load4f<T>(qp + 16 * c) * scale_log2e;
    }
    float m = -INFINITY, l = 0.f;

    for (int k0 = k_lo - k_lo % TL_BK; k0 <= p_last; k0 += TL_BK) {
        __syncthreads();                           // the previous tile's readers are done
        // stage 64 keys and values: thread t has key t % 64 and a quarter of its dims. Keys outside
        // [k_lo, p_last] are not in the pages (not written yet, or given back by a window): zeros.
        {
            const int key = tid % TL_BK, part = tid / TL_BK, j = k0 + key;
            const bool live = j >= k_lo && j <= p_last;
            size_t row = 0;
            if (live) row = static_cast<size_t>(table[j / page_size]) * page_size + j % page_size;
            const T* kp = k_pages + row * kv_dim + kv_off;
            const T* vp = v_pages + row * kv_dim + kv_off;
            const int d_per = head_dim / 4;        // a multiple of 4
            for (int d = part * d_per; d < (part + 1) * d_per; d += 4) {
                f32x4_t kv = f32x4_t{0.f, 0.f, 0.f, 0.f}, vv = kv;
                if (live) { kv = load4f<T>(kp + d); vv = load4f<T>(vp + d); }
                *reinterpret_cast<f32x4_t*>(Ks + key * ldk + d) = kv;
#pragma unroll
                for (int i = 0; i < 4; ++i) Vt[(d + i) * TL_VSTRIDE + key] = vv[i];
            }
        }
        __syncthreads();
        if (k0 > wave_last) continue;              // nothing here for this wavefront's queries (it still keeps the barriers)
        // S^T for the tile: 4 groups of 16 keys; lane holds keys k0 + 16 g + 4 G + i, i = 0..3, of its query
        f32x4_t s[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            s[g] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            const float* kr = Ks + (g * 16 + c16) * ldk + 4 * G;
#pragma unroll
            for (int c = 0; c < DC; ++c) {
                if (c < n_c) {
                    const f32x4_t kf = *reinterpret_cast<const f32x4_t*>(kr + 16 * c);
#pragma unroll
                    for (int j = 0; j < 4; ++j) s[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[j], qf[c][j], s[g], 0, 0, 0);
                }
            }
        }
        // mask, running maximum and sum (scalars per lane, merged over the four lane groups of the query)
        float mx = -INFINITY;
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = k0 + 16 * g + 4 * G + i;
                s[g][i] = (j <= p && j >= my_lo) ? s[g][i] : -INFINITY;
                mx = fmaxf(mx, s[g][i]);
            }
        const float m_new = fmaxf(m, rows_max(mx));
        // (a query none of whose keys has come yet keeps m = -inf: nothing to rescale, all weights zero)
        const float alpha = (m_new == -INFINITY) ? 1.f : exp2_for<T>(m - m_new);
        float sum = 0.f;
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s[g][i] = (m_new == -INFINITY) ? 0.f : exp2_for<T>(s[g][i] - m_new);
                sum += s[g][i];
            }
        l = l * alpha + rows_sum(sum);
        m = m_new;
        // O^T = O^T alpha + V^T P^T
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            if (c < n_c) {
                o[c] *= alpha;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x4_t vf = *reinterpret_cast<const f32x4_t*>(Vt + (16 * c + c16) * TL_VSTRIDE + 16 * g + 4 * G);
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[i], s[g][i], o[c], 0, 0, 0);
                }
            }
        }
    }
    if (!q_ok) return;
    // lane holds O^T[dims 16c + 4G + i][its query]
    const float inv_l = 1.f / l;
    T* op = out + static_cast<size_t>(q_begin + qi) * out_stride + h * head_dim + 4 * G;
#pragma unroll
    for (int c = 0; c < DC; ++c)
        if (c < n_c) store4f<T>(op + 16 * c, o[c] * inv_l);
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

// n_tiles_upper: an upper bound of the number of 64-query tiles, sum over sequences of ceil(q_len / 64)
// (e.g. n_tokens / 64 + n_seqs); surplus workgroups leave at once. The keys and values of the step's own
// tokens must already be in the pages. Returns 0, a HIP error code, or -1 for a head size that is no multiple
// of 16 or beyond 256, rows that are not 16-byte aligned, or more tiles than a grid holds.
int mllm_paged_attention_tiled(const void* q, int q_stride, int q_col, const void* k_pages, const void* v_pages,
                               int kv_dim, const int* block_tables, int max_blocks, const int* cu_q, const int* ctx_len,
                               int n_seqs, int n_tiles_upper, int n_heads, int n_kv_heads, int head_dim, int page_size,
                               float scale, int window, void* out, int out_stride, int dtype, hipStream_t stream) {
    if (n_seqs <= 0 || n_tiles_upper <= 0) return 0;
    if (head_dim % 16 != 0 || head_dim < 16 || head_dim > 256 || n_heads % n_kv_heads != 0 || n_tiles_upper > 65535 ||
        page_size < 1)
        return -1;
    const int esz = dtype == MLLM_F32 ? 4 : 2;
    if ((q_stride * esz) % 16 || (q_col * esz) % 16 || (kv_dim * esz) % 16 || (out_stride * esz) % 8) return -1;
    const dim3 grid(n_heads, n_tiles_upper);
    const size_t smem = (static_cast<size_t>(TL_BK) * (head_dim + 4) + static_cast<size_t>(head_dim) * TL_VSTRIDE) * sizeof(float);
    const float sl2 = scale * 1.44269504088896340736f;
#define TL_CASE(TYPE, DC)                                                                                          \
    do {                                                                                                           \
        static bool lds_allowed = false;      /* more than 64 KB of LDS is asked for once */                       \
        if (!lds_allowed) {                                                                                        \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(paged_attention_tiled<TYPE, DC>),      \
                                               hipFuncAttributeMaxDynamicSharedMemorySize,                         \
                                               static_cast<int>((TL_BK * (16 * DC + 4) + 16 * DC * TL_VSTRIDE) * sizeof(float))); \
            if (e != hipSuccess) return static_cast<int>(e);                                                       \
            lds_allowed = true;                                                                                    \
        }                                                                                                          \
        paged_attention_tiled<TYPE, DC><<<grid, 256, smem, stream>>>(                                              \
            (const TYPE*)q, q_stride, q_col, (const TYPE*)k_pages, (const TYPE*)v_pages, kv_dim, block_tables,     \
            max_blocks, cu_q, ctx_len, n_seqs, n_heads, n_kv_heads, head_dim, page_size, sl2, window, (TYPE*)out,   \
            out_stride);                                                                                           \
    } while (0)
    const int dc = head_dim <= 64 ? 4 : head_dim <= 128 ? 8 : 16;
    if (dtype == MLLM_F32) {
        if (dc == 4) TL_CASE(float, 4); else if (dc == 8) TL_CASE(float, 8); else TL_CASE(float, 16);
    } else {
        if (dc == 4) TL_CASE(bf16_t, 4); else if (dc == 8) TL_CASE(bf16_t, 8); else TL_CASE(bf16_t, 16);
    }
#undef TL_CASE
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

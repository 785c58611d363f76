// Decode attention over the paged cache for gfx950: one query token per (token, head),
// its keys split over `nsplit` workgroups so that small batches still fill the chip.
//
// Inside a workgroup, LPK lanes share one key: each lane loads 16 bytes of the key row
// and of the value row (so a wavefront covers 64/LPK whole rows per load instruction),
// the LPK partial dot products are summed with DPP shuffles, and every lane keeps the
// running maximum, sum and its slice of the output for the keys of its lane group
// (recurrence of /root/reference/src/kernels/prefill/flashattention.cu:129-178, in base 2).
// Groups, wavefronts and splits are merged with the same (m, l, o) rule. The splits of a
// (token, head) pair are merged either by the last workgroup to finish the pair, found through
// an atomic counter (no workgroup ever waits for another), or, with `partial_out`, not here at
// all: every workgroup leaves its state (maximum in base 2, sum, unnormalised output, fp32) in the
// workspace and the kernel that reads the attention output next merges them while it loads its
// operand (the few-row product of the output projection does), which costs no fence and no second
// pass here.
//
// It stands where the reference has its three-pass decode kernel
// (/root/reference/src/kernels/decode/paged_attention.cu:58-120); no 1e-6 is added to
// the denominator.
#include "common.h"

#define DEC_MAX_WAVES 16
#define DEC_TABLE_LDS 4096   // block-table entries staged in LDS: the most pages one workgroup's keys may span

// 16 bytes of a row: kept raw in registers while the load is in flight, widened to fp32 when used.
template <typename T> struct Vec16;
template <> struct Vec16<bf16_t> {
    static constexpr int N = 8;
    __device__ static void widen(const uint4& a, float (&v)[8]) {
        v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
        v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
        v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xffff0000u);
        v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xffff0000u);
    }
};
template <> struct Vec16<float> {
    static constexpr int N = 4;
    __device__ static void widen(const uint4& a, float (&v)[4]) {
        v[0] = __uint_as_float(a.x); v[1] = __uint_as_float(a.y);
        v[2] = __uint_as_float(a.z); v[3] = __uint_as_float(a.w);
    }
};
template <typename T>
__device__ __forceinline__ uint4 load_raw16(const T* p) { return *reinterpret_cast<const uint4*>(p); }
typedef unsigned int u32x4_nt __attribute__((ext_vector_type(4)));
template <typename T>
__device__ __forceinline__ uint4 load_stream16(const T* p) {
    const u32x4_nt v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_nt*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

template <typename T, int N>
__device__ __forceinline__ void merge_state(float& m, float& l, float (&o)[N], float m2, float l2,
                                            const float (&o2)[N]) {
    // empty states carry a large negative finite maximum and zero sums: their weight is 0 or
    // (both empty) irrelevant
    const float mn = fmaxf(m, m2);
    const float a = exp2_for<T>(m - mn), b = exp2_for<T>(m2 - mn);
    l = l * a + l2 * b;
#pragma unroll
    for (int e = 0; e < N; ++e) o[e] = o[e] * a + o2[e] * b;
    m = mn;
}

template <typename T, int LPK, int UNR>
__global__ void __launch_bounds__(UNR > 8 ? 512 : DEC_MAX_WAVES * MLLM_WAVE)
decode_attention_kernel(// the first 16 dwords arrive in registers with the wavefront: what the first loads need
                        const int* __restrict__ token_seq, const int* __restrict__ positions,
                        const int* __restrict__ block_tables, int max_blocks, int n_heads, int n_kv_heads,
                        int page_size, int window, int nsplit, const T* __restrict__ q, int q_stride, int q_col,
                        // the rest is loaded by the kernel
                        const T* __restrict__ k_pages, const T* __restrict__ v_pages, int kv_dim,
                        float scale_log2e, T* __restrict__ out, int out_stride,
                        float* __restrict__ ws_o, float* __restrict__ ws_ml, int* __restrict__ counters,
                        T* __restrict__ k_pages_w, T* __restrict__ v_pages_w, int k_col, int v_col,
                        const int* __restrict__ slots, int partial_out) {
    constexpr int EPL = Vec16<T>::N;        // elements per lane
    constexpr int DH = LPK * EPL;           // head size
    constexpr int KPW = MLLM_WAVE / LPK;    // keys per wavefront and load instruction
    __shared__ float sm_m[DEC_MAX_WAVES], sm_l[DEC_MAX_WAVES];
    __shared__ float sm_o[DEC_MAX_WAVES][DH];
    __shared__ int sm_last;
    __shared__ int sm_table[DEC_TABLE_LDS];
    const int n_waves = blockDim.x / MLLM_WAVE;

    const int pair = blockIdx.x, split = blockIdx.y;
    const int t = pair / n_heads, h = pair % n_heads;
    const int hk = h / (n_heads / n_kv_heads);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MLLM_WAVE), lane = threadIdx.x % MLLM_WAVE;
    const int c = lane % LPK, g = lane / LPK;
    // (token_seq == nullptr: every sequence brings one token, token t belongs to sequence t; the block
    // table can then be requested at once, beside the position, instead of after a load of its own)
    const int b = token_seq != nullptr ? token_seq[t] : t;
    const int* gtable_row = block_tables + static_cast<size_t>(b) * max_blocks;
    // Without a window the keys start at block 0 whatever the position is, and rows of the table are
    // filled to their end (zeros behind a sequence's last block): the whole row goes to LDS without
    // waiting for the position.
    const bool whole_row = window <= 0 && max_blocks <= DEC_TABLE_LDS;
    if (whole_row)
        for (int i = threadIdx.x; i < max_blocks; i += blockDim.x) sm_table[i] = gtable_row[i];
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int n_keys = p - lo + 1;
    const int per = (n_keys + nsplit - 1) / nsplit;
    const int kb = lo + split * per;
    const int ke = min(p + 1, kb + per);
    // With `slots`, the token's own key and value are not in the pages yet: they are read from
    // its row of q (columns k_col, v_col), and written to the pages by the first query head of
    // each key/value head. That key is taken by one lane group after the loop over the pages.
    const bool append = slots != nullptr;
    const bool own_here = append && ke == p + 1 && kb <= p;     // this workgroup's range holds the token itself
    const int ke_pages = own_here ? p : ke;                     // keys [kb, ke_pages) come from the pages
    const size_t col = static_cast<size_t>(hk) * DH + c * EPL;
    const int shift = __ffs(page_size) - 1;                     // page sizes are powers of two

    // The block table entries of this workgroup's keys go to LDS first, so that no key load waits
    // for a table load.
    const int first_blk = whole_row ? 0 : kb >> shift;
    const int n_blk = ke_pages > kb ? ((ke_pages - 1) >> shift) - first_blk + 1 : 0;
    if (!whole_row) {
        const int* gtable = gtable_row + first_blk;
        for (int i = threadIdx.x; i < n_blk; i += blockDim.x) sm_table[i] = gtable[i];
    }

    float qf[EPL];
    Vec16<T>::widen(load_raw16(q + static_cast<size_t>(t) * q_stride + q_col + h * DH + c * EPL), qf);
#pragma unroll
    for (int e = 0; e < EPL; ++e) qf[e] *= scale_log2e;
    uint4 k_own = make_uint4(0, 0, 0, 0), v_own = make_uint4(0, 0, 0, 0);
    const bool own_lanes = own_here && wave == 0 && g == 0;
    if (own_lanes) {
        const T* src = q + static_cast<size_t>(t) * q_stride + col;
        k_own = load_raw16(src + k_col);
        v_own = load_raw16(src + v_col);
        const int slot = slots[t];
        if (slot >= 0 && h % (n_heads / n_kv_heads) == 0) {
            const size_t wrow = static_cast<size_t>(slot) * kv_dim + col;
            *reinterpret_cast<uint4*>(k_pages_w + wrow) = k_own;
            *reinterpret_cast<uint4*>(v_pages_w + wrow) = v_own;
        }
    }
    __syncthreads();       // the table is in LDS

    // Running state (maximum in base 2, sum, output slice). The maximum starts at a large
    // negative finite number, so that no difference of two of them is NaN.
    constexpr float NEG = -1.0e30f;
    float m = NEG, l = 0.f, o[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) o[e] = 0.f;

    // A wavefront takes UNR groups of 64/LPK keys at a time. All their loads are issued
    // first, unconditionally (a key beyond the range loads the last key of the range again and is
    // masked when used): a load under a condition, even one that is uniform over the wavefront,
    // makes every later use wait for all loads in flight (measured: 7.6 -> 8.4 us at 512 keys).
    const int mask = page_size - 1;
    const int group_keys = n_waves * KPW;                 // distance between a wavefront's groups
    for (int j0 = kb + wave * KPW; j0 < ke_pages; j0 += group_keys * UNR) {
        uint4 kraw[UNR], vraw[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int j = min(j0 + u * group_keys + g, ke_pages - 1);
            const size_t row = (static_cast<size_t>(sm_table[(j >> shift) - first_blk]) << shift) + (j & mask);
            kraw[u] = load_stream16(k_pages + row * kv_dim + col);
            vraw[u] = load_stream16(v_pages + row * kv_dim + col);
        }
        float dot[UNR];
        float mx = NEG;
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            float kf[EPL];
            Vec16<T>::widen(kraw[u], kf);
            float d = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) d = fmaf(qf[e], kf[e], d);
            d = group_sum<LPK>(d);
            const bool valid = j0 + u * group_keys + g < ke_pages;
            dot[u] = valid ? d : NEG;
            mx = fmaxf(mx, dot[u]);
        }
        // one rescale of the state for the whole batch of keys
        const float mn = fmaxf(m, mx);
        const float a = exp2_for<T>(m - mn);
        l *= a;
#pragma unroll
        for (int e = 0; e < EPL; ++e) o[e] *= a;
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const float pj = dot[u] > NEG ? exp2_for<T>(dot[u] - mn) : 0.f;
            float vf[EPL];
            Vec16<T>::widen(vraw[u], vf);
            l += pj;
#pragma unroll
            for (int e = 0; e < EPL; ++e) o[e] = fmaf(pj, vf[e], o[e]);
        }
        m = mn;
    }
    if (own_lanes) {
        float kf[EPL], vf[EPL];
        Vec16<T>::widen(k_own, kf);
        Vec16<T>::widen(v_own, vf);
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) d = fmaf(qf[e], kf[e], d);
        d = group_sum<LPK>(d);
        const float mn = fmaxf(m, d);
        const float a = exp2_for<T>(m - mn), pj = exp2_for<T>(d - mn);
        l = l * a + pj;
#pragma unroll
        for (int e = 0; e < EPL; ++e) o[e] = o[e] * a + pj * vf[e];
        m = mn;
    }
    // Merges the states of all lane groups and wavefronts; the result is valid in lane group 0
    // of wavefront 0.
    auto block_merge = [&]() {
#pragma unroll
        for (int off = LPK; off < MLLM_WAVE; off <<= 1) {
            const float m2 = lane_xor(m, off), l2 = lane_xor(l, off);
            float o2[EPL];
#pragma unroll
            for (int e = 0; e < EPL; ++e) o2[e] = lane_xor(o[e], off);
            merge_state<T, EPL>(m, l, o, m2, l2, o2);
        }
        __syncthreads();                      // earlier readers of the LDS arrays are done
        if (g == 0) {
            if (c == 0) { sm_m[wave] = m; sm_l[wave] = l; }
#pragma unroll
            for (int e = 0; e < EPL; ++e) sm_o[wave][c * EPL + e] = o[e];
        }
        __syncthreads();
        if (wave == 0) {
            // lane group G takes the state of wavefront G, G + KPW, ... (all reads at once), then
            // the groups are merged as above
            m = NEG; l = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) o[e] = 0.f;
            for (int w = g; w < n_waves; w += KPW) {
                float o2[EPL];
#pragma unroll
                for (int e = 0; e < EPL; ++e) o2[e] = sm_o[w][c * EPL + e];
                merge_state<T, EPL>(m, l, o, sm_m[w], sm_l[w], o2);
            }
#pragma unroll
            for (int off = LPK; off < MLLM_WAVE; off <<= 1) {
                const float m2 = lane_xor(m, off), l2 = lane_xor(l, off);
                float o2[EPL];
#pragma unroll
                for (int e = 0; e < EPL; ++e) o2[e] = lane_xor(o[e], off);
                merge_state<T, EPL>(m, l, o, m2, l2, o2);
            }
        }
    };
    block_merge();
    T* op = out + static_cast<size_t>(t) * out_stride + h * DH + c * EPL;
    if (partial_out) {
        // the split's state as it is; whoever reads the workspace merges
        const size_t slot = static_cast<size_t>(pair) * nsplit + split;
        if (wave == 0 && g == 0) {
#pragma unroll
            for (int e = 0; e < EPL; ++e) ws_o[slot * DH + c * EPL + e] = o[e];
            if (c == 0) { ws_ml[slot * 2] = m; ws_ml[slot * 2 + 1] = l; }
        }
        return;
    }
    if (nsplit == 1) {
        if (wave == 0 && g == 0) {
            const float inv = 1.0f / l;
#pragma unroll
            for (int e = 0; e < EPL; ++e) op[e] = from_float<T>(o[e] * inv);
        }
        return;
    }
    // partial result of this split
    const size_t slot = static_cast<size_t>(pair) * nsplit + split;
    if (wave == 0 && g == 0) {
#pragma unroll
        for (int e = 0; e < EPL; ++e) ws_o[slot * DH + c * EPL + e] = o[e];
        if (c == 0) { ws_ml[slot * 2] = m; ws_ml[slot * 2 + 1] = l; }
    }
    // One thread's fences order the partial results around the counter (after the barrier its
    // release covers every thread's stores); a fence in every thread would write back and
    // invalidate the L2 once per wavefront, tens of microseconds in all.
    __syncthreads();
    if (threadIdx.x == 0) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        const int arrived = __hip_atomic_fetch_add(&counters[pair], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sm_last = (arrived == nsplit - 1) ? 1 : 0;
        if (sm_last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    __syncthreads();
    if (!sm_last) return;
    // Last workgroup of this (token, head): lane group G takes split G (all loads in flight at
    // once), then the same merge as above.
    m = NEG; l = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) o[e] = 0.f;
    for (int s0 = 0; s0 < nsplit; s0 += n_waves * KPW) {
        const int sidx = s0 + wave * KPW + g;
        if (sidx < nsplit) {
            const size_t sl = static_cast<size_t>(pair) * nsplit + sidx;
            const float m2 = __hip_atomic_load(&ws_ml[sl * 2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const float l2 = __hip_atomic_load(&ws_ml[sl * 2 + 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            float o2[EPL];
#pragma unroll
            for (int e = 0; e < EPL; ++e)
                o2[e] = __hip_atomic_load(&ws_o[sl * DH + c * EPL + e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            merge_state<T, EPL>(m, l, o, m2, l2, o2);
        }
    }
    block_merge();
    if (wave == 0 && g == 0) {
        const float inv = 1.0f / l;
#pragma unroll
        for (int e = 0; e < EPL; ++e) op[e] = from_float<T>(o[e] * inv);
    }
    if (threadIdx.x == 0) counters[pair] = 0;     // ready for the next launch
}

template <typename T>
static int launch_decode(int lpk, dim3 grid, int waves, hipStream_t stream, const T* q, int q_stride, int q_col,
                         const T* k_pages, const T* v_pages, int kv_dim, const int* block_tables,
                         int max_blocks, const int* token_seq, const int* positions, int n_heads,
                         int n_kv_heads, int page_size, float scale_log2e, int window, int nsplit, T* out,
                         int out_stride, float* ws_o, float* ws_ml, int* counters, T* k_pages_w, T* v_pages_w,
                         int k_col, int v_col, const int* slots, int partial_out) {
#define DEC_ARGS token_seq, positions, block_tables, max_blocks, n_heads, n_kv_heads, page_size, window,  \
            nsplit, q, q_stride, q_col, k_pages, v_pages, kv_dim, scale_log2e, out, out_stride,        \
            ws_o, ws_ml, counters, k_pages_w, v_pages_w, k_col, v_col, slots, partial_out
#define DEC_CASE(L)                                                                                    \
    case L:                                                                                            \
        decode_attention_kernel<T, L, 8><<<grid, waves * MLLM_WAVE, 0, stream>>>(DEC_ARGS);             \
        return 0;
    switch (lpk) {
        DEC_CASE(2) DEC_CASE(4) DEC_CASE(8) DEC_CASE(16) DEC_CASE(32) DEC_CASE(64)
        default: return -1;
    }
#undef DEC_CASE
#undef DEC_ARGS
}

// Merges the splits' states that `partial_out` left in the workspace into the attention output:
// one thread per 4 elements. For readers of the output that do not merge while they load.
template <typename T>
__global__ void merge_splits_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml, int nsplit,
                                    int head_dim, int n_heads, T* __restrict__ out, int out_stride, int total4) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total4) return;
    const int per_pair = head_dim / 4;
    const int pair = i / per_pair, e = (i % per_pair) * 4;
    float mx = -INFINITY;
    for (int s = 0; s < nsplit; ++s) mx = fmaxf(mx, ws_ml[(static_cast<size_t>(pair) * nsplit + s) * 2]);
    float l = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < nsplit; ++s) {
        const size_t slot = static_cast<size_t>(pair) * nsplit + s;
        const float w = exp2_for<T>(ws_ml[slot * 2] - mx);
        l += w * ws_ml[slot * 2 + 1];
        const float4 v = *reinterpret_cast<const float4*>(ws_o + slot * head_dim + e);
        o[0] += w * v.x; o[1] += w * v.y; o[2] += w * v.z; o[3] += w * v.w;
    }
    const float inv = 1.0f / l;
    T* dst = out + static_cast<size_t>(pair / n_heads) * out_stride + (pair % n_heads) * head_dim + e;
#pragma unroll
    for (int k = 0; k < 4; ++k) dst[k] = from_float<T>(o[k] * inv);
}

extern "C" {

// out[t, h * head_dim + e] from the states of `partial_out` (head_dim % 4 == 0).
int mllm_merge_attention_splits(const float* ws, int n_q, int n_heads, int head_dim, int nsplit, void* out,
                                int out_stride, int dtype, hipStream_t stream) {
    if (n_q <= 0) return 0;
    if (head_dim % 4 != 0 || nsplit < 1) return -1;
    const float* ws_o = ws;
    const float* ws_ml = ws + static_cast<size_t>(n_q) * n_heads * nsplit * head_dim;
    const int total4 = n_q * n_heads * (head_dim / 4);
    if (dtype == MLLM_F32)
        merge_splits_kernel<float><<<(total4 + 255) / 256, 256, 0, stream>>>(ws_o, ws_ml, nsplit, head_dim, n_heads,
                                                                             static_cast<float*>(out), out_stride, total4);
    else
        merge_splits_kernel<bf16_t><<<(total4 + 255) / 256, 256, 0, stream>>>(ws_o, ws_ml, nsplit, head_dim, n_heads,
                                                                              static_cast<bf16_t*>(out), out_stride, total4);
    MLLM_LAUNCH_CHECK();
    return 0;
}

// Number of floats of workspace (partial outputs and their max/sum) for n_q tokens.
long mllm_decode_attention_ws_floats(int n_q, int n_heads, int head_dim, int nsplit) {
    return static_cast<long>(n_q) * n_heads * nsplit * (head_dim + 2);
}

// Returns 0, a HIP error code, or -1 for sizes the kernel refuses: head_dim * element size / 16
// must be a power of two in [2, 64], page_size a power of two, and max_blocks at most 4096. `counters` holds n_q*n_heads ints that are zero before the
// first launch (the kernel leaves them zero). With `slots` (n_q rows of the page pools, < 0: none) the
// tokens' own keys/values are taken from columns k_col/v_col of q and written to the pages by this
// kernel; without, they must be in the pages already.
// partial_out != 0: nothing is written to `out`; the workspace holds, for pair = token * n_heads + head
// and split s, the unnormalised output at ws[(pair * nsplit + s) * head_dim ..] and (maximum in base 2,
// sum) at ws[n_q * n_heads * nsplit * head_dim + (pair * nsplit + s) * 2 ..]; a split without keys has
// sum 0 and a large negative maximum.
int mllm_decode_attention(const void* q, int q_stride, int q_col, const void* k_pages, const void* v_pages,
                          int kv_dim, const int* block_tables, int max_blocks, const int* token_seq,
                          const int* positions, int n_q, int n_heads, int n_kv_heads, int head_dim,
                          int page_size, float scale, int window, int nsplit, int waves, void* out,
                          int out_stride, float* ws, int* counters, int k_col, int v_col, const int* slots,
                          int partial_out, int dtype, hipStream_t stream) {
    if (n_q <= 0) return 0;
    const int esz = dtype == MLLM_F32 ? 4 : 2;
    const int lpk = head_dim * esz / 16;
    if (head_dim * esz % 16 != 0 || n_heads % n_kv_heads != 0 || nsplit < 1 || nsplit > 65535 ||
        waves < 1 || waves > DEC_MAX_WAVES) return -1;
    if (page_size < 1 || (page_size & (page_size - 1)) != 0 || max_blocks > DEC_TABLE_LDS) return -1;
    dim3 grid(n_q * n_heads, nsplit);
    float* ws_o = ws;
    float* ws_ml = ws + static_cast<size_t>(n_q) * n_heads * nsplit * head_dim;
    const float sl2 = scale * 1.44269504088896340736f;
    int rc;
    if (dtype == MLLM_F32)
        rc = launch_decode<float>(lpk, grid, waves, stream, (const float*)q, q_stride, q_col, (const float*)k_pages,
                                  (const float*)v_pages, kv_dim, block_tables, max_blocks, token_seq, positions,
                                  n_heads, n_kv_heads, page_size, sl2, window, nsplit, (float*)out, out_stride,
                                  ws_o, ws_ml, counters, (float*)k_pages, (float*)v_pages, k_col, v_col, slots, partial_out);
    else
        rc = launch_decode<bf16_t>(lpk, grid, waves, stream, (const bf16_t*)q, q_stride, q_col, (const bf16_t*)k_pages,
                                   (const bf16_t*)v_pages, kv_dim, block_tables, max_blocks, token_seq, positions,
                                   n_heads, n_kv_heads, page_size, sl2, window, nsplit, (bf16_t*)out, out_stride,
                                   ws_o, ws_ml, counters, (bf16_t*)k_pages, (bf16_t*)v_pages, k_col, v_col, slots, partial_out);
    if (rc != 0) return rc;
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

// Prefill attention on the MFMA units of gfx950, bf16 with fp32 softmax: causal (optionally
// windowed) attention of a step's query rows over the paged cache. A workgroup takes 64
// consecutive queries of one sequence and one head; its four wavefronts take 16 queries each
// and walk the keys in tiles of 128, which are gathered through the block table into LDS (keys
// row-major, values transposed), so prompt portions that start anywhere read what earlier steps
// left in the pages. With eight wavefronts (head sizes 64 and 128) two wavefronts share 16 queries and
// take one half of every key tile each; their states are merged through LDS at the end. A launch lasts as
// long as its longest workgroup (the last 64 queries of the longest prompt, one key tile after the
// other), and halving a wavefront's share of a tile nearly halves that.
//
// Everything is computed transposed so that a lane owns ONE query:
//   S^T = K Q^T   (A = 16 keys x 32 dims from LDS, B = the lane's query fragment, held in registers)
//   O^T = V^T P^T (A = 16 dims x 32 keys from the transposed values, B = P^T straight from the S^T
//                  accumulators: the MFMA's k index may be permuted freely as long as both operands
//                  agree, so no shuffle or LDS round trip is needed)
// The running maximum and sum are then scalars per lane, merged over the four lane groups with two
// DPP steps. Recurrence: /root/reference/src/kernels/prefill/flashattention.cu:129-178, in base 2;
// the reference reads its keys from the step's own qkv buffer (:99-111) and so cannot continue a
// prompt from the cache.
#include "common.h"

#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define PF_BM 64
#define PF_BN 128
#define PF_TABLE_LDS 2048   // most block-table entries of a sequence (the table is staged in LDS)
#define PF_VT_STRIDE (PF_BN + 12)   // elements per transposed value row: 70 words, which spreads both the staging writes
                                    // (rows 8 apart) and the fragment reads (16 neighbouring rows, 4 word pairs each)
                                    // evenly over the banks (measured against 65, 66 and 68 words: 3 to 8 % of the kernel)

union Frag8 {
    bf16x8 v;
    uint4 q;
    uint32_t w[4];
    uint16_t h[8];
};

// (At most 2 wavefronts per SIMD: the compiler may then use 256 registers, and keeps both
// prefetched tiles in registers instead of private memory.)
template <int DH, int NW>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(1, (DH >= 128 && NW == 4) ? 1 : 2)))
prefill_attention_kernel(const bf16_t* __restrict__ q, int q_stride, int q_col,
                         const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages, int kv_dim,
                         const int* __restrict__ block_tables, int max_blocks,
                         const int* __restrict__ cu_q, const int* __restrict__ ctx_len, int n_seqs,
                         int n_heads, int n_kv_heads, int page_size, float scale_log2e, int window,
                         bf16_t* __restrict__ out, int out_stride) {
    constexpr int KS = DH / 32;            // k steps of S^T
    constexpr int DT = DH / 16;            // 16-dim tiles of O^T
    constexpr int KSTRIDE = DH + 8;
    constexpr int NTH = NW * 64;           // threads
    constexpr int KH = NW / 4;             // wavefronts per 16 queries: each takes 1/KH of a key tile
    constexpr int NT_PER = PF_BN / 16 / KH;      // 16-key groups of a tile per wavefront
    constexpr int SL_PER = PF_BN / 32 / KH;      // 32-key slabs of a tile per wavefront
    static_assert(NW == 4 || NW == 8, "one or two wavefronts per 16 queries");
    // two buffers of keys and of values: a tile is staged while the one before it is multiplied
    __shared__ __attribute__((aligned(16))) bf16_t Ks2[2][PF_BN * KSTRIDE];
    __shared__ __attribute__((aligned(16))) bf16_t Vt2[2][DH * PF_VT_STRIDE];
    extern __shared__ int sm_table[];          // the sequence's block table (max_blocks entries)

    // Which sequence and which of its 64-query tiles this workgroup has. Heads vary fastest and the
    // tiles are handed out last-first: a causal tile's work grows with its position, so the long
    // ones start in the first wave of workgroups and the short ones fill the tail.
    int tile = gridDim.y - 1 - blockIdx.y, b = 0, q_begin = 0, q_len = 0;
    for (; b < n_seqs; ++b) {
        q_begin = cu_q[b];
        q_len = cu_q[b + 1] - q_begin;
        const int nt = (q_len + PF_BM - 1) / PF_BM;
        if (tile < nt) break;
        tile -= nt;
    }
    if (b >= n_seqs) return;               // surplus workgroup; the whole workgroup leaves

    const int h = blockIdx.x, hk = h / (n_heads / n_kv_heads);
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64) % 4;      // which 16 queries
    const int kh = __builtin_amdgcn_readfirstlane(tid / 64) / 4;        // which part of every key tile
    const int G = lane / 16, c16 = lane % 16;
    const int start = ctx_len[b] - q_len;                 // position of the step's first query
    const int q0 = tile * PF_BM;
    const int qi = q0 + wave * 16 + c16;                  // this lane's query within the step's rows
    const bool q_ok = qi < q_len;
    const int p = start + qi;                             // its position
    const int p_first = start + q0;
    const int p_last = start + min(q0 + PF_BM, q_len) - 1;
    const int k_lo = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    // The sequence's block table goes to LDS first: the gathers below then depend on an LDS read,
    // not on a global load that would have to be waited for in front of every key load.
    // (The host passes page sizes that are powers of two and tables of at most PF_TABLE_LDS blocks.)
    const int* gtable = block_tables + static_cast<size_t>(b) * max_blocks;
    const int shift = __ffs(page_size) - 1;
    const int n_blocks_needed = (p_last >> shift) + 1;
    for (int i = tid; i < n_blocks_needed; i += NTH) sm_table[i] = gtable[i];
    __syncthreads();
    auto page_row = [&](int j) -> size_t {
        return (static_cast<size_t>(sm_table[j >> shift]) << shift) + (j & (page_size - 1));
    };

    Frag8 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)      // a lane beyond the last query takes that query again; its scores are masked
        qf[ks].q = *reinterpret_cast<const uint4*>(q + static_cast<size_t>(q_begin + min(qi, q_len - 1)) * q_stride +
                                                   q_col + h * DH + 32 * ks + 8 * G);

    float m = -INFINITY, l = 0.f;
    f32x4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    const size_t kv_col = static_cast<size_t>(hk) * DH;

    // Tiles are fetched into registers ahead of their use, so the gather of the next keys and
    // values is in flight while the matrix cores work on the current ones. Every load of a fetch
    // is issued unconditionally, from a key clamped into [k_lo, p_last] (always a held page): a
    // load under a condition would make the compiler wait for all loads in flight. Keys outside
    // that range are masked in the scores, so what was loaded in their place never counts.
    // A thread takes KPT neighbouring keys (one group, inside one page) and 8 dims of them, keys
    // and values alike: one block-table lookup and one address per tile, the rest are constant
    // steps from it.
    constexpr int CH = DH / 8;                               // 16-byte chunks per row
    constexpr int KPT = PF_BN * CH / NTH;                    // keys per thread: 2, 4, 8 for head sizes 32, 64, 128 (half with 8 wavefronts)
    static_assert(KPT * NTH == PF_BN * CH && (KPT & (KPT - 1)) == 0 && KPT >= 2, "whole key groups per thread, keys in pairs");
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    u32x4 ak[KPT], av[KPT];      // register set a: tiles of even order, in flight from memory
    u32x4 bk[KPT], bv[KPT];      // register set b: tiles of odd order
    const int ch = tid % CH, grp = tid / CH;
    const int g_lo = k_lo & ~(KPT - 1), g_hi = p_last & ~(KPT - 1);      // first keys of the groups that hold k_lo and p_last
    auto fetch = [&](u32x4 (&rk)[KPT], u32x4 (&rv)[KPT], int kt) {
        const int g0 = min(max(kt * PF_BN + grp * KPT, g_lo), g_hi);
        const size_t base = page_row(g0) * kv_dim + kv_col + 8 * ch;
#pragma unroll
        for (int u = 0; u < KPT; ++u) {
            const int off = (min(max(g0 + u, k_lo), p_last) - g0) * kv_dim;     // stays inside the group
            rk[u] = *reinterpret_cast<const u32x4*>(k_pages + base + off);
            rv[u] = *reinterpret_cast<const u32x4*>(v_pages + base + off);
        }
    };
    auto stage = [&](const u32x4 (&rk)[KPT], const u32x4 (&rv)[KPT], int buf) {
        // keys row-major; values transposed: dim i of the thread's KPT keys becomes KPT/2 neighbouring words
        bf16_t* Ks = Ks2[buf];
        bf16_t* Vt = Vt2[buf];
#pragma unroll
        for (int u = 0; u < KPT; ++u)
            *reinterpret_cast<u32x4*>(Ks + (grp * KPT + u) * KSTRIDE + 8 * ch) = rk[u];
        Frag8 v[KPT];
#pragma unroll
        for (int u = 0; u < KPT; ++u) v[u].v = __builtin_bit_cast(bf16x8, rv[u]);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            uint32_t w[KPT / 2];
#pragma unroll
            for (int u = 0; u < KPT; u += 2)
                w[u / 2] = static_cast<uint32_t>(v[u].h[i]) | (static_cast<uint32_t>(v[u + 1].h[i]) << 16);
            uint32_t* dst = reinterpret_cast<uint32_t*>(Vt + (8 * ch + i) * PF_VT_STRIDE + grp * KPT);
#pragma unroll
            for (int u = 0; u < KPT / 2; ++u) dst[u] = w[u];
        }
    };

    // Positions of this wavefront's first and last query: a key tile that every one of them sees
    // in full needs no mask.
    const int pw_min = start + q0 + wave * 16, pw_max = pw_min + 15;
    auto compute = [&](int kt, int buf, auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const int j_base = kt * PF_BN;
        const bf16_t* Ks = Ks2[buf];
        const bf16_t* Vt = Vt2[buf];
        // S^T: s[nt][r] is the score of key j_base + 16*(nt0+nt) + 4*G + r with this lane's query
        const int nt0 = kh * NT_PER;
        float s[NT_PER][4];
        float tile_max = -INFINITY;
#pragma unroll
        for (int nt = 0; nt < NT_PER; ++nt) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8 a = *reinterpret_cast<const bf16x8*>(Ks + (16 * (nt0 + nt) + c16) * KSTRIDE + 32 * ks + 8 * G);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[ks].v, acc, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                s[nt][r] = acc[r];                   // raw dot product; the scale is applied with the exponent
                if (MASKED) {
                    const int j = j_base + 16 * (nt0 + nt) + 4 * G + r;
                    const bool seen = q_ok && j <= p && (window <= 0 || j > p - window);
                    if (!seen) s[nt][r] = -INFINITY;
                }
                tile_max = fmaxf(tile_max, s[nt][r]);
            }
        }
        // the four lane groups of a query agree on the maximum
        tile_max = rows_max(tile_max);
        const float m_new = fmaxf(m, tile_max * scale_log2e);        // the scale is positive
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;      // nothing seen yet: all weights are 0
        const float alpha = fast_exp2(m - m_use);
        m = m_new;
        float psum = 0.f;
#pragma unroll
        for (int nt = 0; nt < NT_PER; ++nt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                s[nt][r] = fast_exp2(fmaf(s[nt][r], scale_log2e, -m_use));
                psum += s[nt][r];
            }
        l = l * alpha + psum;                 // this lane's share of the sum; merged over groups at the end
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[dt][r] *= alpha;

        // O^T += V^T P^T over slabs of 32 keys. k slot i of lane group G stands for key
        // 32*slab + 4*G + i (i < 4) or 32*slab + 16 + 4*G + i - 4 (i >= 4) in both operands.
#pragma unroll
        for (int sl = 0; sl < SL_PER; ++sl) {
            const int slab = kh * SL_PER + sl;           // its place in the tile's transposed values
            Frag8 pf;
            pf.w[0] = pack_bf16x2(s[2 * sl][0], s[2 * sl][1]);
            pf.w[1] = pack_bf16x2(s[2 * sl][2], s[2 * sl][3]);
            pf.w[2] = pack_bf16x2(s[2 * sl + 1][0], s[2 * sl + 1][1]);
            pf.w[3] = pack_bf16x2(s[2 * sl + 1][2], s[2 * sl + 1][3]);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const uint32_t* vrow = reinterpret_cast<const uint32_t*>(Vt + (16 * dt + c16) * PF_VT_STRIDE);
                Frag8 vf;
                vf.w[0] = vrow[16 * slab + 2 * G];
                vf.w[1] = vrow[16 * slab + 2 * G + 1];
                vf.w[2] = vrow[16 * slab + 8 + 2 * G];
                vf.w[3] = vrow[16 * slab + 8 + 2 * G + 1];
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, o[dt], 0, 0, 0);
            }
        }
    };

    auto run_tile = [&](int kt, int buf) {
        const int j_base = kt * PF_BN;
        const bool full = j_base + PF_BN - 1 <= pw_min && (window <= 0 || j_base > pw_max - window);
        if (full) compute(kt, buf, std::false_type{}); else compute(kt, buf, std::true_type{});
    };

    // Tile t is multiplied from LDS buffer t % 2 while tile t+1 is written to the other buffer: one barrier
    // per tile. The loop body has no branch around a load; past the last tile the fetches repeat clamped
    // keys, which are staged and never multiplied.
    const int kt_first = k_lo / PF_BN, kt_last = p_last / PF_BN;
    if constexpr (NW == 8) {
        // Two register sets, every tile requested two tiles ahead of its staging: with half a tile's
        // arithmetic per wavefront, one tile ahead is not enough and the loop runs at the latency of the
        // gather (measured).
        fetch(ak, av, kt_first);
        __builtin_amdgcn_sched_barrier(0);     // set a's loads stay the older ones, as on every later iteration
        fetch(bk, bv, kt_first + 1);
        stage(ak, av, 0);
        fetch(ak, av, kt_first + 2);
        lds_barrier();
        for (int kt = kt_first; kt <= kt_last; kt += 2) {
            stage(bk, bv, 1);                  // (its last readers passed the barrier that ended the tile before)
            fetch(bk, bv, kt + 3);
            run_tile(kt, 0);
            lds_barrier();
            stage(ak, av, 0);
            fetch(ak, av, kt + 4);
            if (kt + 1 <= kt_last) run_tile(kt + 1, 1);
            lds_barrier();
        }
    } else {
        // One register set, requested one tile ahead: a whole tile's arithmetic covers the gather, and the
        // registers saved keep more of the softmax's values out of the way (measured: 28.8 against 31.0 us
        // at 25 heads).
        fetch(ak, av, kt_first);
        stage(ak, av, 0);
        fetch(ak, av, kt_first + 1);
        lds_barrier();
        for (int kt = kt_first; kt <= kt_last; ++kt) {
            const int buf = (kt - kt_first) & 1;
            stage(ak, av, buf ^ 1);
            fetch(ak, av, kt + 2);
            run_tile(kt, buf);
            lds_barrier();
        }
    }
    if constexpr (KH == 2) {
        // The two wavefronts of a query group merge their states: the second leaves its maximum, its
        // share of the sum and its outputs in LDS (the tiles are done with), the first adds them.
        constexpr int STATE = 2 + 4 * DT;
        static_assert(sizeof(Ks2) >= 4 * 64 * STATE * sizeof(float), "the states fit the key buffers");
        float* state = reinterpret_cast<float*>(&Ks2[0][0]) + (wave * 64 + lane) * STATE;
        if (kh == 1) {
            state[0] = m;
            state[1] = l;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) state[2 + 4 * dt + r] = o[dt][r];
        }
        lds_barrier();
        if (kh == 1) return;
        const float m1 = state[0];
        const float m_new = fmaxf(m, m1);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float a0 = fast_exp2(m - m_use), a1 = fast_exp2(m1 - m_use);
        l = l * a0 + state[1] * a1;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[dt][r] = o[dt][r] * a0 + state[2 + 4 * dt + r] * a1;
    }
    l = rows_sum(l);
    if (!q_ok) return;
    const float inv = 1.0f / l;
    // o[dt][r] is dimension 16*dt + 4*G + r of this lane's query
    bf16_t* orow = out + static_cast<size_t>(q_begin + qi) * out_stride + h * DH;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        uint2 pk;
        pk.x = pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv);
        pk.y = pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv);
        *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * G) = pk;
    }
}

extern "C" {

// n_tiles_upper: an upper bound of the number of 64-query tiles, sum over sequences of
// ceil(q_len / 64) (e.g. n_tokens / 64 + n_seqs); surplus workgroups leave at once.
// Returns 0, a HIP error code, or -1 when the head size is not 32, 64 or 128, the page size is no
// power of two or smaller than head_dim / 16 (a thread's group of keys must lie in one page), or a
// block table has more than PF_TABLE_LDS entries.
int mllm_prefill_attention_bf16(const void* q, int q_stride, int q_col, const void* k_pages, const void* v_pages,
                                int kv_dim, const int* block_tables, int max_blocks, const int* cu_q,
                                const int* ctx_len, int n_seqs, int n_tiles_upper, int n_heads, int n_kv_heads,
                                int head_dim, int page_size, float scale, int window, void* out, int out_stride,
                                hipStream_t stream) {
    if (n_seqs <= 0 || n_tiles_upper <= 0) return 0;
    if (n_heads % n_kv_heads != 0 || n_tiles_upper > 65535) return -1;
    if ((page_size & (page_size - 1)) != 0 || page_size < head_dim / 16 || max_blocks > PF_TABLE_LDS) return -1;
    const dim3 grid(n_heads, n_tiles_upper);
    const size_t table_bytes = static_cast<size_t>(max_blocks) * sizeof(int);
    const float sl2 = scale * 1.44269504088896340736f;
#define PF_CASE(D, W, KEY)                                                                                  \
    case KEY: {                                                                                               \
        static bool lds_allowed = false;      /* static and dynamic LDS together pass 64 KB: asked for once */ \
        if (!lds_allowed) {                                                                                 \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_attention_kernel<D, W>), \
                                               hipFuncAttributeMaxDynamicSharedMemorySize,                  \
                                               PF_TABLE_LDS * static_cast<int>(sizeof(int)));               \
            if (e != hipSuccess) return static_cast<int>(e);                                                \
            lds_allowed = true;                                                                             \
        }                                                                                                   \
        prefill_attention_kernel<D, W><<<grid, W * 64, table_bytes, stream>>>(                                            \
            (const bf16_t*)q, q_stride, q_col, (const bf16_t*)k_pages, (const bf16_t*)v_pages, kv_dim,      \
            block_tables, max_blocks, cu_q, ctx_len, n_seqs, n_heads, n_kv_heads, page_size, sl2, window,   \
            (bf16_t*)out, out_stride);                                                                      \
        break;                                                                                              \
    }
    // Eight wavefronts (two per 16 queries, half a key tile each) shorten the longest workgroup's chain of
    // key tiles, which is what a launch of few workgroups lasts (2 x 1,024 tokens, 12 heads of 64: 384
    // workgroups, 20.6 -> 18.2 us); they also take a compute unit each, so launches of many workgroups, which
    // the units work off in rounds, keep four (25 heads, 800 workgroups: 28.5 us against 37.5). At head size
    // 128 a workgroup has a unit to itself either way.
    const bool eight = head_dim == 128 || (head_dim == 64 && static_cast<long>(n_heads) * n_tiles_upper <= 512);
    switch (head_dim * 2 + (eight ? 1 : 0)) {
        PF_CASE(32, 4, 64) PF_CASE(64, 4, 128) PF_CASE(64, 8, 129) PF_CASE(128, 8, 257)
        default: return -1;
    }
#undef PF_CASE
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

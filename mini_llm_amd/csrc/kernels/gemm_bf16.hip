// bf16 matrix products on the MFMA units of gfx950, fp32 accumulation:
//   C[M,N] = A[M,K] * W[N,K]^T + bias, with the epilogues of common.h fused
// (bias, GELU, residual add into the fp32 stream, fp32 store for logits).
// Both operands are k-contiguous, so each lane feeds v_mfma_f32_32x32x16_bf16 with one
// 16-byte LDS read per operand. Tiles are staged through LDS with the next tile's
// global loads in flight during the current tile's MFMAs.
//
// It stands where the reference has its tiled SGEMM with fused store path
// (/root/reference/src/kernels/gemm.cu:394-580, epilogue :534-564).
// Requires K % 8 == 0 and 16-byte aligned rows; any M and N.
#include "common.h"

#include <algorithm>
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define N_XCD 8       // accelerator dies of an MI355X, each with its own L2

// ---------------------------------------------------------------------------------------------
// Many rows (prefill): WM x WN wavefronts, each TM x TN MFMA tiles of 32x32. LDS is double
// buffered (one barrier per k tile), global loads run DEPTH-1 tiles ahead in rotating register
// sets, per-thread pointers only advance, and a K that is a multiple of the k tile takes a k loop
// without checks, chosen at compile time (rows and columns beyond the matrices cost nothing there). Within a tile the memory instructions are spread between
// the MFMA groups of its k steps, so that the matrix units work while they queue. For a long K
// two such groups of wavefronts share a workgroup's tile, each on half of a twice as wide k tile,
// and add their sums in LDS. The weight
// fragment is the MFMA's A operand, so a lane's accumulator registers hold 4 consecutive columns
// of one output row; the epilogue turns that, through LDS, into stores of whole rows.
// ---------------------------------------------------------------------------------------------
// Optional second destination of a plain bf16 store: columns [q_cols, q_cols + kv_dim) of output row
// m also go to row slots[m] of the key pages and the next kv_dim columns to the value pages (the
// fused QKV product writes a step's keys and values where attention reads them;
// /root/reference/src/kernels/prefill/append_kv.cu:28-46 is a kernel of its own). slots == nullptr: off.
struct KvScatter {
    const int* slots;
    bf16_t* k_pages;
    bf16_t* v_pages;
    int q_cols, kv_dim;
};

template <int MODE>
__device__ __forceinline__ void store4(void* C, size_t idx, const float (&v)[4], bool vec, int n_left) {
    // v: 4 consecutive columns of one row, bias already added; n_left: columns that exist (1..4)
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
        o[e] = MODE == EPI_GELU_TANH ? gelu_tanh(v[e]) : MODE == EPI_GELU_ERF ? gelu_erf(v[e]) : v[e];
    if (MODE == EPI_ADD_RESIDUAL || MODE == EPI_STORE_F32) {
        float* c = static_cast<float*>(C) + idx;
        if (vec && n_left >= 4) {
            float4 r = make_float4(o[0], o[1], o[2], o[3]);
            if (MODE == EPI_ADD_RESIDUAL) {
                const float4 old = *reinterpret_cast<const float4*>(c);
                r.x += old.x; r.y += old.y; r.z += old.z; r.w += old.w;
            }
            *reinterpret_cast<float4*>(c) = r;
        } else {
            for (int e = 0; e < n_left; ++e) c[e] = (MODE == EPI_ADD_RESIDUAL ? c[e] : 0.f) + o[e];
        }
    } else {
        bf16_t* c = static_cast<bf16_t*>(C) + idx;
        if (vec && n_left >= 4) {
            uint2 pk;
            pk.x = pack_bf16x2(o[0], o[1]);
            pk.y = pack_bf16x2(o[2], o[3]);
            *reinterpret_cast<uint2*>(c) = pk;
        } else {
            for (int e = 0; e < n_left; ++e) c[e] = float_to_bf16(o[e]);
        }
    }
}

template <int WM, int WN, int TM, int TN, int BKP, int DEPTH, bool EDGE, int MODE, int KG = 1>
__global__ void __launch_bounds__(WM * WN * KG * 64)
gemm_bf16_mfma(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
               const float* __restrict__ bias, void* __restrict__ C, int ldc, int M, int N, int K,
               int tiles_m, int tiles_n, int xm, int xn, KvScatter kv) {
    // KG groups of WM x WN wavefronts share the tile: a k tile is KG * BKP wide and group g multiplies
    // its g-th part, so a barrier interval covers KG times the depth; the groups' sums meet in LDS.
    constexpr int NT = WM * WN * KG * 64;
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    constexpr int BKT = BKP * KG;
    constexpr int STRIDE = BKT + 8;
    constexpr int CPR = BKT / 8;                      // 16-byte chunks per row
    constexpr int KS = BKP / 16;                      // MFMA k steps per tile
    constexpr int A_CH = (BM * CPR + NT - 1) / NT, W_CH = (BN * CPR + NT - 1) / NT, N_LOADS = A_CH + W_CH;
    constexpr int EPI_STRIDE = 36;                    // floats per row of a 32x32 sub-tile in the epilogue
    static_assert(KS % 2 == 0 && DEPTH >= 3, "the k loop alternates two fragment sets and three register sets");
    constexpr int EPI_BASE = KG > 1 ? BM * BN : 0;    // floats: behind the groups' sums
    static_assert(2 * (BM + BN) * STRIDE * 2 >= (EPI_BASE + WM * WN * 32 * EPI_STRIDE) * 4, "the tiles' LDS holds the epilogue's regions");
    // one array: two buffers of A rows, two of W rows; the epilogue reuses it, a region per wavefront
    __shared__ __attribute__((aligned(16))) bf16_t smem[2 * (BM + BN) * STRIDE];
    __shared__ __attribute__((aligned(16))) float bias_s[BN];
    bf16_t (*As)[BM * STRIDE] = reinterpret_cast<bf16_t (*)[BM * STRIDE]>(smem);
    bf16_t (*Ws)[BN * STRIDE] = reinterpret_cast<bf16_t (*)[BN * STRIDE]>(smem + 2 * BM * STRIDE);

    const int tid = threadIdx.x, lane = tid % 64;
    const int kg = tid / 64 / (WM * WN), wave = tid / 64 % (WM * WN);      // k group; wavefront within it
    const int wm = wave / WN, wn = wave % WN;
    // Workgroups are handed to the 8 XCDs round-robin and every XCD has an L2 of its own, so the
    // tiles of one XCD (workgroup id % 8) form one compact rectangle of the output: the rows of A
    // and W it needs then fit in its L2 instead of every XCD streaming both matrices.
    const int xcd = blockIdx.x % N_XCD, local = blockIdx.x / N_XCD;
    const int rect_m = (tiles_m + xm - 1) / xm, rect_n = (tiles_n + xn - 1) / xn;
    const int tm = (xcd / xn) * rect_m + local / rect_n, tn = (xcd % xn) * rect_n + local % rect_n;
    if (local >= rect_m * rect_n || tm >= tiles_m || tn >= tiles_n) return;      // padding of the grid
    const int m0 = tm * BM, n0 = tn * BN;
    if (bias != nullptr)         // read again in the epilogue, after the k loop's barriers
        for (int c = tid; c < BN; c += NT) bias_s[c] = n0 + c < N ? bias[n0 + c] : 0.f;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // per-thread chunk pointers (row fixed, k advances by BKP per tile) and LDS offsets
    const bf16_t* pa[A_CH];
    const bf16_t* pw[W_CH];
    int la[A_CH], lw[W_CH];
    bool va[A_CH], vw[W_CH];
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
        const int c = tid + i * NT, row = c / CPR, kc = c % CPR;
        va[i] = (BM * CPR % NT == 0 || c < BM * CPR) && m0 + row < M;
        pa[i] = A + static_cast<size_t>(va[i] ? m0 + row : 0) * lda + kc * 8;
        la[i] = row * STRIDE + kc * 8;
    }
#pragma unroll
    for (int i = 0; i < W_CH; ++i) {
        const int c = tid + i * NT, row = c / CPR, kc = c % CPR;
        vw[i] = (BN * CPR % NT == 0 || c < BN * CPR) && n0 + row < N;
        pw[i] = W + static_cast<size_t>(vw[i] ? n0 + row : 0) * ldw + kc * 8;
        lw[i] = row * STRIDE + kc * 8;
    }
    struct TileRegs {
        uint4 ra[A_CH], rw[W_CH];
    };
    TileRegs regs[DEPTH];
    // (Rows of A or W beyond the matrix: the pointer stays on a row that exists, and what is computed
    // from it lands in output rows or columns that are never stored. Only a K that is no multiple of
    // the k tile needs care in the loop, EDGE: addresses clamped into the row, and zeros staged for
    // what lies beyond K.)
    // A tile's loads and its LDS writes are cut into KS portions (portion `part`, or all of them
    // with part < 0), so that they can be issued between the MFMA groups of the tile in work.
    // Every thread issues every load, with the address clamped into the matrix: the number of loads
    // in flight is then the same on every path through the loop, and only so does the compiler wait
    // for exactly the registers that are staged next while later loads stay in flight. What lies
    // beyond K is zeroed when the tile is staged.
    auto fetch = [&](TileRegs& t, int k0, int part) {
#pragma unroll
        for (int i = 0; i < A_CH; ++i) {
            if (part >= 0 && i * KS / N_LOADS != part) continue;
            const int kc8 = (tid + i * NT) % CPR * 8;
            const int k = EDGE ? min(k0 + kc8, K - 8) - kc8 : k0;
            t.ra[i] = *reinterpret_cast<const uint4*>(pa[i] + k);
        }
#pragma unroll
        for (int i = 0; i < W_CH; ++i) {
            if (part >= 0 && (A_CH + i) * KS / N_LOADS != part) continue;
            const int kc8 = (tid + i * NT) % CPR * 8;
            const int k = EDGE ? min(k0 + kc8, K - 8) - kc8 : k0;
            t.rw[i] = *reinterpret_cast<const uint4*>(pw[i] + k);
        }
    };
    auto stage = [&](const TileRegs& t, int buf, int k0, int part) {
#pragma unroll
        for (int i = 0; i < A_CH; ++i) {
            if (part >= 0 && i * KS / N_LOADS != part) continue;
            const int kc8 = (tid + i * NT) % CPR * 8;
            const bool ok = !EDGE || k0 + kc8 < K;
            if (BM * CPR % NT == 0 || tid + i * NT < BM * CPR)
                *reinterpret_cast<uint4*>(&As[buf][la[i]]) = ok ? t.ra[i] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < W_CH; ++i) {
            if (part >= 0 && (A_CH + i) * KS / N_LOADS != part) continue;
            const int kc8 = (tid + i * NT) % CPR * 8;
            const bool ok = !EDGE || k0 + kc8 < K;
            if (BN * CPR % NT == 0 || tid + i * NT < BN * CPR)
                *reinterpret_cast<uint4*>(&Ws[buf][lw[i]]) = ok ? t.rw[i] : make_uint4(0, 0, 0, 0);
        }
    };
    // two sets of MFMA operands: the fragments of k step ks+1 are read while step ks multiplies
    const int a_off = (wm * TM * 32 + lane % 32) * STRIDE + kg * BKP + 8 * (lane / 32);
    const int w_off = (wn * TN * 32 + lane % 32) * STRIDE + kg * BKP + 8 * (lane / 32);
    bf16x8 fa[2][TM], fb[2][TN];
    auto read_frags = [&](int buf, int ks, int set) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
            fa[set][i] = *reinterpret_cast<const bf16x8*>(&As[buf][a_off + i * 32 * STRIDE + ks * 16]);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            fb[set][j] = *reinterpret_cast<const bf16x8*>(&Ws[buf][w_off + j * 32 * STRIDE + ks * 16]);
    };
    auto mma = [&](int set) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[set][j], fa[set][i], acc[i][j], 0, 0, 0);
    };

    const int nk = (K + BKT - 1) / BKT;
    // tiles 0 .. DEPTH-2 are requested (past the last tile: the last one again, never used);
    // tile 0 is staged
#pragma unroll
    for (int d = 0; d < DEPTH - 1; ++d) fetch(regs[d], min(d, nk - 1) * BKT, -1);
    stage(regs[0], 0, 0, -1);
    lds_barrier();
    read_frags(0, 0, 0);
    // Whole groups of DEPTH tiles run without a branch in the body (a load or a use of it under a
    // condition would be moved or waited for conservatively); the last nk % DEPTH tiles, which
    // fetch nothing any more, follow under conditions. In the body, tile t is in LDS buffer t%2
    // and every k step issues, in this order: its share of the loads of tile t+DEPTH-1, its share
    // of the LDS writes of tile t+1 (into the other buffer, whose last readers passed the barrier
    // that ended the previous iteration), the fragment reads of the next k step, its MFMAs. The
    // scheduling barriers keep that order: left alone, the compiler gathers the loads at the end
    // of the iteration and the writes at its start, and a wavefront then issues nothing else while
    // its memory instructions queue up.
    const int n_groups = nk / DEPTH, n_tail = nk % DEPTH;
    for (int g = 0; g < n_groups; ++g) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int t = g * DEPTH + d;
            const int k_fetch = min(t + DEPTH - 1, nk - 1) * BKT;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                fetch(regs[(d + DEPTH - 1) % DEPTH], k_fetch, ks);
                stage(regs[(d + 1) % DEPTH], (t + 1) & 1, (t + 1) * BKT, ks);
                if (ks + 1 < KS) read_frags(t & 1, ks + 1, (ks + 1) & 1);
                mma(ks & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            lds_barrier();
            read_frags((t + 1) & 1, 0, 0);
        }
    }
#pragma unroll
    for (int d = 0; d < DEPTH - 1; ++d) {
        const int t = n_groups * DEPTH + d;
        if (d < n_tail) {
            if (d + 1 < n_tail) stage(regs[(d + 1) % DEPTH], (t + 1) & 1, (t + 1) * BKT, -1);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if (ks + 1 < KS) read_frags(t & 1, ks + 1, (ks + 1) & 1);
                mma(ks & 1);
            }
            lds_barrier();
            if (d + 1 < n_tail) read_frags((t + 1) & 1, 0, 0);
        }
    }

    // With the weights as the A operand, register r of lane l holds output row l%32 and column
    // 8*(r/4) + 4*(l/32) + r%4 of a 32x32 sub-tile. Stored from there, one instruction would touch
    // 16 bytes in each of 32 rows. So each sub-tile goes through the wavefront's own region of LDS
    // (the tiles are done with theirs): written as the MFMA left it, read back with 8 lanes per row,
    // and a store instruction then covers 8 whole rows of the sub-tile.
    if constexpr (KG > 1) {
        // the other groups leave their sums in LDS, register by register, and go; group 0 adds them
        float4* sums = reinterpret_cast<float4*>(smem);
        if (kg > 0) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        sums[((wave * TM * TN + i * TN + j) * 4 + g) * 64 + lane] =
                            make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
        }
        lds_barrier();
        if (kg > 0) return;
        static_assert(KG == 2, "one other group's sums fit in front of the epilogue's regions");
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float4 t = sums[((wave * TM * TN + i * TN + j) * 4 + g) * 64 + lane];
                    acc[i][j][4 * g] += t.x; acc[i][j][4 * g + 1] += t.y; acc[i][j][4 * g + 2] += t.z; acc[i][j][4 * g + 3] += t.w;
                }
    }
    const bool vec = (ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0);
    float* epi = reinterpret_cast<float*>(smem) + EPI_BASE + wave * (32 * EPI_STRIDE);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            wave_lds_sync();          // the reads of the sub-tile before are done
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<float4*>(&epi[(lane % 32) * EPI_STRIDE + 8 * g + 4 * (lane / 32)]) =
                    make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
            wave_lds_sync();
            const int mb = m0 + (wm * TM + i) * 32, nb = n0 + (wn * TN + j) * 32;
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int r = it * 8 + lane / 8, c4 = (lane % 8) * 4;
                const int m = mb + r, n = nb + c4;
                if (m >= M || n >= N) continue;
                const int n_left = min(4, N - n);
                const float4 t = *reinterpret_cast<const float4*>(&epi[r * EPI_STRIDE + c4]);
                float v[4] = {t.x, t.y, t.z, t.w};
                if (bias != nullptr) {
                    const float4 b = *reinterpret_cast<const float4*>(&bias_s[nb - n0 + c4]);
                    v[0] += b.x; v[1] += b.y; v[2] += b.z; v[3] += b.w;
                }
                store4<MODE>(C, static_cast<size_t>(m) * ldc + n, v, vec, n_left);
                if (MODE == EPI_STORE && kv.slots != nullptr && n >= kv.q_cols) {
                    const int slot = kv.slots[m];
                    if (slot >= 0) {
                        // q_cols and kv_dim are multiples of 4: the four columns lie in one of the two parts
                        const int c = n - kv.q_cols;
                        bf16_t* dst = (c < kv.kv_dim ? kv.k_pages + c : kv.v_pages + (c - kv.kv_dim)) +
                                      static_cast<size_t>(slot) * kv.kv_dim;
                        if (n_left >= 4) {
                            uint2 pk;
                            pk.x = pack_bf16x2(v[0], v[1]);
                            pk.y = pack_bf16x2(v[2], v[3]);
                            *reinterpret_cast<uint2*>(dst) = pk;
                        } else {
                            for (int e = 0; e < n_left; ++e) dst[e] = float_to_bf16(v[e]);
                        }
                    }
                }
            }
        }
    }
}

template <int WM, int WN, int TM, int TN, int BKP, int DEPTH, int KG = 1>
static void launch_tiled(const bf16_t* a, int lda, const bf16_t* w, int ldw, const float* bias, void* C, int ldc,
                         int M, int N, int K, int mode, hipStream_t stream, KvScatter kv = KvScatter{}) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    // split of the output among the XCDs (xm x xn = 8) that keeps the A rows plus W rows of one XCD smallest
    int xm = 1, xn = N_XCD;
    double best = 1e300;
    for (int cand = 1; cand <= N_XCD; cand *= 2) {
        const int cm = cand, cn = N_XCD / cand;
        const double rows = static_cast<double>((tiles_m + cm - 1) / cm) * BM + static_cast<double>((tiles_n + cn - 1) / cn) * BN;
        if (rows < best) { best = rows; xm = cm; xn = cn; }
    }
    const int per_xcd = ((tiles_m + xm - 1) / xm) * ((tiles_n + xn - 1) / xn);
    const dim3 grid(per_xcd * N_XCD), block(WM * WN * KG * 64);
    const bool edge = K % (BKP * KG) != 0;      // rows and columns beyond the matrices need no other kernel, see EDGE
#define TILED(E, MD) gemm_bf16_mfma<WM, WN, TM, TN, BKP, DEPTH, E, MD, KG><<<grid, block, 0, stream>>>(a, lda, w, ldw, bias, C, ldc, M, N, K, tiles_m, tiles_n, xm, xn, kv)
#define TILED_MODE(MD) case MD: if (edge) TILED(true, MD); else TILED(false, MD); break;
    switch (mode) {
        TILED_MODE(EPI_STORE) TILED_MODE(EPI_GELU_TANH) TILED_MODE(EPI_GELU_ERF) TILED_MODE(EPI_ADD_RESIDUAL)
        default: if (edge) TILED(true, EPI_STORE_F32); else TILED(false, EPI_STORE_F32); break;
    }
#undef TILED_MODE
#undef TILED
}

// ---------------------------------------------------------------------------------------------
// Few rows (decode; up to 64 rows always, up to 256 while the workgroups stay few, see the
// dispatch). The product is bound by streaming W once, and how fast a compute
// unit streams depends on the shape of a wavefront's load: 8 consecutive lanes take one 128-byte
// line (8 weight rows x 1 line per load) at up to 90 GB/s per unit, but the MFMA operand layout
// (consecutive lanes = consecutive weight rows, 4 lines per 4 lanes) at under 40 (measured). So
// the loads use the first shape and the 16-byte pieces change lanes through a region of LDS
// private to the wavefront (2 KB per weight tile and k block, up to two k blocks at a time; no
// barrier: LDS serves a wavefront's requests in order), swizzled so that neither the writes nor
// the reads conflict. A workgroup owns 16 rows of the output (more
// rows: more workgroups per column range, placed on the same XCD so that the weights they share
// come from its L2).
//   SPLIT_K:  one workgroup per 16-column tile, its wavefronts split K (wavefront w takes the
//             64-element k blocks w, w+NW, ...) and their partial sums are added in LDS in a fixed
//             order: for the narrow products, where tiles alone are too few to fill the chip.
//             With k_parts > 1 several workgroups share a tile as well (blockIdx.y is the part):
//             each writes its sum to a workspace, and the last one to arrive, found through a
//             counter per tile, adds the parts in the order of their index and runs the
//             epilogue. For products whose tiles alone use a fraction of the compute units and
//             whose K is long (the second product of the feed-forward).
//   !SPLIT_K: one wavefront per tile over the whole of K (wide products such as the logits head).
// The activations come from global memory (A_GLOBAL: a few KB, shared by all workgroups, read
// from L2), are copied into LDS once per workgroup (A_STAGED: wide products), or are normalised
// from the fp32 stream into LDS first (A_NORMED): LayerNorm
// (/root/reference/src/kernels/layernorm.cu:32-49) fused into the product that follows it.
// A_MERGED: A is the output of decode attention that split every (token, head) pair's keys over
// several workgroups and left their states in a workspace (attention_decode.hip, partial_out): a lane
// that would load 8 elements of a row loads those elements of every split's unnormalised output and
// the splits' maxima and sums instead, and merges them in registers. The attention kernel then
// needs no pass that waits for its last workgroup, and more workgroups stream the keys.
// ---------------------------------------------------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));

enum { A_GLOBAL = 0, A_NORMED = 1, A_STAGED = 2, A_MERGED = 3 };
#define MERGE_MAX_SPLITS 4      // splits of a pair that the merging load takes (registers: 10 per split and load)

// The states of up to MERGE_MAX_SPLITS splits for 8 consecutive elements of one head of one token.
struct SplitStates {
    float2 ml[MERGE_MAX_SPLITS];          // maximum (base 2), sum
    float4 o[MERGE_MAX_SPLITS][2];        // 8 elements of the unnormalised output
};

template <int MT, int ASRC, bool SPLIT_K, int U, bool A_TWO = true, int NT = 1>
__global__ void __launch_bounds__(ASRC == A_NORMED ? 512 : (ASRC == A_GLOBAL || ASRC == A_MERGED ? 768 : 1024))
gemm_bf16_skinny(// the first 16 dwords arrive in registers with the wavefront: what the first loads need
                 const bf16_t* __restrict__ W, int ldw, int N, int K, int M, int col_blocks, int row_blocks,
                 int cols_per_wg, int k_parts, const void* __restrict__ Ain, int lda, int mode,
                 const float* __restrict__ bias,
                 // the rest is loaded by the kernel and needed later
                 void* __restrict__ C, int ldc, const float* __restrict__ gamma, const float* __restrict__ beta,
                 float eps, const int* __restrict__ rows, float* __restrict__ part_sums,
                 int* __restrict__ part_counters,
                 // A_MERGED: the attention splits' states (layout: attention_decode.hip), their number,
                 // heads per token and head size (K = heads x head size)
                 const float* __restrict__ split_o = nullptr, const float* __restrict__ split_ml = nullptr,
                 int n_splits = 1, int a_heads = 1, int a_head_dim = 8) {
    // NT > 1 (SPLIT_K, MT == 1): the workgroup owns cols_per_wg <= 16 NT columns, NT tiles that share
    // the rows of A, the last one possibly narrower: for products with more than 256 tiles, whose
    // columns are dealt out evenly to 256 workgroups (one per compute unit; a kernel of this size
    // keeps one workgroup per unit, so 400 one-tile workgroups would take two rounds).
    static_assert(NT == 1 || (MT == 1 && SPLIT_K), "column tiles per workgroup: split-K kernels of one row tile");
    constexpr int T = MT * NT;      // accumulators: row tiles (NT == 1) or column tiles (MT == 1)
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    __shared__ int sm_last;
    constexpr bool LN_FUSED = ASRC == A_NORMED;
    constexpr bool IN_LDS = ASRC == A_NORMED || ASRC == A_STAGED;
    constexpr bool A_REGS = !IN_LDS;      // the rows of A travel through registers and the wavefront's LDS region
    // The wavefront's index as a scalar: what depends on it alone (its k blocks, whether it has a
    // whole chunk, whether it owns outputs) then branches for real. Derived from threadIdx it would
    // count as divergent, both sides of every such condition would run one after the other under
    // masks, and loads pending from one side would be waited for on the other.
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
    const int nw = blockDim.x / 64;
    const int row16 = lane % 16, kq = lane / 16;
    // workgroup id -> (column block, row block): the row blocks of one column block have ids that
    // agree modulo 8, i.e. run on one XCD
    const int g = blockIdx.x;
    const int cb = (g / (N_XCD * row_blocks)) * N_XCD + g % N_XCD, rb = (g / N_XCD) % row_blocks;
    if (cb >= col_blocks) return;
    const int m_base = rb * 16 * MT;
    const int n0 = SPLIT_K ? cb * cols_per_wg : (cb * nw + wave) * 16;
    // K is dealt out in blocks of 64 elements, one 128-byte line of a weight row. In the MFMAs
    // lane group kq takes elements 16*kq .. 16*kq+15 of a block, the first 8 in one MFMA and the
    // rest in the next (the k index of an MFMA may be permuted as long as both operands agree).
    // (with k_parts workgroups on the tile, over all their wavefronts alike)
    const int part = SPLIT_K ? blockIdx.y : 0;
    const int k_first = SPLIT_K ? (part * nw + wave) * 64 : 0;      // first k block of this wavefront
    const int k_stride = SPLIT_K ? nw * k_parts * 64 : 64;         // distance between its k blocks
    const size_t red_bytes = SPLIT_K ? static_cast<size_t>(nw) * T * 256 * sizeof(float) : 0;
    // per wavefront: SB k blocks at a time change lanes through LDS, each NT weight tiles (+ the A block)
    constexpr int SB = (ASRC == A_STAGED || (A_REGS && NT > 1) || U < 4) ? 1 : 2;
    constexpr int STAGE_BYTES = SB * (NT * 2048 + (A_REGS ? 2048 : 0));
    float* red = reinterpret_cast<float*>(smem_raw);                       // [nw][T][256]
    bf16x8* stage_w = reinterpret_cast<bf16x8*>(smem_raw + red_bytes + static_cast<size_t>(wave) * STAGE_BYTES);
    bf16x8* stage_a = stage_w + SB * NT * 128;                             // (A_GLOBAL only)
    bf16_t* a_s = reinterpret_cast<bf16_t*>(smem_raw + red_bytes + static_cast<size_t>(nw) * STAGE_BYTES);   // [16*MT][K+8]
    const int a_stride = K + 8;
    // (fused norm only) the scale and shift vectors, loaded once per workgroup: [2][K] fp32
    float4* gb_s = reinterpret_cast<float4*>(a_s + static_cast<size_t>(16) * MT * a_stride);
    const int n = n0 + row16;
    const bool n_ok = n < N;
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    // Loads: lane -> (row lr = lane / 8 of 8, 16-byte piece lane % 8 of the row's 128-byte line);
    // two loads cover the tile's 16 rows. The piece a lane fetches is its slot number XORed with a
    // swizzle of the row (the row modulo 8, its lowest bit flipped for rows 8..15), so that slot s
    // of row r, written to LDS lane-linearly, holds piece s ^ swizzle(r): then the 16 lanes of an
    // operand read (rows 0..15, one piece number) fall on 16 different 16-byte bank groups.
    const int lr = lane / 8;
    const int piece[2] = {(lane % 8) ^ lr, (lane % 8) ^ lr ^ 1};
    // (columns beyond the workgroup's or the matrix's: the last valid one, never stored)
    const bf16_t* wrow[NT][2];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < 2; ++j)
            wrow[t][j] = W + static_cast<size_t>(min(n0 + min(16 * t + lr + 8 * j, cols_per_wg - 1), N - 1)) * ldw;
    // reads: this lane's MFMA row/column is row16; for MFMA step `half` it wants piece 2*kq + half
    const int rd_swz = row16 < 8 ? row16 : ((row16 - 8) ^ 1);

    f32x4 acc[T];
#pragma unroll
    for (int i = 0; i < T; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Split-K epilogue operands (thread tid < 256 owns output element tid of the 16x16 tile, in
    // accumulator order): requested now so that their latency hides behind the product.
    bool ep_ok[NT];
    size_t ep_idx[NT];
    float ep_bias[NT], ep_old[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) { ep_ok[t] = false; ep_idx[t] = 0; ep_bias[t] = 0.f; ep_old[t] = 0.f; }
    if (SPLIT_K && MT == 1 && wave < 4) {
        // (loads without a per-lane condition: outputs beyond M or N read the last row or column)
        const int m = m_base + 4 * (lane / 16) + wave;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int ct = 16 * t + lane % 16, nn = n0 + ct;
            ep_ok[t] = m < M && nn < N && ct < cols_per_wg;
            ep_idx[t] = static_cast<size_t>(min(m, M - 1)) * ldc + min(nn, N - 1);
            if (bias) ep_bias[t] = bias[min(nn, N - 1)];
            if (mode == EPI_ADD_RESIDUAL) ep_old[t] = static_cast<const float*>(C)[ep_idx[t]];
        }
    }

    // A wavefront takes its k blocks in chunks of H = U/2. All loads of a chunk are issued
    // together and without a condition inside (a load under a condition makes the compiler wait
    // for every load in flight); the conditions that decide whether a chunk is loaded at all are
    // uniform over the wavefront. No load goes to a line that another load may still have in
    // flight: loads that hit such a line queue up behind it in the vector cache. Two chunks
    // alternate so that one is in flight while the other is multiplied; the first is requested
    // before the norm or the copy of A, so that its latency overlaps them. Blocks left over
    // (fewer than H) follow one by one. Only the last block of K can be short: its lanes beyond K
    // load the row's last 16 bytes and their weight fragment is zeroed.
    constexpr int H = U / 2;
    static_assert(U % 2 == 0, "whole k blocks per chunk");
    const bf16_t* A = static_cast<const bf16_t*>(Ain);
    // A_GLOBAL: the rows of A travel like the weights (rows beyond M: the last one, never stored);
    // a workgroup with at most 8 rows needs one load per k block
    const bf16_t* arow[2] = {A, A};
    int arow_idx[2] = {0, 0};
    // (A_TWO false: the launcher knows that M <= 8, and the chunks keep half the registers for A)
    const bool a_two = A_TWO && M - m_base > 8;
    if (A_REGS) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            arow_idx[j] = min(m_base + lr + 8 * j, M - 1);
            arow[j] = A + static_cast<size_t>(arow_idx[j]) * lda;
        }
    }
    // A_MERGED: requests the splits' states for the 8 elements from k on of row `row` (all loads together;
    // splits beyond n_splits take the last one again and get no weight), and merges them later
    auto fetch_splits = [&](SplitStates& st, int row, int k) {
        const int h = k / a_head_dim, e = k - h * a_head_dim;
        const size_t pair = static_cast<size_t>(row) * a_heads + h;
#pragma unroll
        for (int sidx = 0; sidx < MERGE_MAX_SPLITS; ++sidx) {
            const size_t slot = pair * n_splits + min(sidx, n_splits - 1);
            st.ml[sidx] = *reinterpret_cast<const float2*>(split_ml + slot * 2);
            const float4* src = reinterpret_cast<const float4*>(split_o + slot * a_head_dim + e);
            st.o[sidx][0] = src[0];
            st.o[sidx][1] = src[1];
        }
    };
    auto merge_splits = [&](const SplitStates& st) -> bf16x8 {
        float mx = st.ml[0].x;
#pragma unroll
        for (int sidx = 1; sidx < MERGE_MAX_SPLITS; ++sidx) mx = fmaxf(mx, sidx < n_splits ? st.ml[sidx].x : mx);
        float l = 0.f, o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sidx = 0; sidx < MERGE_MAX_SPLITS; ++sidx) {
            const float w = sidx < n_splits ? fast_exp2(st.ml[sidx].x - mx) : 0.f;
            l = fmaf(w, st.ml[sidx].y, l);
            o[0] = fmaf(w, st.o[sidx][0].x, o[0]); o[1] = fmaf(w, st.o[sidx][0].y, o[1]);
            o[2] = fmaf(w, st.o[sidx][0].z, o[2]); o[3] = fmaf(w, st.o[sidx][0].w, o[3]);
            o[4] = fmaf(w, st.o[sidx][1].x, o[4]); o[5] = fmaf(w, st.o[sidx][1].y, o[5]);
            o[6] = fmaf(w, st.o[sidx][1].z, o[6]); o[7] = fmaf(w, st.o[sidx][1].w, o[7]);
        }
        const float inv = 1.0f / l;
        union { uint32_t w[4]; bf16x8 v; } pk;
#pragma unroll
        for (int i = 0; i < 4; ++i) pk.w[i] = pack_bf16x2(o[2 * i] * inv, o[2 * i + 1] * inv);
        return pk.v;
    };
    const int n_blocks = k_first < K ? (K - k_first + k_stride - 1) / k_stride : 0;   // of this wavefront
    const int n_chunks = n_blocks / H;
    struct Chunk {
        bf16x8 b[NT][U];
        bf16x8 a[A_REGS ? (A_TWO ? U : U / 2) : 1];
    };
    // (A_MERGED) the states requested for a chunk's blocks, rows 0..7 and 8..15
    SplitStates pending[ASRC == A_MERGED ? U / 2 : 1][ASRC == A_MERGED && A_TWO ? 2 : 1];
    auto fetch_block_splits = [&](int h, int k0) {
        if (ASRC != A_MERGED) return;
#pragma unroll
        for (int j = 0; j < (A_TWO ? 2 : 1); ++j)
            if (j == 0 || a_two) fetch_splits(pending[h][j], arow_idx[j], min(k0 + 8 * piece[j], K - 8));
    };
    auto merge_block_splits = [&](Chunk& c, int h) {
        if (ASRC != A_MERGED) return;
#pragma unroll
        for (int j = 0; j < (A_TWO ? 2 : 1); ++j)
            if (j == 0 || a_two) c.a[A_TWO ? 2 * h + j : h] = merge_splits(pending[h][j]);
    };
    auto load_steps = [&](Chunk& c, int u0, int k0) {      // the k block at k0 (rows 0..7, rows 8..15) into slots u0, u0+1
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int k = min(k0 + 8 * piece[j], K - 8);
            // Weights that one workgroup alone reads (one row block: at most 8 rows, or the fused
            // norm's 16) and the wide product's (the logits head, as large as all the layers') are
            // requested with streaming loads: read once a step, they would only displace what is
            // read again (activations, scale and shift vectors, biases) from the caches. With
            // several row blocks the later ones find the weights in L2 and plain loads are kept.
            constexpr bool STREAM = ASRC != A_GLOBAL || !A_TWO;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const bf16x8* src = reinterpret_cast<const bf16x8*>(wrow[t][j] + k);
                c.b[t][u0 + j] = STREAM ? __builtin_nontemporal_load(src) : *src;
            }
            if (ASRC == A_GLOBAL && (j == 0 || a_two)) c.a[A_TWO ? u0 + j : u0 / 2] = *reinterpret_cast<const bf16x8*>(arow[j] + k);
            // (A_MERGED: the splits' states were requested before the weights and are merged after them)
        }
    };
    auto wave_lds_order = [&]() {       // orders the wavefront's own LDS writes and reads (no instruction)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // CNT (1 or 2) consecutive k blocks of a chunk, slots u0.., first k index k0: all their pieces go
    // through the wavefront's LDS region in one round trip (writes, then reads, then the MFMAs)
    auto mma_blocks = [&](const Chunk& c, int u0, int k0, auto cnt_tag) {
        constexpr int CNT = decltype(cnt_tag)::value;
        static_assert(CNT <= SB, "staging room");
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            if (A_REGS) {
                stage_a[i * 128 + lane] = c.a[A_TWO ? u0 + 2 * i : (u0 + 2 * i) / 2];
                if (a_two) stage_a[i * 128 + 64 + lane] = c.a[A_TWO ? u0 + 2 * i + 1 : 0];
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                stage_w[(i * NT + t) * 128 + lane] = c.b[t][u0 + 2 * i];
                stage_w[(i * NT + t) * 128 + 64 + lane] = c.b[t][u0 + 2 * i + 1];
            }
        }
        wave_lds_order();
        bf16x8 af[CNT][2], bf[CNT][NT][2];
#pragma unroll
        for (int i = 0; i < CNT; ++i)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int slot = row16 * 8 + ((2 * kq + half) ^ rd_swz);
                if (A_REGS) af[i][half] = stage_a[i * 128 + slot];
#pragma unroll
                for (int t = 0; t < NT; ++t) bf[i][t][half] = stage_w[(i * NT + t) * 128 + slot];
            }
        wave_lds_order();
#pragma unroll
        for (int i = 0; i < CNT; ++i)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int k = k0 + i * k_stride + 16 * kq + 8 * half;
                const int kc = min(k, K - 8);
#pragma unroll
                for (int mi = 0; mi < MT; ++mi) {
                    bf16x8 a;
                    if (IN_LDS) a = *reinterpret_cast<const bf16x8*>(a_s + static_cast<size_t>(mi * 16 + row16) * a_stride + kc);
                    else a = af[i][half];
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        const bf16x8 b = k < K ? bf[i][t][half] : zero;
                        acc[mi * NT + t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mi * NT + t], 0, 0, 0);
                    }
                }
            }
    };
    // `count` of the blocks in slots 0, 2, 4, ... of a chunk (count is uniform over the wavefront), k
    // indices from k0 on
    auto mma_some = [&](const Chunk& c, int count, int k0) {
#pragma unroll
        for (int h = 0; h < H; h += SB) {
            if (SB == 2 && h + 1 < H && h + 1 < count)
                mma_blocks(c, 2 * h, k0 + h * k_stride, std::integral_constant<int, SB>{});
            else if (h < count)
                mma_blocks(c, 2 * h, k0 + h * k_stride, std::integral_constant<int, 1>{});
        }
    };
    auto load_chunk = [&](Chunk& c, int chunk) {            // chunk index within this wavefront's blocks
        if (ASRC == A_MERGED) {
#pragma unroll
            for (int h = 0; h < H; ++h) fetch_block_splits(h, k_first + (chunk * H + h) * k_stride);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int h = 0; h < H; ++h) load_steps(c, 2 * h, k_first + (chunk * H + h) * k_stride);
        // the instruction scheduler must not sink these loads towards their uses: they are issued
        // here to be in flight together
        __builtin_amdgcn_sched_barrier(0);
        if (ASRC == A_MERGED) {
#pragma unroll
            for (int h = 0; h < H; ++h) merge_block_splits(c, h);
        }
    };
    auto mma_chunk = [&](const Chunk& c, int chunk) { mma_some(c, H, k_first + chunk * H * k_stride); };
    // rows of the fp32 stream that this wavefront normalises (read before the weights are
    // requested: loads complete in order, and the row addresses depend on these)
    int src_row[2] = {0, 0};
    if (LN_FUSED) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int m = min(m_base + wave + 8 * j, M - 1);      // 8 wavefronts, rows wave and wave + 8
            src_row[j] = rows ? rows[m] : m;
        }
    }
    Chunk c0, c1;
    auto load_left = [&]() {                                // the blocks after the last whole chunk
        const int first = n_chunks * H, left = n_blocks - first;
        if (ASRC == A_MERGED) {
#pragma unroll
            for (int h = 0; h < H - 1; ++h)
                if (h < left) fetch_block_splits(h, k_first + (first + h) * k_stride);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int h = 0; h < H - 1; ++h)
            if (h < left) load_steps(c1, 2 * h, k_first + (first + h) * k_stride);
        __builtin_amdgcn_sched_barrier(0);
        if (ASRC == A_MERGED) {
#pragma unroll
            for (int h = 0; h < H - 1; ++h)
                if (h < left) merge_block_splits(c1, h);
        }
    };
    // The first loads are one whole chunk for every wavefront, without a condition: a wavefront
    // with fewer blocks than a chunk takes its last block again (its own line, requested a moment
    // earlier) and leaves it unused. (Whole chunk or leftovers, decided by a branch, would hand the
    // norm that follows registers that count as pending on one side of the branch, and it would
    // wait for the weights.)
    const int last_block = n_blocks > 0 ? n_blocks - 1 : 0;
    auto first_loads = [&]() {
        if (ASRC == A_MERGED) {
#pragma unroll
            for (int h = 0; h < H; ++h) fetch_block_splits(h, k_first + min(h, last_block) * k_stride);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int h = 0; h < H; ++h) load_steps(c0, 2 * h, k_first + min(h, last_block) * k_stride);
        __builtin_amdgcn_sched_barrier(0);
        if (ASRC == A_MERGED) {
#pragma unroll
            for (int h = 0; h < H; ++h) merge_block_splits(c0, h);
        }
    };
    // The fused norm's operands are requested before the weights: loads return in the order of
    // their requests, so the norm (whose rows come from L2) can be computed while the weights are
    // still on their way from memory, which it could not if it had to wait for them first.
    const int nq = K / 4, n_u = (nq + 63) / 64;       // float4 per row; per lane (uniform)
    float4 gb_piece[2], v[2][8];
    // whether this wavefront's two rows exist is uniform over it: rows beyond M are not read
    const bool row_ok[2] = {m_base + wave < M, m_base + wave + 8 < M};
    if (LN_FUSED) {
        const float* x = static_cast<const float*>(Ain);
        const float4* g4 = reinterpret_cast<const float4*>(gamma);
        const float4* b4 = reinterpret_cast<const float4*>(beta);
        // (the rows first: they come from L2, and their mean and variance need nothing else)
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (u < n_u) {
                const int i = min(lane + 64 * u, nq - 1);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    if (row_ok[j]) v[j][u] = reinterpret_cast<const float4*>(x + static_cast<size_t>(src_row[j]) * lda)[i];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // scale and shift: 2 K / 4 pieces of 16 bytes over the workgroup's 512 threads (K <= 2048:
        // at most two each), shared through LDS instead of every wavefront loading all of both
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int i = min(tid + 512 * r, 2 * nq - 1);
            const float4* src = i < nq ? g4 + i : (beta ? b4 + (i - nq) : g4);
            gb_piece[r] = *src;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    first_loads();
    if (ASRC == A_STAGED) {
        // the workgroup's rows of A, copied once into LDS for all its wavefronts
        // (four 16-byte pieces per thread requested together, then written)
        const int kv = K / 8, total = 16 * MT * kv;
        for (int base = tid; base < total; base += 4 * blockDim.x) {
            bf16x8 v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int idx = min(base + j * static_cast<int>(blockDim.x), total - 1);
                const int m = idx / kv, c = idx - m * kv;
                v[j] = *reinterpret_cast<const bf16x8*>(A + static_cast<size_t>(min(m_base + m, M - 1)) * lda + 8 * c);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int idx = base + j * static_cast<int>(blockDim.x);
                const int m = idx / kv, c = idx - m * kv;
                if (idx < total)
                    *reinterpret_cast<bf16x8*>(a_s + static_cast<size_t>(m) * a_stride + 8 * c) =
                        (m_base + m < M) ? v[j] : zero;
            }
        }
        __syncthreads();
    }
    if (LN_FUSED) {
        // 8 wavefronts, two rows each; a row lives in registers (K <= 2048, K % 4 == 0): mean,
        // then variance of the centred values, all in fp32.
        float mean[2] = {0.f, 0.f}, inv[2] = {0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (!row_ok[j]) continue;
            float sum = 0.f;
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (u < n_u && lane + 64 * u < nq) sum += (v[j][u].x + v[j][u].y) + (v[j][u].z + v[j][u].w);
            mean[j] = wave_sum(sum) / static_cast<float>(K);
            float q = 0.f;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (u < n_u && lane + 64 * u < nq) {
                    const float a = v[j][u].x - mean[j], b = v[j][u].y - mean[j], c = v[j][u].z - mean[j], d = v[j][u].w - mean[j];
                    q += (a * a + b * b) + (c * c + d * d);
                }
            }
            inv[j] = 1.0f / sqrtf(wave_sum(q) / static_cast<float>(K) + eps);
        }
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int i = tid + 512 * r;
            if (i < 2 * nq) gb_s[i] = (i >= nq && !beta) ? make_float4(0.f, 0.f, 0.f, 0.f) : gb_piece[r];
        }
        lds_barrier();                 // scale and shift are in LDS (the weights stay in flight)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int m = wave + 8 * j;
            bf16_t* dst = a_s + static_cast<size_t>(m) * a_stride;
            if (!row_ok[j]) {
                for (int i = lane; i < nq; i += 64) *reinterpret_cast<uint2*>(dst + 4 * i) = make_uint2(0, 0);
                continue;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i = lane + 64 * u;
                if (u < n_u && i < nq) {
                    const float4 g = gb_s[i], b = gb_s[nq + i];
                    uint2 pk;
                    pk.x = pack_bf16x2((v[j][u].x - mean[j]) * inv[j] * g.x + b.x, (v[j][u].y - mean[j]) * inv[j] * g.y + b.y);
                    pk.y = pack_bf16x2((v[j][u].z - mean[j]) * inv[j] * g.z + b.z, (v[j][u].w - mean[j]) * inv[j] * g.w + b.w);
                    *reinterpret_cast<uint2*>(dst + 4 * i) = pk;
                }
            }
        }
        lds_barrier();
    }

    if (n_chunks == 0) {
        mma_some(c0, n_blocks, k_first);
    } else if (n_chunks == 1) {
        mma_chunk(c0, 0);
    } else if (n_chunks > 1) {
        // past the last chunk the prefetch takes chunk 0 again (long since arrived, never used)
        for (int ci = 0; ci < n_chunks; ci += 2) {
            load_chunk(c1, ci + 1 < n_chunks ? ci + 1 : 0);
            mma_chunk(c0, ci);
            load_chunk(c0, ci + 2 < n_chunks ? ci + 2 : 0);
            if (ci + 1 < n_chunks) mma_chunk(c1, ci + 1);
        }
    }
    {
        // blocks left over: fewer than H, loaded together
        const int first = n_chunks * H, left = n_chunks > 0 ? n_blocks - first : 0;
        if (left > 0) load_left();
        mma_some(c1, left, k_first + first * k_stride);
    }
    // accumulator layout of the 16x16 tile: register r of lane l holds row 4*(l/16) + r, column l%16
    if (!SPLIT_K) {
        if (!n_ok) return;
        const float bv = bias ? bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m_base + i * 16 + 4 * kq + r;
                if (m < M) epilogue<bf16_t>(mode, acc[i][r], bv, C, static_cast<size_t>(m) * ldc + n);
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[(static_cast<size_t>(wave) * T + i) * 256 + r * 64 + lane] = acc[i][r];
    __syncthreads();
    if (MT == 1) {
        // one output per tile and thread (the first 256); its bias and old residual value were
        // requested before the MFMA loop
        float vt[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            vt[t] = 0.f;
            if (tid < 256)
                for (int w = 0; w < nw; ++w) vt[t] += red[(static_cast<size_t>(w) * NT + t) * 256 + tid];
        }
        float& v = vt[0];
        if (NT == 1 && k_parts > 1) {
            // The parts of a tile meet in the workspace. Stores and loads of it are at device scope
            // (workgroups of one tile may run on different XCDs, whose L2 caches do not see each
            // other's lines); one thread's fences order them around the counter (a fence in every
            // thread costs tens of microseconds here, one about 1.5). The last workgroup leaves the
            // counter at zero for the next launch.
            const int tile = cb * row_blocks + rb;
            float* sums = part_sums + static_cast<size_t>(tile) * k_parts * 256;
            if (tid < 256) __hip_atomic_store(&sums[part * 256 + tid], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            if (tid == 0) {
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");      // after the barrier: covers every thread's stores
                const int arrived = __hip_atomic_fetch_add(&part_counters[tile], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                sm_last = (arrived == k_parts - 1) ? 1 : 0;
                if (sm_last) {
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                    __hip_atomic_store(&part_counters[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            __syncthreads();
            if (!sm_last) return;
            v = 0.f;
            if (tid < 256)
                for (int p = 0; p < k_parts; ++p)
                    v += __hip_atomic_load(&sums[p * 256 + tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (ep_ok[t]) {
                const float r = vt[t] + ep_bias[t];
                if (mode == EPI_ADD_RESIDUAL) static_cast<float*>(C)[ep_idx[t]] = ep_old[t] + r;
                else epilogue<bf16_t>(mode, r, 0.f, C, ep_idx[t]);
            }
        }
        return;
    }
    for (int idx = tid; idx < MT * 256; idx += blockDim.x) {
        const int i = idx / 256, r = (idx % 256) / 64, l = idx % 64;
        const int m = m_base + i * 16 + 4 * (l / 16) + r, nn = n0 + l % 16;
        if (m >= M || nn >= N) continue;
        const float bv = bias ? bias[nn] : 0.f;
        float v = 0.f;
        for (int w = 0; w < nw; ++w) v += red[(static_cast<size_t>(w) * MT + i) * 256 + r * 64 + l];
        epilogue<bf16_t>(mode, v, bv, C, static_cast<size_t>(m) * ldc + nn);
    }
}

constexpr int MAX_DYNAMIC_LDS = 160 * 1024 - 1024;      // the unit's LDS less the kernel's static variables
constexpr int SPLIT_COUNTERS = 4096;      // tiles that may be shared by several workgroups
constexpr int SPLIT_MAX_PARTS = 8;
constexpr int SPLIT_MIN_K_BLOCKS = 12;    // k blocks of 64 elements that every part keeps at least
constexpr int SPLIT_FROM_K_BLOCKS = 80;   // shorter K: the fences cost more than the parallelism gains (measured)

struct MergedA {        // A_MERGED: where the attention splits' states lie
    const float* split_o = nullptr;
    const float* split_ml = nullptr;
    int n_splits = 1, heads = 1, head_dim = 8;
};

template <bool LN_FUSED, bool MERGED = false>
static int launch_skinny(const void* A, int lda, const bf16_t* W, int ldw, const float* bias, void* C, int ldc,
                         int M, int N, int K, int mode, const float* gamma, const float* beta, float eps,
                         const int* rows, hipStream_t stream, void* workspace = nullptr, size_t workspace_bytes = 0,
                         MergedA merged = MergedA{}) {
    static_assert(!(LN_FUSED && MERGED), "one source of A");
    const int tiles = (N + 15) / 16;
    const bool split_k = tiles < 1024;
    // Narrow products: 16 rows per workgroup and one workgroup per 16 rows (more workgroups, each
    // reading only its rows). Wide products: every wavefront keeps all rows of its tile in
    // registers (up to 4 accumulators), so the weights are streamed once.
    int row_blocks = split_k ? (M + 15) / 16 : 1;
    int mt = split_k ? 1 : (M + 15) / 16;
    // Wide products without the fused norm: every wavefront needs all rows of A for its tile, as
    // many bytes as the tile's weights or more, so the workgroup copies its rows into LDS once
    // (at most 160 KB: more rows than fit are split over row blocks).
    const bool staged = !LN_FUSED && !split_k;
    size_t staged_bytes = 0;
    if (staged) {
        const size_t row16_bytes = static_cast<size_t>(16) * (K + 8) * sizeof(bf16_t);
        int fit = static_cast<int>((160 - 32) * 1024 / row16_bytes);      // 32 KB: the wavefronts' transposition regions
        if (fit < 1) return -2;
        if (fit > 4) fit = 4;
        row_blocks = (mt + fit - 1) / fit;
        mt = (mt + row_blocks - 1) / row_blocks;
        staged_bytes = row16_bytes * mt;
    }
    int nw;
    int k_blocks = (K + 63) / 64;
    // Narrow products with a long K (from SPLIT_FROM_K_BLOCKS blocks): k_parts workgroups per tile,
    // as many as fit one round over the 256 compute units while each keeps at least
    // SPLIT_MIN_K_BLOCKS k blocks. Needs the workspace: SPLIT_COUNTERS counters, then 256 floats
    // per tile and part.
    int k_parts = 1;
    if (MERGED && (!split_k || M > 16 || merged.n_splits < 1 || merged.n_splits > MERGE_MAX_SPLITS ||
                   merged.head_dim % 8 != 0 || merged.heads * merged.head_dim != K))
        return -2;
    if (split_k && !LN_FUSED && !MERGED && workspace != nullptr && k_blocks >= SPLIT_FROM_K_BLOCKS) {
        const int wgs = tiles * row_blocks;
        k_parts = std::min(std::min(256 / std::max(wgs, 1), k_blocks / SPLIT_MIN_K_BLOCKS), SPLIT_MAX_PARTS);
        if (k_parts < 2 || wgs > SPLIT_COUNTERS ||
            workspace_bytes < SPLIT_COUNTERS * sizeof(int) + static_cast<size_t>(wgs) * k_parts * 256 * sizeof(float))
            k_parts = 1;
        k_blocks = (k_blocks + k_parts - 1) / k_parts;      // per workgroup from here on
    }
    int* part_counters = static_cast<int*>(workspace);
    float* part_sums = reinterpret_cast<float*>(static_cast<char*>(workspace) + SPLIT_COUNTERS * sizeof(int));
    if (split_k) {
        // the wavefront count (at least 4: one thread per output of the tile) that leaves every
        // wavefront the fewest k blocks; among equals the smallest, which has the least to add up
        // (the fused norm is written for 8 wavefronts, two rows each)
        // (at most 12: two chunks of loads in flight per wavefront need more than the 128 registers
        // that 16 wavefronts would leave each)
        nw = 4;
        for (int cand = 5; cand <= 12; ++cand)
            if ((k_blocks + cand - 1) / cand < (k_blocks + nw - 1) / nw) nw = cand;
        if (LN_FUSED) nw = 8;
    } else {
        // one round of workgroups over the 256 compute units, each wavefront one tile
        nw = (tiles * row_blocks + 255) / 256;
        nw = nw < 4 ? 4 : (nw > 16 ? 16 : nw);
    }
    // More than 256 tiles (and one row block): two tiles per workgroup, the columns dealt out evenly
    // to 256 workgroups.
    int cols_per_wg = 16;
    const bool two_tiles = !MERGED && split_k && row_blocks == 1 && k_parts == 1 && tiles > 256 && tiles <= 512 &&
                           (LN_FUSED || M <= 8);
    if (two_tiles) cols_per_wg = (N + 255) / 256;
    // Fewer than 256 tiles, one row block and a long K (the second product of the feed-forward):
    // narrower tiles, down to 4 columns, so that more compute units share the weights. (Short K, or
    // the fused norm: the kernel's time is latency, not bytes, and nothing is gained; measured.)
    if (split_k && !LN_FUSED && !MERGED && row_blocks == 1 && k_parts == 1 && tiles < 256 && k_blocks >= 48)
        cols_per_wg = std::min(16, std::max((N + 255) / 256, 4));
    const int col_blocks = split_k ? (N + cols_per_wg - 1) / cols_per_wg : (tiles + nw - 1) / nw;
    const dim3 grid((col_blocks + N_XCD - 1) / N_XCD * N_XCD * row_blocks, k_parts), block(nw * 64);
    size_t smem = split_k ? static_cast<size_t>(nw) * mt * (two_tiles ? 2 : 1) * 256 * sizeof(float) : 0;
    // the wavefronts' transposition regions (two k blocks at a time where the kernel stages two)
    smem += static_cast<size_t>(nw) * (staged ? 2048 : LN_FUSED ? (two_tiles ? 8192 : 4096) : (two_tiles ? 6144 : 8192));
    if (staged) {
        staged_bytes += smem;
#define SKINNY_STAGED(MTV)                                                                             \
    case MTV: {                                                                                        \
        auto kernel = gemm_bf16_skinny<MTV, A_STAGED, false, 4>;                                        \
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),                      \
                                           hipFuncAttributeMaxDynamicSharedMemorySize,                 \
                                           static_cast<int>(staged_bytes));                            \
        if (e != hipSuccess) return static_cast<int>(e);                                               \
        kernel<<<grid, block, staged_bytes, stream>>>(W, ldw, N, K, M, col_blocks, row_blocks, 16, 1, A, lda, mode, \
                                                      bias, C, ldc, gamma, beta, eps, rows, nullptr, nullptr, \
                                                      nullptr, nullptr, 1, 1, 8);                      \
        break;                                                                                         \
    }
        switch (mt) {
            SKINNY_STAGED(1) SKINNY_STAGED(2) SKINNY_STAGED(3) SKINNY_STAGED(4)
            default: return -2;
        }
#undef SKINNY_STAGED
        return 0;
    }
    if (LN_FUSED) {
        smem += static_cast<size_t>(16) * mt * (K + 8) * sizeof(bf16_t) + static_cast<size_t>(2) * K * sizeof(float);
        if (K > 2048 || (reinterpret_cast<uintptr_t>(A) & 15) || lda % 4 != 0 ||
            (reinterpret_cast<uintptr_t>(gamma) & 15) || (reinterpret_cast<uintptr_t>(beta) & 15))
            return -2;
    }
    if (smem > MAX_DYNAMIC_LDS) return -2;
    constexpr int ASRC = LN_FUSED ? A_NORMED : (MERGED ? A_MERGED : A_GLOBAL);
#define SKINNY_LAUNCH(SPLIT, UV, A2, NTV)                                                              \
    do {                                                                                               \
        auto kernel = gemm_bf16_skinny<1, ASRC, SPLIT, UV, A2, NTV>;                                   \
        static bool lds_allowed = false;      /* more than 64 KB of dynamic LDS has to be asked for once */ \
        if (!lds_allowed) {                                                                            \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),                  \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, MAX_DYNAMIC_LDS); \
            if (e != hipSuccess) return static_cast<int>(e);                                           \
            lds_allowed = true;                                                                        \
        }                                                                                              \
        kernel<<<grid, block, smem, stream>>>(W, ldw, N, K, M, col_blocks, row_blocks, cols_per_wg, k_parts, A, lda, \
                                              mode, bias, C, ldc, gamma, beta, eps, rows, part_sums,      \
                                              part_counters, merged.split_o, merged.split_ml, merged.n_splits, \
                                              merged.heads, merged.head_dim);                          \
    } while (0)
    if (split_k) {
        // a chunk holds all k blocks of a wavefront when they are at most 3 (4 without the fused
        // norm and with at most 8 rows): whole chunks only, so nothing is requested twice. The
        // largest chunks of the kernels without the norm spill a few registers, and are still
        // faster than smaller chunks (measured)
        const int per_wave = (k_blocks + nw - 1) / nw;
        if (two_tiles) {
            // (two tiles per chunk slot: half the blocks per chunk)
            if (per_wave <= 1 || !LN_FUSED) SKINNY_LAUNCH(true, 2, false, 2);
            else SKINNY_LAUNCH(true, 4, false, 2);
        } else if (LN_FUSED) {
            switch (std::min(per_wave, 3)) {
                case 1: SKINNY_LAUNCH(true, 2, false, 1); break;
                case 2: SKINNY_LAUNCH(true, 4, false, 1); break;
                default: SKINNY_LAUNCH(true, 6, false, 1); break;
            }
        } else if (MERGED) {
            // the splits' states of a whole chunk are in flight together: one chunk holds all of a
            // wavefront's k blocks, at most 3
            if (per_wave > 3) return -2;
            if (M <= 8) {
                switch (per_wave) {
                    case 1: SKINNY_LAUNCH(true, 2, false, 1); break;
                    case 2: SKINNY_LAUNCH(true, 4, false, 1); break;
                    default: SKINNY_LAUNCH(true, 6, false, 1); break;
                }
            } else {
                switch (per_wave) {
                    case 1: SKINNY_LAUNCH(true, 2, true, 1); break;
                    case 2: SKINNY_LAUNCH(true, 4, true, 1); break;
                    default: SKINNY_LAUNCH(true, 6, true, 1); break;
                }
            }
        } else if (M <= 8) {
            switch (std::min(per_wave, 4)) {
                case 1: SKINNY_LAUNCH(true, 2, false, 1); break;
                case 2: SKINNY_LAUNCH(true, 4, false, 1); break;
                case 3: SKINNY_LAUNCH(true, 6, false, 1); break;
                default: SKINNY_LAUNCH(true, 8, false, 1); break;
            }
        } else {
            switch (std::min(per_wave, 3)) {
                case 1: SKINNY_LAUNCH(true, 2, true, 1); break;
                case 2: SKINNY_LAUNCH(true, 4, true, 1); break;
                default: SKINNY_LAUNCH(true, 6, true, 1); break;
            }
        }
    } else {
        // wide products (the logits head): normalising the rows once in a kernel of its own and
        // staging them in LDS is faster than every workgroup normalising them again
        return -2;
    }
#undef SKINNY_LAUNCH
    return 0;
}


static int gemm_bf16_dispatch(const void* A, int lda, const void* W, int ldw, const float* bias, void* C, int ldc,
                              int M, int N, int K, int mode, hipStream_t stream, KvScatter kv,
                              void* workspace = nullptr, size_t workspace_bytes = 0) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0 || lda % 8 != 0 || ldw % 8 != 0) return -1;
    if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(W) & 15)) return -1;
    const bf16_t* a = static_cast<const bf16_t*>(A);
    const bf16_t* w = static_cast<const bf16_t*>(W);
    const bool scatter = kv.slots != nullptr;       // only the many-row kernel scatters
    // Which kernel for up to 256 rows. Up to 16 rows (one row block) and for the widest products (the
    // logits head) the weight-streaming kernel, always. In between both are priced, in microseconds,
    // by formulas fitted to measurements on the products of GPT-2 small to XL at 24 to 256 rows: the
    // weight-streaming kernel runs its 16-row by 16-column workgroups in rounds of 256 whose time
    // grows with K (steeply beyond 3072, where a wavefront's share of K no longer fits its chunks);
    // the tiled kernel's time is its k loop, a little more where K makes it take the checked loop.
    const int col_tiles = (N + 15) / 16, row_blocks16 = (M + 15) / 16;
    auto streaming_is_faster = [&]() {
        const double rounds = static_cast<double>((static_cast<long>(col_tiles) * row_blocks16 + 255) / 256);
        const double streaming = 2.0 + rounds * (K <= 3072 ? 1.2 + 0.0008 * K : 0.0025 * K);
        const double blocks = static_cast<double>((M + 63) / 64) * ((N + 63) / 64);
        const bool ragged = K % 64 != 0;
        const double tiled = (blocks <= 128 ? 4.0 : 5.0) + 0.18 * (K / 64.0) * std::max(1.0, blocks / 256.0) + (ragged ? 2.0 : 0.0) +
                             (M <= 32 ? 4.0 : 0.0);       // (up to 32 rows the tiled kernel has one shape, 32x128)
        return streaming <= tiled;
    };
    const bool few_rows = M <= 16 || (M <= 64 && col_tiles >= 1024) || (M <= 256 && streaming_is_faster());
    if (!scatter && few_rows && launch_skinny<false>(A, lda, w, ldw, bias, C, ldc, M, N, K, mode, nullptr, nullptr,
                                                    0.f, nullptr, stream, workspace, workspace_bytes) == 0) {
        // few rows: weight-streaming kernel
    } else if (M <= 32) {
        launch_tiled<1, 4, 1, 1, 64, 3>(a, lda, w, ldw, bias, C, ldc, M, N, K, mode, stream, kv);
    } else {
        // Tile choice. The compute units run the workgroups in rounds of 256, and a workgroup's time
        // grows with its tile's area, less so for large tiles (they move fewer bytes per flop). So
        // each shape is priced as rounds x area / efficiency, the efficiencies fitted to measurements
        // at 2048 rows on the products of GPT-2 small to XL, and the cheapest runs. Few workgroups
        // (one round for every shape) thus take the smallest tiles, which spread over more units
        // (64x32 where even 64x64 tiles leave most units idle: decode at 48 to 128 rows).
        struct Shape { int bm, bn; double efficiency; };
        static const Shape shapes[] = {{128, 256, 1.05}, {128, 192, 1.0}, {128, 128, 0.9}, {64, 128, 0.7},
                                       {64, 96, 0.65},   {64, 64, 0.55}, {64, 32, 0.4}};
        int best = 0;
        double best_cost = 1e300;
        for (int c = 0; c < 7; ++c) {
            if (c == 4 && N > 1024) continue;       // 64x96 pays on narrow outputs only (measured: up to twice the time of 64x64 on wide ones)
            const long blocks = static_cast<long>((M + shapes[c].bm - 1) / shapes[c].bm) * ((N + shapes[c].bn - 1) / shapes[c].bn);
            const double cost = static_cast<double>((blocks + 255) / 256) * shapes[c].bm * shapes[c].bn / shapes[c].efficiency;
            if (cost < best_cost) { best_cost = cost; best = c; }
        }
        // With a long K the smaller tiles' time goes to the barrier intervals of the k loop, and two
        // groups of wavefronts per workgroup, each on half of a twice as wide k tile, halve their
        // number (measured at K of 3072 to 6400: 9 to 17 % less time; at K of 768 to 1600: none).
        const bool long_k = K >= 2048;
#define TILE(...) launch_tiled<__VA_ARGS__>(a, lda, w, ldw, bias, C, ldc, M, N, K, mode, stream, kv)
        switch (best) {
            case 0: TILE(2, 4, 2, 2, 64, 4); break;
            case 1: TILE(4, 2, 1, 3, 64, 3); break;
            case 2: if (long_k) TILE(2, 4, 2, 1, 64, 3, 2); else TILE(2, 4, 2, 1, 64, 3); break;
            case 3: TILE(2, 4, 1, 1, 64, 4); break;
            case 4: if (long_k) TILE(2, 3, 1, 1, 64, 5, 2); else TILE(2, 3, 1, 1, 64, 5); break;
            case 5: if (long_k) TILE(2, 2, 1, 1, 64, 4, 2); else TILE(2, 2, 1, 1, 64, 4); break;
            default: TILE(2, 1, 1, 1, 64, 4, 2); break;     // 64x32 (few workgroups in all): two wavefronts, always two groups
        }
#undef TILE
    }
    MLLM_LAUNCH_CHECK();
    return 0;
}

extern "C" {

// Returns 0, a HIP error code, or -1 when K or the row strides are not multiples of 8
// elements or a base pointer is not 16-byte aligned.
// `workspace` (optional; 4-byte aligned, zero when first handed over, never written by anyone else)
// lets narrow products of few rows and a long K share a tile among several workgroups: 16 KB of
// counters, then 1 KB per workgroup of such a launch (at most 256). Launches that use one
// workspace must not overlap.
int mllm_gemm_bf16(const void* A, int lda, const void* W, int ldw, const float* bias, void* C, int ldc,
                   int M, int N, int K, int mode, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    return gemm_bf16_dispatch(A, lda, W, ldw, bias, C, ldc, M, N, K, mode, stream, KvScatter{}, workspace,
                              workspace_bytes);
}


// The plain bf16 store (mode 0) with the key/value scatter of KvScatter fused: C = A W^T + bias, and
// columns [q_cols, q_cols + kv_dim) / [q_cols + kv_dim, q_cols + 2 kv_dim) of row m also go to row
// slots[m] (>= 0) of k_pages / v_pages ([rows, kv_dim] bf16). q_cols and kv_dim must be multiples
// of 4 and N == q_cols + 2 kv_dim; -1 otherwise or as mllm_gemm_bf16.
int mllm_gemm_bf16_kv(const void* A, int lda, const void* W, int ldw, const float* bias, void* C, int ldc,
                      int M, int N, int K, const int* slots, void* k_pages, void* v_pages, int q_cols, int kv_dim,
                      hipStream_t stream) {
    if (slots == nullptr || q_cols < 0 || kv_dim <= 0 || q_cols % 4 != 0 || kv_dim % 4 != 0 ||
        N != q_cols + 2 * kv_dim)
        return -1;
    KvScatter kv{slots, static_cast<bf16_t*>(k_pages), static_cast<bf16_t*>(v_pages), q_cols, kv_dim};
    return gemm_bf16_dispatch(A, lda, W, ldw, bias, C, ldc, M, N, K, EPI_STORE, stream, kv);
}

// The product whose A is the output of split decode attention, merged from the splits' states while it
// is loaded: C = epilogue(merge(states) W^T + bias) with A[m, h * head_dim + e] = sum_s w_s o_s[e] /
// sum_s w_s l_s, w_s = 2^(m_s - max m). M <= 16 tokens, n_splits <= 4, head_dim % 8 == 0, K = n_heads *
// head_dim <= 2304 or so. Returns 0, a HIP error code, -1 for misaligned operands, or -2 when the sizes
// are not ones this kernel takes (the caller then merges with mllm_merge_attention_splits and runs the
// ordinary product).
int mllm_gemm_bf16_merged(const float* split_o, const float* split_ml, int n_splits, int n_heads, int head_dim,
                          const void* W, int ldw, const float* bias, void* C, int ldc, int M, int N, int mode,
                          hipStream_t stream) {
    const int K = n_heads * head_dim;
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0 || ldw % 8 != 0 || (reinterpret_cast<uintptr_t>(W) & 15) ||
        (reinterpret_cast<uintptr_t>(split_o) & 15) || (reinterpret_cast<uintptr_t>(split_ml) & 7))
        return -1;
    MergedA merged{split_o, split_ml, n_splits, n_heads, head_dim};
    int rc = launch_skinny<false, true>(nullptr, K, static_cast<const bf16_t*>(W), ldw, bias, C, ldc, M, N, K, mode,
                                        nullptr, nullptr, 0.f, nullptr, stream, nullptr, 0, merged);
    if (rc != 0) return rc;
    MLLM_LAUNCH_CHECK();
    return 0;
}

// LayerNorm of the fp32 rows x[M,K] (row m taken from x[rows[m]] when `rows` is given) fused into the
// product with W[N,K]: C = epilogue(LN(x) W^T + bias).
// M <= 64, N < 16384. Returns 0, a HIP error code, -1 for misaligned operands, or -2 when M, N or K is too
// large for the fused kernel (the caller then runs the norm and the product separately).
int mllm_ln_gemm_bf16(const float* x, int ldx, const int* rows, const float* gamma, const float* beta, float eps,
                      const void* W, int ldw, const float* bias, void* C, int ldc, int M, int N, int K, int mode,
                      hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0 || ldw % 8 != 0 || (reinterpret_cast<uintptr_t>(W) & 15)) return -1;
    if (M > 64) return -2;
    int rc = launch_skinny<true>(x, ldx, static_cast<const bf16_t*>(W), ldw, bias, C, ldc, M, N, K, mode, gamma,
                                 beta, eps, rows, stream);
    if (rc != 0) return rc;
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

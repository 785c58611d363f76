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

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define BK 64
#define LDS_STRIDE (BK + 8)   // 144-byte rows: 16-byte reads of 32 consecutive rows hit distinct banks

template <int WM, int WN, int TM, int TN>
__global__ void __launch_bounds__(256)
gemm_bf16_mfma(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
               const float* __restrict__ bias, void* __restrict__ C, int ldc, int M, int N, int K, int mode) {
    static_assert(WM * WN == 4, "four wavefronts per block");
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    constexpr int A_CHUNKS = BM * (BK / 8) / 256, W_CHUNKS = BN * (BK / 8) / 256;
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) bf16_t Ws[BN * LDS_STRIDE];

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int wm = wave / WN, wn = wave % WN;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    uint4 ra[A_CHUNKS], rw[W_CHUNKS];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + i * 256, row = c / (BK / 8), kc = c % (BK / 8);
            const int m = m0 + row, k = k0 + kc * 8;
            ra[i] = (m < M && k < K) ? *reinterpret_cast<const uint4*>(A + static_cast<size_t>(m) * lda + k)
                                     : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const int c = tid + i * 256, row = c / (BK / 8), kc = c % (BK / 8);
            const int n = n0 + row, k = k0 + kc * 8;
            rw[i] = (n < N && k < K) ? *reinterpret_cast<const uint4*>(W + static_cast<size_t>(n) * ldw + k)
                                     : make_uint4(0, 0, 0, 0);
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + i * 256, row = c / (BK / 8), kc = c % (BK / 8);
            *reinterpret_cast<uint4*>(As + row * LDS_STRIDE + kc * 8) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const int c = tid + i * 256, row = c / (BK / 8), kc = c % (BK / 8);
            *reinterpret_cast<uint4*>(Ws + row * LDS_STRIDE + kc * 8) = rw[i];
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();            // readers of the previous tile are done
        stage();
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            const int kofs = ks * 16 + 8 * (lane / 32);
            bf16x8 a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                a[i] = *reinterpret_cast<const bf16x8*>(As + ((wm * TM + i) * 32 + lane % 32) * LDS_STRIDE + kofs);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                b[j] = *reinterpret_cast<const bf16x8*>(Ws + ((wn * TN + j) * 32 + lane % 32) * LDS_STRIDE + kofs);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    }

    // accumulator layout of the 32x32 tile: register r of lane l holds
    // row 8*(r/4) + 4*(l/32) + r%4, column l%32
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + (wn * TN + j) * 32 + lane % 32;
            if (n >= N) continue;
            const float bv = bias ? bias[n] : 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + (wm * TM + i) * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
                if (m < M) epilogue<bf16_t>(mode, acc[i][j][r], bv, C, static_cast<size_t>(m) * ldc + n);
            }
        }
    }
}

extern "C" {

// Returns 0, a HIP error code, or -1 when K or the row strides are not multiples of 8
// elements or a base pointer is not 16-byte aligned.
int mllm_gemm_bf16(const void* A, int lda, const void* W, int ldw, const float* bias, void* C, int ldc,
                   int M, int N, int K, int mode, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0 || lda % 8 != 0 || ldw % 8 != 0) return -1;
    if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(W) & 15)) return -1;
    const bf16_t* a = static_cast<const bf16_t*>(A);
    const bf16_t* w = static_cast<const bf16_t*>(W);
    auto blocks = [&](int bm, int bn) { return static_cast<long>((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if (M <= 32) {
        dim3 grid((N + 127) / 128, (M + 31) / 32);
        gemm_bf16_mfma<1, 4, 1, 1><<<grid, 256, 0, stream>>>(a, lda, w, ldw, bias, C, ldc, M, N, K, mode);
    } else if (blocks(128, 128) >= 512) {
        dim3 grid((N + 127) / 128, (M + 127) / 128);
        gemm_bf16_mfma<2, 2, 2, 2><<<grid, 256, 0, stream>>>(a, lda, w, ldw, bias, C, ldc, M, N, K, mode);
    } else {
        dim3 grid((N + 63) / 64, (M + 63) / 64);
        gemm_bf16_mfma<2, 2, 1, 1><<<grid, 256, 0, stream>>>(a, lda, w, ldw, bias, C, ldc, M, N, K, mode);
    }
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

// True fp32 matrix product for the 32-bit path: C[M,N] = A[M,K] * W[N,K]^T (+ bias, epilogue).
// Plain FMA in fp32, every output accumulated over k in a fixed order, so a row's
// result does not depend on which other rows share the launch (beyond the choice between the
// two kernels below, which add in different orders). No reduced-precision matrix mode is
// involved. Any M, N, K.
//
// Same contract as the reference's bounds-safe kernel
// (/root/reference/src/kernels/gemm.cu:238-392: alpha*acc + beta*old + bias, optional GELU),
// with the weight held as [N,K] (k contiguous) instead of [K,N].
#include "common.h"

#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

__global__ void __launch_bounds__(256)
gemm_f32_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                const float* __restrict__ bias, void* __restrict__ C, int ldc, int M, int N, int K, int mode) {
    __shared__ float As[F32_BK][F32_BM + 4];
    __shared__ float Ws[F32_BK][F32_BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * F32_BM, n0 = blockIdx.x * F32_BN;
    // loader mapping: 64 rows x 4 k-quads
    const int lrow = tid / 4, lk = (tid % 4) * 4;
    const bool vec_a = (lda % 4 == 0) && ((reinterpret_cast<uintptr_t>(A) & 15) == 0);
    const bool vec_w = (ldw % 4 == 0) && ((reinterpret_cast<uintptr_t>(W) & 15) == 0);

    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += F32_BK) {
        float av[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
        const int kk = k0 + lk;
        const int am = m0 + lrow, wn = n0 + lrow;
        if (am < M) {
            const float* p = A + static_cast<size_t>(am) * lda + kk;
            if (vec_a && kk + 3 < K) {
                float4 v = *reinterpret_cast<const float4*>(p);
                av[0] = v.x; av[1] = v.y; av[2] = v.z; av[3] = v.w;
            } else {
                for (int i = 0; i < 4; ++i) if (kk + i < K) av[i] = p[i];
            }
        }
        if (wn < N) {
            const float* p = W + static_cast<size_t>(wn) * ldw + kk;
            if (vec_w && kk + 3 < K) {
                float4 v = *reinterpret_cast<const float4*>(p);
                wv[0] = v.x; wv[1] = v.y; wv[2] = v.z; wv[3] = v.w;
            } else {
                for (int i = 0; i < 4; ++i) if (kk + i < K) wv[i] = p[i];
            }
        }
        __syncthreads();   // the previous tile's readers are done
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            As[lk + i][lrow] = av[i];
            Ws[lk + i][lrow] = wv[i];
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < F32_BK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            epilogue<float>(mode, acc[i][j], bias ? bias[n] : 0.f, C, static_cast<size_t>(m) * ldc + n);
        }
    }
}

// Few rows (decode): the product is bound by reading W once, and the tiled kernel above would
// start N/64 workgroups for it. Here a wavefront owns one output column (WAVES columns a workgroup):
// its lanes walk the column's weights in 16-byte steps (a wavefront's load is 1 KB of one row), the
// activations of up to ROWS rows wait in LDS in chunks of F32R_KC floats, and a lane's partial sums
// (k ascending) are added over the wavefront in a fixed order. More rows than ROWS take further passes over W.
// Needs K and the row strides in multiples of 4 floats and 16-byte aligned operands.
#define F32R_KC 512      // 128 16-byte steps: two per lane

template <int ROWS, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
gemm_f32_rows_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                     const float* __restrict__ bias, void* __restrict__ C, int ldc, int M, int N, int K, int mode) {
    __shared__ __attribute__((aligned(16))) float a_s[ROWS][F32R_KC];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
    const int n = blockIdx.x * WAVES + wave;
    const float* wrow = W + static_cast<size_t>(min(n, N - 1)) * ldw;       // a surplus wavefront repeats the last column
    constexpr int STAGED = (ROWS * (F32R_KC / 4) + 64 * WAVES - 1) / (64 * WAVES);   // 16-byte steps of a chunk a thread stages
    for (int m0 = 0; m0 < M; m0 += ROWS) {
        float acc[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) acc[r] = 0.f;
        // With a handful of wavefronts on a compute unit nothing hides a load's latency but the kernel itself:
        // the weights and the activations of the next chunk are asked for before the chunk in LDS is used.
        // A chunk is at most two 16-byte steps per lane (the second from a clamped address; its product is
        // left out where it is past the chunk).
        const int q0 = lane, q1 = lane + 64;
        float4 w0, w1, v[STAGED];
        auto fetch = [&](int kc0) {
            const int quads = min(F32R_KC, K - kc0) / 4;
            w0 = *reinterpret_cast<const float4*>(wrow + kc0 + 4 * min(q0, quads - 1));
            w1 = *reinterpret_cast<const float4*>(wrow + kc0 + 4 * min(q1, quads - 1));
#pragma unroll
            for (int u = 0; u < STAGED; ++u) {
                const int idx = tid + 64 * WAVES * u, r = idx / quads, q = idx % quads;
                v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (idx < ROWS * quads && m0 + r < M)
                    v[u] = *reinterpret_cast<const float4*>(A + static_cast<size_t>(m0 + r) * lda + kc0 + 4 * q);
            }
        };
        fetch(0);
        for (int kc0 = 0; kc0 < K; kc0 += F32R_KC) {
            const int quads = min(F32R_KC, K - kc0) / 4;
            const float4 c0 = w0, c1 = w1;
            __syncthreads();          // the chunk before has been read
#pragma unroll
            for (int u = 0; u < STAGED; ++u) {
                const int idx = tid + 64 * WAVES * u, r = idx / quads, q = idx % quads;
                if (idx < ROWS * quads) *reinterpret_cast<float4*>(&a_s[r][4 * q]) = v[u];
            }
            if (kc0 + F32R_KC < K) fetch(kc0 + F32R_KC);
            __syncthreads();
            if (q0 < quads) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    const float4 a4 = *reinterpret_cast<const float4*>(&a_s[r][4 * q0]);
                    acc[r] = fmaf(a4.x, c0.x, acc[r]);
                    acc[r] = fmaf(a4.y, c0.y, acc[r]);
                    acc[r] = fmaf(a4.z, c0.z, acc[r]);
                    acc[r] = fmaf(a4.w, c0.w, acc[r]);
                }
            }
            if (q1 < quads) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    const float4 a4 = *reinterpret_cast<const float4*>(&a_s[r][4 * q1]);
                    acc[r] = fmaf(a4.x, c1.x, acc[r]);
                    acc[r] = fmaf(a4.y, c1.y, acc[r]);
                    acc[r] = fmaf(a4.z, c1.z, acc[r]);
                    acc[r] = fmaf(a4.w, c1.w, acc[r]);
                }
            }
        }
        float mine = 0.f;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const float t = wave_sum(acc[r]);
            if (lane == r) mine = t;
        }
        if (n < N && lane < ROWS && m0 + lane < M)
            epilogue<float>(mode, mine, bias ? bias[n] : 0.f, C, static_cast<size_t>(m0 + lane) * ldc + n);
    }
}

extern "C" {

int mllm_gemm_f32(const float* A, int lda, const float* W, int ldw, const float* bias, void* C, int ldc,
                  int M, int N, int K, int mode, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    const bool quads = K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 &&
                       ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(W)) & 15) == 0;
    if (M <= 64 && quads && K > 0) {
        // Workgroups start at a limited rate (a few hundred a microsecond over the chip): from 2,048 columns on
        // a workgroup takes eight instead of four, which also halves what is staged (sixteen lose again: at
        // 50,257 columns 54 us against 45).
        if (N >= 2048) {
            const dim3 rows_grid((N + 7) / 8);
            if (M <= 8) gemm_f32_rows_kernel<8, 8><<<rows_grid, 512, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, mode);
            else gemm_f32_rows_kernel<16, 8><<<rows_grid, 512, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, mode);
        } else {
            const dim3 rows_grid((N + 3) / 4);
            if (M <= 8) gemm_f32_rows_kernel<8, 4><<<rows_grid, 256, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, mode);
            else gemm_f32_rows_kernel<16, 4><<<rows_grid, 256, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, mode);
        }
        MLLM_LAUNCH_CHECK();
        return 0;
    }
    dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
    gemm_f32_kernel<<<grid, 256, 0, stream>>>(A, lda, W, ldw, bias, C, ldc, M, N, K, mode);
    MLLM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"

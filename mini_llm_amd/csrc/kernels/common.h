// Shared device helpers for the gfx950 kernels: bf16 conversion, wave/block
// reductions for 64-wide wavefronts, activation functions and the GEMM epilogue.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define MLLM_WAVE 64

// dtype codes of the C ABI
#define MLLM_F32 0
#define MLLM_BF16 1

// GEMM epilogues
#define EPI_STORE 0         // out[m,n] = acc + bias            (activation dtype)
#define EPI_GELU_TANH 1     // out[m,n] = gelu_tanh(acc + bias) (activation dtype)
#define EPI_GELU_ERF 2      // out[m,n] = gelu_erf(acc + bias)  (activation dtype)
#define EPI_ADD_RESIDUAL 3  // res[m,n] += acc + bias           (fp32, in place)
#define EPI_STORE_F32 4     // out[m,n] = acc + bias            (fp32)

struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_to_float(bf16_t v) {
    return __uint_as_float(static_cast<uint32_t>(v.bits) << 16);
}

// Round to nearest, ties to even (the hardware conversion of gfx950, v_cvt_pk_bf16_f32).
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
    bf16_t r;
    r.bits = __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
    return r;
}
// Two values converted by one instruction; `a` lands in the low half.
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const bf16x2_t v = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
    return __builtin_bit_cast(uint32_t, v);
}
// 2^x by the hardware instruction alone: for arguments <= 0, where results below the normal
// range may flush to zero (softmax weights).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// 2^x for a kernel instantiated for element type T: the bare instruction for bfloat16, the library's
// full-range, full-precision exp2f for the 32-bit path.
template <typename T> __device__ __forceinline__ float exp2_for(float x) {
    return sizeof(T) == 4 ? exp2f(x) : __builtin_amdgcn_exp2f(x);
}

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return bf16_to_float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return float_to_bf16(v); }

// Loads 8 consecutive elements as floats; the address must be 16-byte aligned.
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
    float4 a = *reinterpret_cast<const float4*>(p);
    float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
    uint4 a = *reinterpret_cast<const uint4*>(p);
    v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
    v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
    v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xffff0000u);
    v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xffff0000u);
}

// Reductions over the 64 lanes of a wavefront; every lane gets the same result. Within a row of
// 16 lanes the values move through the DPP path of the vector ALU (lane swaps inside quads, then
// the mirrored half row and the mirrored row: after each step all lanes of the growing group hold
// the group's result, since the operation is commutative), the four row results are read as
// scalars. A shuffle through LDS (__shfl_xor, ds_bpermute) has several times the latency per step.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
constexpr int DPP_SWAP_1 = 0xB1;          // quad_perm:[1,0,3,2]
constexpr int DPP_SWAP_2 = 0x4E;          // quad_perm:[2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141;    // lane i <-> 7 - i within 8
constexpr int DPP_ROW_MIRROR = 0x140;     // lane i <-> 15 - i within 16
__device__ __forceinline__ float row_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
// Exchange between the rows of 16 lanes, on the vector ALU: gfx950's v_permlane16_swap exchanges the odd
// rows of its first operand with the even rows of its second, v_permlane32_swap the upper half of the
// first with the lower half of the second. Given the same value twice, the two results hold, in every
// lane, the lane's own value and that of lane ^ 16 (lane ^ 32), in an order that depends on the lane: a
// commutative operation on the pair is the exchange-and-combine step of a reduction, without the trip
// through LDS that __shfl_xor makes (ds_bpermute).
__device__ __forceinline__ void lane_pair_16(float v, float& a, float& b) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __builtin_bit_cast(float, static_cast<unsigned>(r[0]));
    b = __builtin_bit_cast(float, static_cast<unsigned>(r[1]));
}
__device__ __forceinline__ void lane_pair_32(float v, float& a, float& b) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    a = __builtin_bit_cast(float, static_cast<unsigned>(r[0]));
    b = __builtin_bit_cast(float, static_cast<unsigned>(r[1]));
}
// The value of lane (l ^ off) for off = 8, 16 or 32 on the vector ALU (a rotation by 8 within the row of 16
// lanes; the row swaps above and a select); other distances go through LDS. `off` is a constant once the
// caller's loop is unrolled.
constexpr int DPP_ROW_ROR_8 = 0x128;      // lane i <- lane (i + 8) % 16 of its row
__device__ __forceinline__ float lane_xor(float v, int off) {
    if (off == 8) return dpp_move<DPP_ROW_ROR_8>(v);
    if (off == 16 || off == 32) {
        float a, b;
        if (off == 16) lane_pair_16(v, a, b); else lane_pair_32(v, a, b);
        return (threadIdx.x & off) ? a : b;      // (wavefronts start at multiples of 64 threads)
    }
    return __shfl_xor(v, off, MLLM_WAVE);
}

// Maximum / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (one lane of each row), in all four.
__device__ __forceinline__ float rows_max(float v) {
    float a, b;
    lane_pair_16(v, a, b);
    v = fmaxf(a, b);
    lane_pair_32(v, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float rows_sum(float v) {
    float a, b;
    lane_pair_16(v, a, b);
    v = a + b;
    lane_pair_32(v, a, b);
    return a + b;
}

// Sum over aligned groups of LANES consecutive lanes (a power of two), in every lane of the group.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(LANES >= 1 && LANES <= MLLM_WAVE && (LANES & (LANES - 1)) == 0, "a power of two up to the wavefront");
    if (LANES >= 2) v += dpp_move<DPP_SWAP_1>(v);
    if (LANES >= 4) v += dpp_move<DPP_SWAP_2>(v);
    if (LANES >= 8) v += dpp_move<DPP_HALF_MIRROR>(v);
    if (LANES >= 16) v += dpp_move<DPP_ROW_MIRROR>(v);
    if (LANES >= 32) v += lane_xor(v, 16);
    if (LANES >= 64) v += lane_xor(v, 32);
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    static_assert(MLLM_WAVE == 64, "four rows of 16 lanes");
    v += dpp_move<DPP_SWAP_1>(v);
    v += dpp_move<DPP_SWAP_2>(v);
    v += dpp_move<DPP_HALF_MIRROR>(v);
    v += dpp_move<DPP_ROW_MIRROR>(v);
    return (row_lane(v, 0) + row_lane(v, 16)) + (row_lane(v, 32) + row_lane(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<DPP_SWAP_1>(v));
    v = fmaxf(v, dpp_move<DPP_SWAP_2>(v));
    v = fmaxf(v, dpp_move<DPP_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_move<DPP_ROW_MIRROR>(v));
    return fmaxf(fmaxf(row_lane(v, 0), row_lane(v, 16)), fmaxf(row_lane(v, 32), row_lane(v, 48)));
}

// Orders LDS traffic between the lanes of ONE wavefront (which run in lockstep):
// what lanes wrote before it is visible to all lanes after it.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every
// outstanding global load, which would drain the loads a kernel has deliberately in flight for
// a later tile; this one leaves them in flight (their registers are waited for where first used).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Block-wide sum for blocks of up to 1024 threads; `scratch` holds >= 16 floats of LDS.
// Every thread gets the result. Safe to call repeatedly with the same scratch.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int wave = threadIdx.x / MLLM_WAVE, lane = threadIdx.x % MLLM_WAVE;
    const int n_waves = (blockDim.x + MLLM_WAVE - 1) / MLLM_WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < n_waves; ++w) t += scratch[w];
    return t;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
    v = wave_max(v);
    const int wave = threadIdx.x / MLLM_WAVE, lane = threadIdx.x % MLLM_WAVE;
    const int n_waves = (blockDim.x + MLLM_WAVE - 1) / MLLM_WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = scratch[0];
    for (int w = 1; w < n_waves; ++w) t = fmaxf(t, scratch[w]);
    return t;
}

// GELU, tanh form: /root/reference/src/kernels/gelu.cu:7-9.
// 0.5 (1 + tanh u) = 1 / (1 + exp(-2u)): one hardware exponential and one reciprocal instead of the
// library's tanhf, which costs several times the rest of a product's epilogue. exp(-2u) = inf for
// very negative u gives v * 0, as the limit wants.
__device__ __forceinline__ float gelu_tanh(float v) {
    const float u = 0.7978845608f * (v + 0.044715f * v * v * v);
    return v * __builtin_amdgcn_rcpf(1.f + __expf(-2.f * u));
}
// The same in full 32-bit precision (library tanhf, no approximate reciprocal): the 32-bit path.
__device__ __forceinline__ float gelu_tanh_precise(float v) {
    const float u = 0.7978845608f * (v + 0.044715f * v * v * v);
    return 0.5f * v * (1.f + tanhf(u));
}
// GELU, exact form 0.5 v (1 + erf(v / sqrt 2)); the reference has only the tanh form.
__device__ __forceinline__ float gelu_erf(float v) {
    return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
}

// (a 32-bit output takes the full-precision activation: the 32-bit path has no fast approximations)
template <typename OutT>
__device__ __forceinline__ void epilogue(int mode, float acc, float bias, void* out, size_t idx) {
    float v = acc + bias;
    switch (mode) {
        case EPI_STORE: reinterpret_cast<OutT*>(out)[idx] = from_float<OutT>(v); break;
        case EPI_GELU_TANH:
            reinterpret_cast<OutT*>(out)[idx] = from_float<OutT>(sizeof(OutT) == 4 ? gelu_tanh_precise(v) : gelu_tanh(v));
            break;
        case EPI_GELU_ERF: reinterpret_cast<OutT*>(out)[idx] = from_float<OutT>(gelu_erf(v)); break;
        case EPI_ADD_RESIDUAL: reinterpret_cast<float*>(out)[idx] += v; break;
        default: reinterpret_cast<float*>(out)[idx] = v; break;
    }
}

#define MLLM_LAUNCH_CHECK()                                   \
    do {                                                      \
        hipError_t e_ = hipGetLastError();                    \
        if (e_ != hipSuccess) return static_cast<int>(e_);    \
    } while (0)

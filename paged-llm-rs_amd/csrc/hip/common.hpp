// Shared by every kernel file: element types, conversions, wave reductions and
// the error channel of the C interface.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define PL_DTYPE_F32 0
#define PL_DTYPE_BF16 1

#define PL_WAVE 64

// bfloat16 as its sixteen bits.
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) {
    return __uint_as_float(static_cast<uint32_t>(x.bits) << 16);
}

// Round-to-nearest-even through the hardware's conversion (v_cvt_pk_bf16_f32); a NaN stays a NaN.
__device__ __forceinline__ uint16_t bf16_bits_from_float(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

template <typename T>
__device__ __forceinline__ T from_float(float f);
template <>
__device__ __forceinline__ float from_float<float>(float f) {
    return f;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
    bf16_t r;
    r.bits = bf16_bits_from_float(f);
    return r;
}

// A value of one of two element types chosen at run time (norm gains may be
// stored wider than the activations).
__device__ __forceinline__ float load_as_float(const void* p, int dtype, size_t i) {
    return dtype == PL_DTYPE_F32 ? static_cast<const float*>(p)[i]
                                 : to_float(static_cast<const bf16_t*>(p)[i]);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = PL_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PL_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = PL_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, PL_WAVE));
    return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// The order of the additions is fixed by the thread layout alone.
__device__ __forceinline__ float block_sum(float v, float* scratch /* >= 16 floats of LDS */) {
    const int lane = threadIdx.x % PL_WAVE;
    const int wave = threadIdx.x / PL_WAVE;
    const int waves = (blockDim.x + PL_WAVE - 1) / PL_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < waves; ++w) total += scratch[w];
    return total;
}

// ---- the activation of a gated feed-forward's gate branch ------------------------
#define PL_ACT_SILU 0
#define PL_ACT_GELU_TANH 1
#define PL_ACT_GELU 2

// EXACT: the library's exponential (what the 32-bit path needs); otherwise the hardware's.  `act` is the
// same for a whole launch.
template <bool EXACT>
__device__ __forceinline__ float pl_activate(float g, int act) {
    if (act == PL_ACT_SILU) return g / (1.f + (EXACT ? expf(-g) : __expf(-g)));
    if (act == PL_ACT_GELU_TANH) return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    return 0.5f * g * (1.f + erff(g * 0.7071067811865476f));
}

// ---- the error channel -------------------------------------------------------
// Launchers return 0 or a negative code and leave a message for pl_last_error().
void pl_set_error(const char* fmt, ...);

// The compute units of the current device (launch-size choices go by it).
int pl_compute_units();

#define PL_REQUIRE(cond, ...)            \
    do {                                 \
        if (!(cond)) {                   \
            pl_set_error(__VA_ARGS__);   \
            return -1;                   \
        }                                \
    } while (0)

#define PL_CHECK_LAUNCH(name)                                                   \
    do {                                                                        \
        hipError_t e_ = hipGetLastError();                                      \
        if (e_ != hipSuccess) {                                                 \
            pl_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return -2;                                                          \
        }                                                                       \
    } while (0)

__host__ __device__ static inline int pl_ceil_div(int a, int b) { return (a + b - 1) / b; }

// Choosing the next token on the device.
#include "common.hpp"

// ---------------------------------------------------------------------------
// Greedy: the index of the largest logit of each row; the first maximum wins
// (ties go to the lower index), NaNs never win.  Two stages, so that a few rows
// over a vocabulary of a hundred and fifty thousand still fill the chip: every
// row is cut into ARGMAX_CHUNKS stretches whose winners a second kernel compares.
// ---------------------------------------------------------------------------
#define ARGMAX_CHUNKS 64

__device__ __forceinline__ void better(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) {
        bv = v;
        bi = i;
    }
}

__device__ __forceinline__ void block_best(float& bv, int& bi) {
    __shared__ float best_v[4];
    __shared__ int best_i[4];
#pragma unroll
    for (int off = PL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, PL_WAVE);
        const int oi = __shfl_xor(bi, off, PL_WAVE);
        better(bv, bi, ov, oi);
    }
    const int wave = threadIdx.x / PL_WAVE;
    if (threadIdx.x % PL_WAVE == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int w = 1; w < static_cast<int>(blockDim.x) / PL_WAVE; ++w) better(bv, bi, best_v[w], best_i[w]);
}

__global__ void __launch_bounds__(256)
argmax_stage1_kernel(const float* __restrict__ logits, float* __restrict__ part_v, int* __restrict__ part_i, int V) {
    const int row = blockIdx.y, chunk = blockIdx.x;
    const int per = (V + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
    const int begin = chunk * per, end = min(V, begin + per);
    const float* x = logits + static_cast<size_t>(row) * V;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) better(bv, bi, x[i], i);
    block_best(bv, bi);
    if (threadIdx.x == 0) {
        part_v[row * ARGMAX_CHUNKS + chunk] = bv;
        part_i[row * ARGMAX_CHUNKS + chunk] = bi;
    }
}

__global__ void __launch_bounds__(64)
argmax_stage2_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i, int* __restrict__ out) {
    const int row = blockIdx.x;
    float bv = part_v[row * ARGMAX_CHUNKS + threadIdx.x];
    int bi = part_i[row * ARGMAX_CHUNKS + threadIdx.x];
#pragma unroll
    for (int off = PL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, PL_WAVE);
        const int oi = __shfl_xor(bi, off, PL_WAVE);
        better(bv, bi, ov, oi);
    }
    if (threadIdx.x == 0) out[row] = bi == 0x7fffffff ? 0 : bi;
}

// scratch: m * 64 floats and m * 64 ints.
extern "C" int pl_argmax(const float* logits, int* out, float* scratch_v, int* scratch_i, int m, int V,
                         hipStream_t stream) {
    PL_REQUIRE(m >= 0 && V > 0 && m <= 65535, "argmax: rows %d, vocabulary %d", m, V);
    if (m == 0) return 0;
    static_assert(ARGMAX_CHUNKS == PL_WAVE, "the second stage is one wave a row");
    argmax_stage1_kernel<<<dim3(ARGMAX_CHUNKS, m), 256, 0, stream>>>(logits, scratch_v, scratch_i, V);
    PL_CHECK_LAUNCH("argmax");
    argmax_stage2_kernel<<<m, 64, 0, stream>>>(scratch_v, scratch_i, out);
    PL_CHECK_LAUNCH("argmax");
    return 0;
}

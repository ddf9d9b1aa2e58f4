// Choosing the next token on the device.
#include "common.hpp"

// ---------------------------------------------------------------------------
// Greedy: the index of the largest logit of each row; the first maximum wins
// (ties go to the lower index), NaNs never win.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V, size_t row_stride) {
    __shared__ float best_v[4];
    __shared__ int best_i[4];
    const float* row = logits + static_cast<size_t>(blockIdx.x) * row_stride;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float v = row[i];
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    }
#pragma unroll
    for (int off = PL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, PL_WAVE);
        const int oi = __shfl_xor(bi, off, PL_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    const int wave = threadIdx.x / PL_WAVE;
    if (threadIdx.x % PL_WAVE == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w) {
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        }
        out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
    }
}

extern "C" int pl_argmax(const float* logits, int* out, int m, int V, hipStream_t stream) {
    PL_REQUIRE(m >= 0 && V > 0, "argmax: rows %d, vocabulary %d", m, V);
    if (m == 0) return 0;
    argmax_kernel<<<m, 256, 0, stream>>>(logits, out, V, static_cast<size_t>(V));
    PL_CHECK_LAUNCH("argmax");
    return 0;
}

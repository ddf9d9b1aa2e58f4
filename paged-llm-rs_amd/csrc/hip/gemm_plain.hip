// y[n, N] = x[n, K] . w[N, K]^T with 32-bit multiply-add on the vector units.
//
// This is the matrix product of the true 32-bit path: no matrix-core mode, no
// reduced precision anywhere.  Each output element is the sum over k in
// ascending order, whatever n is, so a row's result does not depend on what
// else is in the batch.  The same kernel over bfloat16 inputs (products and
// sums in 32-bit) is the fallback for shapes the fast kernels refuse.
#include "common.hpp"

#define TILE_M 64
#define TILE_N 64
#define TILE_K 16

template <typename T, typename OUT>
__global__ void __launch_bounds__(256)
gemm_nt_kernel(const T* __restrict__ x, const T* __restrict__ w, OUT* __restrict__ y, int n, int N,
               int K, int ldx, int ldy) {
    // Tiles are stored k-major so that the inner loop reads consecutive LDS words.
    __shared__ float xs[TILE_K][TILE_M + 4];
    __shared__ float ws[TILE_K][TILE_N + 4];

    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * TILE_M;
    const int n0 = blockIdx.x * TILE_N;
    const int tx = tid % 16;  // 4 columns each
    const int ty = tid / 16;  // 4 rows each

    float acc[4][4] = {};

    for (int k0 = 0; k0 < K; k0 += TILE_K) {
        // 64 rows x 16 k = 1024 elements per tile, 4 per thread.
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + i * 256;
            const int r = e / TILE_K;
            const int k = e % TILE_K;
            const int gm = m0 + r, gn = n0 + r, gk = k0 + k;
            xs[k][r] = (gm < n && gk < K) ? to_float(x[static_cast<size_t>(gm) * ldx + gk]) : 0.f;
            ws[k][r] = (gn < N && gk < K) ? to_float(w[static_cast<size_t>(gn) * K + gk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TILE_K; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + ty * 4 + i;
        if (gm >= n) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx * 4 + j;
            if (gn < N) y[static_cast<size_t>(gm) * ldy + gn] = from_float<OUT>(acc[i][j]);
        }
    }
}

// dtype: element type of x and w.  out_f32: write y as 32-bit floats whatever dtype is.
extern "C" int pl_gemm_plain(const void* x, const void* w, void* y, int n, int N, int K, int ldx,
                             int ldy, int dtype, int out_f32, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && N > 0 && K > 0 && ldx >= K && ldy >= N,
               "gemm: %d x %d x %d with row strides %d and %d", n, N, K, ldx, ldy);
    if (n == 0) return 0;
    dim3 grid(pl_ceil_div(N, TILE_N), pl_ceil_div(n, TILE_M));
    PL_REQUIRE(grid.y <= 65535, "gemm: %d rows are more than one launch covers", n);
    if (dtype == PL_DTYPE_F32) {
        gemm_nt_kernel<float, float><<<grid, 256, 0, stream>>>(
            static_cast<const float*>(x), static_cast<const float*>(w), static_cast<float*>(y), n, N, K, ldx, ldy);
    } else if (dtype == PL_DTYPE_BF16) {
        if (out_f32)
            gemm_nt_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(
                static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<float*>(y), n, N, K, ldx, ldy);
        else
            gemm_nt_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>(
                static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(y), n, N, K, ldx, ldy);
    } else {
        PL_REQUIRE(false, "gemm: dtype code %d", dtype);
    }
    PL_CHECK_LAUNCH("gemm_plain");
    return 0;
}

// y[n, N] = x[n, K] . w[N, K]^T for few rows (n <= 64), bfloat16 in, 32-bit accumulate,
// on the matrix cores.
//
// With few rows the product is a stream of the weight matrix through the chip:
// every weight is read once and the time is the time of that read.  One
// workgroup of four waves owns 16 output columns (16 rows of w); the waves split
// K between them so that the whole matrix is in flight at once, and their partial
// tiles are added in a fixed order through LDS.  Each wave feeds
// v_mfma_f32_16x16x32_bf16 straight from global memory: both operands are
// contiguous along K, so a lane's 16 bytes are one load.
//
// Epilogues: a plain store (bfloat16 or 32-bit), or SwiGLU, where the workgroup
// owns 16 gate columns and the 16 up columns that belong to them and stores
// silu(gate) * up.
#include "common.hpp"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define SK_TILE_N 16
#define SK_WAVES 4
#define SK_KSTEP 32

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) {
    return *reinterpret_cast<const bf16x8*>(p);
}

__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    return z;
}

// MT: 16-row tiles of x (n <= 16*MT).  SWIGLU: two weight tiles, gate at column c and up at column N_out + c.
template <int MT, int UNR, bool SWIGLU, typename OUT>
__global__ void __launch_bounds__(256)
gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, OUT* __restrict__ y, int n,
                   int N_out, int K) {
    constexpr int BT = SWIGLU ? 2 : 1;
    __shared__ float red[SK_WAVES][BT][MT][256];

    const int lane = threadIdx.x % PL_WAVE;
    const int wave = threadIdx.x / PL_WAVE;
    const int c = lane % 16;  // column of the tile (a row of w), and the row of x inside its tile
    const int g = lane / 16;  // which 8 of the 32 values of a K step
    const int n0 = blockIdx.x * SK_TILE_N;

    // K is cut into four stretches of whole steps.
    const int steps = (K + SK_KSTEP - 1) / SK_KSTEP;
    const int per_wave = (steps + SK_WAVES - 1) / SK_WAVES;
    const int kbeg = wave * per_wave * SK_KSTEP;
    const int kend = min(K, (wave + 1) * per_wave * SK_KSTEP);

    const bool col_ok = n0 + c < N_out;
    const bf16_t* wrow[BT];
    wrow[0] = w + static_cast<size_t>(n0 + c) * K;
    if (SWIGLU) wrow[BT - 1] = w + static_cast<size_t>(N_out + n0 + c) * K;

    f32x4 acc[BT][MT];
#pragma unroll
    for (int b = 0; b < BT; ++b)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[b][m] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int k0 = kbeg; k0 < kend; k0 += SK_KSTEP * UNR) {
        bf16x8 bw[BT][UNR];
        bf16x8 ax[MT][UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int kk = k0 + u * SK_KSTEP + g * 8;
            const bool k_ok = kk < kend;  // K is a multiple of 8, so a chunk is whole or absent
#pragma unroll
            for (int b = 0; b < BT; ++b) bw[b][u] = (k_ok && col_ok) ? load8(wrow[b] + kk) : zero8();
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = m * 16 + c;
                ax[m][u] = (k_ok && row < n) ? load8(x + static_cast<size_t>(row) * K + kk) : zero8();
            }
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u)
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int b = 0; b < BT; ++b)
                    acc[b][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[m][u], bw[b][u], acc[b][m], 0, 0, 0);
    }

    // A lane holds rows (lane/16)*4 + i, i = 0..3, of column lane%16 of its 16x16 tile.
#pragma unroll
    for (int b = 0; b < BT; ++b)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][b][m][lane * 4 + i] = acc[b][m][i];
    __syncthreads();

    const int t = threadIdx.x;
    const int src_lane = t / 4, i = t % 4;
    const int row_in_tile = (src_lane / 16) * 4 + i;
    const int col = n0 + src_lane % 16;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int row = m * 16 + row_in_tile;
        float v[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            float s = 0.f;
#pragma unroll
            for (int wv = 0; wv < SK_WAVES; ++wv) s += red[wv][b][m][t];
            v[b] = s;
        }
        if (row < n && col < N_out) {
            float r = v[0];
            if (SWIGLU) r = v[0] / (1.f + __expf(-v[0])) * v[BT - 1];
            y[static_cast<size_t>(row) * N_out + col] = from_float<OUT>(r);
        }
    }
}

template <int MT, int UNR, bool SWIGLU>
static int launch_skinny(const void* x, const void* w, void* y, int n, int N_out, int K, int out_f32,
                         hipStream_t stream) {
    const int grid = pl_ceil_div(N_out, SK_TILE_N);
    if (out_f32)
        gemm_skinny_kernel<MT, UNR, SWIGLU, float><<<grid, 256, 0, stream>>>(
            static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<float*>(y), n, N_out, K);
    else
        gemm_skinny_kernel<MT, UNR, SWIGLU, bf16_t><<<grid, 256, 0, stream>>>(
            static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<bf16_t*>(y), n, N_out, K);
    PL_CHECK_LAUNCH("gemm_skinny");
    return 0;
}

// y = x . w^T (swiglu 0, w is [N_out, K]) or y = silu(x . wg^T) * (x . wu^T) (swiglu 1, w is [2*N_out, K],
// gate rows first).  bfloat16 x and w; y is bfloat16 or, with out_f32, 32-bit.
extern "C" int pl_gemm_skinny(const void* x, const void* w, void* y, int n, int N_out, int K, int swiglu,
                              int out_f32, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && n <= 64, "skinny product: %d rows, it takes up to 64", n);
    PL_REQUIRE(N_out > 0 && K > 0 && K % 8 == 0, "skinny product: %d columns, inner width %d (a multiple of 8 is needed)", N_out, K);
    if (n == 0) return 0;
    const int mt = pl_ceil_div(n, 16);
    if (swiglu) {
        switch (mt) {
            case 1: return launch_skinny<1, 4, true>(x, w, y, n, N_out, K, out_f32, stream);
            case 2: return launch_skinny<2, 2, true>(x, w, y, n, N_out, K, out_f32, stream);
            case 3: return launch_skinny<3, 2, true>(x, w, y, n, N_out, K, out_f32, stream);
            default: return launch_skinny<4, 2, true>(x, w, y, n, N_out, K, out_f32, stream);
        }
    }
    switch (mt) {
        case 1: return launch_skinny<1, 8, false>(x, w, y, n, N_out, K, out_f32, stream);
        case 2: return launch_skinny<2, 4, false>(x, w, y, n, N_out, K, out_f32, stream);
        case 3: return launch_skinny<3, 2, false>(x, w, y, n, N_out, K, out_f32, stream);
        default: return launch_skinny<4, 2, false>(x, w, y, n, N_out, K, out_f32, stream);
    }
}

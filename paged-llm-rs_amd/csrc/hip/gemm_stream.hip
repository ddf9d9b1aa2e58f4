// y[n, N] = x[n, K] . w[N, K]^T for up to 64 rows over a large weight matrix: bfloat16 in, 32-bit sums on the
// matrix cores.
//
// With so few rows the product is one pass of the weights through the chip, and a matrix of tens or hundreds of
// megabytes is long enough for the rate of that pass to be all that counts.  What the rate needs is that every
// compute unit always has tens of kilobytes on their way, and that x, which every workgroup needs whole, costs
// little beside the weights.  So a workgroup (four waves) owns 128 rows of w, 32 a wave, and a stretch of K; it
// walks the stretch in chunks of 128.  A wave's weights go from memory straight into its registers, laid out
// as v_mfma_f32_16x16x32_bf16 wants them (a lane's 16 bytes are one load); two chunks' worth of registers take
// turns, so the chunk after the one being multiplied is always in flight.  The chunk of x (64 rows at most)
// goes through LDS, where all four waves read it: the workgroup fetches n/128 bytes of x a byte of w, and
// from the L2.  One barrier a chunk.
//
// A matrix with few rows (a projection back to the width of the model) has too few stretches of 128 rows for
// the chip; then K is split between workgroups as well, every workgroup leaves its 32-bit partial tile in a
// workspace and a second small kernel adds the partial tiles in a fixed order and does what follows the
// product.  What follows (as the last stage here, or in that second kernel): store (bfloat16 or 32-bit),
// act(gate) * up over rows j and N + j of a stacked weight, or the sum into the 32-bit residual stream.
#include "common.hpp"

typedef __bf16 gs_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gs_f32x4 __attribute__((ext_vector_type(4)));

struct __attribute__((aligned(16))) gs_u32x4 {
    uint32_t v[4];
};

#define GS_WAVES 4
#define GS_BK 128                 // elements of K a chunk
#define GS_XROW (GS_BK + 8)       // a row of x in LDS: 16 rows, 16 bytes each, then fall on all 64 banks
#define GS_MAX_ROWS 64
#define GS_MAX_SPLITS 16

#define GS_STORE_BF16 0
#define GS_STORE_F32 1
#define GS_SWIGLU 2
#define GS_ADD 3
#define GS_PARTIAL 4

// MT: 16-row tiles of x.  MODE: what follows the product.  WV: waves a workgroup.  blockIdx.x: the stretch of rows of w (columns of
// y), blockIdx.y: the stretch of K.  Nw: rows of w (twice N_out for GS_SWIGLU).
template <int MT, int MODE, int WV>
__global__ void __launch_bounds__(64 * WV)
gemm_stream_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ y_,
                   float* __restrict__ ws, int n, int N_out, int Nw, int K, int act, int chunks_per_split) {
    __shared__ __attribute__((aligned(16))) bf16_t xs[2][MT * 16 * GS_XROW];
    const int tid = threadIdx.x;
    const int lane = tid % PL_WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / PL_WAVE);
    const int c = lane % 16, g = lane / 16;

    // the wave's two tiles of 16 rows of w
    int wrow[2];
    int col0;   // first column of y of the wave's first tile
    if constexpr (MODE == GS_SWIGLU) {
        col0 = (blockIdx.x * WV + wave) * 16;
        const int j = min(col0 + c, N_out - 1);
        wrow[0] = j;
        wrow[1] = N_out + j;
    } else {
        col0 = (blockIdx.x * WV + wave) * 32;
        wrow[0] = min(col0 + c, Nw - 1);
        wrow[1] = min(col0 + 16 + c, Nw - 1);
    }
    const bf16_t* wp[2] = {w + static_cast<size_t>(wrow[0]) * K + g * 8, w + static_cast<size_t>(wrow[1]) * K + g * 8};

    // The stretch of chunks of this workgroup.  Only the last chunk of a K that is no multiple of 128 has a
    // part past K; it is done after the others, with loads that look where they read.
    const int nchunks = pl_ceil_div(K, GS_BK);
    const int c_lo = blockIdx.y * chunks_per_split;
    const int c_hi = min(nchunks, c_lo + chunks_per_split);
    const int count = min(c_hi, K / GS_BK) - c_lo;     // whole chunks
    const bool ragged = c_hi > K / GS_BK;

    // a thread's share of a chunk of x: rows p*XR + tid/16, 16 bytes at element 8 (tid%16) of the chunk
    constexpr int XR = 4 * WV;                          // rows of x the workgroup's threads cover at once
    constexpr int XP = (MT * 16 + XR - 1) / XR;         // turns a thread takes
    const int xpiece = tid % 16, xr = tid / 16;
    const bf16_t* xp[XP];
#pragma unroll
    for (int p = 0; p < XP; ++p) xp[p] = x + static_cast<size_t>(min(p * XR + xr, n - 1)) * K + xpiece * 8;

    auto ask_w = [&](int ci, gs_u32x4* buf) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < 4; ++s) buf[t * 4 + s] = *reinterpret_cast<const gs_u32x4*>(wp[t] + ci * GS_BK + s * 32);
    };
    auto ask_x = [&](int ci, gs_u32x4* stage) {
#pragma unroll
        for (int p = 0; p < XP; ++p) stage[p] = *reinterpret_cast<const gs_u32x4*>(xp[p] + ci * GS_BK);
    };
    auto put_x = [&](int buf, const gs_u32x4* stage) {
#pragma unroll
        for (int p = 0; p < XP; ++p)
            if (XP * XR == MT * 16 || p * XR + xr < MT * 16)
                *reinterpret_cast<gs_u32x4*>(&xs[buf][(p * XR + xr) * GS_XROW + xpiece * 8]) = stage[p];
    };

    gs_f32x4 acc[2][MT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[t][m] = gs_f32x4{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](int buf, const gs_u32x4* wb) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            gs_bf16x8 a[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m)
                a[m] = *reinterpret_cast<const gs_bf16x8*>(&xs[buf][(m * 16 + c) * GS_XROW + s * 32 + g * 8]);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const gs_bf16x8 b = __builtin_bit_cast(gs_bf16x8, wb[t * 4 + s]);
#pragma unroll
                for (int m = 0; m < MT; ++m) acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[m], b, acc[t][m], 0, 0, 0);
            }
        }
    };

    // x of a chunk is asked for before the chunk's weights, so that waiting for it leaves the weights in flight.
    // In the loop nothing is conditional: chunk i is multiplied out of (xs[0], wa) while chunk i+1 is on its
    // way into (stage, wb), and chunk i+2 is asked for as soon as wa is free.
    // (The loop can only be reached with both chunks asked for: where paths with fewer loads in flight join
    // it, the compiler places its waits for the fewest, and the queue of loads runs dry once a round.)
    gs_u32x4 wa[8], wb[8], stage[XP];
    if (count >= 2) {
        ask_x(c_lo, stage);
        ask_w(c_lo, wa);
        put_x(0, stage);
        ask_x(c_lo + 1, stage);
        ask_w(c_lo + 1, wb);
        __syncthreads();
        int i = 0;
        for (; i + 3 < count; i += 2) {
            multiply(0, wa);
            put_x(1, stage);
            ask_x(c_lo + i + 2, stage);
            ask_w(c_lo + i + 2, wa);
            __syncthreads();
            multiply(1, wb);
            put_x(0, stage);
            ask_x(c_lo + i + 3, stage);
            ask_w(c_lo + i + 3, wb);
            __syncthreads();
        }
        // two or three chunks are left: chunk i is ready, chunk i+1 on its way
        const bool third = i + 2 < count;
        multiply(0, wa);
        put_x(1, stage);
        if (third) {
            ask_x(c_lo + i + 2, stage);
            ask_w(c_lo + i + 2, wa);
        }
        __syncthreads();
        multiply(1, wb);
        if (third) {
            put_x(0, stage);
            __syncthreads();
            multiply(0, wa);
        }
    } else if (count == 1) {
        ask_x(c_lo, stage);
        ask_w(c_lo, wa);
        put_x(0, stage);
        __syncthreads();
        multiply(0, wa);
    }
    if (ragged) {
        const int k0 = (K / GS_BK) * GS_BK;
        __syncthreads();        // whoever still reads xs[0]
        const bool x_in = k0 + xpiece * 8 < K;
#pragma unroll
        for (int p = 0; p < XP; ++p) {
            // (a lane whose piece lies past K reads the start of its row instead: K is 8 at least)
            const gs_u32x4 got = *reinterpret_cast<const gs_u32x4*>(xp[p] + (x_in ? k0 : -xpiece * 8));
#pragma unroll
            for (int e = 0; e < 4; ++e) stage[p].v[e] = x_in ? got.v[e] : 0u;
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const bool in = k0 + s * 32 + g * 8 < K;
                const gs_u32x4 got = *reinterpret_cast<const gs_u32x4*>(wp[t] + (in ? k0 + s * 32 : -g * 8));
#pragma unroll
                for (int e = 0; e < 4; ++e) wa[t * 4 + s].v[e] = in ? got.v[e] : 0u;
            }
        put_x(0, stage);
        __syncthreads();
        multiply(0, wa);
    }

    // A lane holds rows m*16 + g*4 + i, i = 0..3, of column c of each of its tiles.
#pragma unroll
    for (int m = 0; m < MT; ++m) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = m * 16 + g * 4 + i;
            if (row >= n) continue;
            if constexpr (MODE == GS_SWIGLU) {
                const int col = col0 + c;
                if (col < N_out)
                    static_cast<bf16_t*>(y_)[static_cast<size_t>(row) * N_out + col] =
                        from_float<bf16_t>(pl_activate<false>(acc[0][m][i], act) * acc[1][m][i]);
            } else {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int col = col0 + t * 16 + c;
                    if (col >= Nw) continue;
                    const float v = acc[t][m][i];
                    if constexpr (MODE == GS_PARTIAL) {
                        ws[(static_cast<size_t>(blockIdx.y) * n + row) * Nw + col] = v;
                    } else if constexpr (MODE == GS_STORE_BF16) {
                        static_cast<bf16_t*>(y_)[static_cast<size_t>(row) * N_out + col] = from_float<bf16_t>(v);
                    } else if constexpr (MODE == GS_STORE_F32) {
                        static_cast<float*>(y_)[static_cast<size_t>(row) * N_out + col] = v;
                    } else {
                        static_cast<float*>(y_)[static_cast<size_t>(row) * N_out + col] += v;
                    }
                }
            }
        }
    }
}

// Adds the partial tiles of the stretches of K, in their order, and does what follows the product.
// A thread takes V neighbouring columns of a row (V = 4 where the width allows 16-byte loads, else 1), and
// for GS_SWIGLU the gate's and the up's.
template <int MODE, int V>
__global__ void __launch_bounds__(256)
gemm_stream_finish_kernel(const float* __restrict__ ws, void* __restrict__ y_, int n, int N_out, int Nw, int splits, int act) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int groups = N_out / V;                       // (V divides N_out)
    if (idx >= static_cast<size_t>(n) * groups) return;
    const int row = static_cast<int>(idx / groups), col = static_cast<int>(idx - static_cast<size_t>(row) * groups) * V;
    float first[V], second[V];
#pragma unroll
    for (int e = 0; e < V; ++e) first[e] = second[e] = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* at = ws + (static_cast<size_t>(s) * n + row) * Nw;
        if constexpr (V == 4) {
            const gs_f32x4 a = *reinterpret_cast<const gs_f32x4*>(at + col);
#pragma unroll
            for (int e = 0; e < 4; ++e) first[e] += a[e];
            if constexpr (MODE == GS_SWIGLU) {
                const gs_f32x4 b = *reinterpret_cast<const gs_f32x4*>(at + N_out + col);
#pragma unroll
                for (int e = 0; e < 4; ++e) second[e] += b[e];
            }
        } else {
            first[0] += at[col];
            if constexpr (MODE == GS_SWIGLU) second[0] += at[N_out + col];
        }
    }
    const size_t out = static_cast<size_t>(row) * N_out + col;
    if constexpr (V == 4 && (MODE == GS_ADD || MODE == GS_STORE_F32)) {
        // (16-byte aligned: the launcher looked at y as it looked at ws)
        gs_f32x4* to = reinterpret_cast<gs_f32x4*>(static_cast<float*>(y_) + out);
        gs_f32x4 v = {first[0], first[1], first[2], first[3]};
        if constexpr (MODE == GS_ADD) v += *to;
        *to = v;
        return;
    }
#pragma unroll
    for (int e = 0; e < V; ++e) {
        if constexpr (MODE == GS_SWIGLU) static_cast<bf16_t*>(y_)[out + e] = from_float<bf16_t>(pl_activate<false>(first[e], act) * second[e]);
        else if constexpr (MODE == GS_STORE_BF16) static_cast<bf16_t*>(y_)[out + e] = from_float<bf16_t>(first[e]);
        else if constexpr (MODE == GS_STORE_F32) static_cast<float*>(y_)[out + e] = first[e];
        else static_cast<float*>(y_)[out + e] += first[e];
    }
}

// mode: one of GS_STORE_BF16, GS_STORE_F32, GS_SWIGLU, GS_ADD.
static void gs_finish(const float* ws, void* y, int n, int N_out, int Nw, int splits, int mode, int act, hipStream_t stream) {
    const bool wide = N_out % 4 == 0 && Nw % 4 == 0 && reinterpret_cast<uintptr_t>(ws) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
    const int blocks = static_cast<int>((static_cast<size_t>(n) * (N_out / (wide ? 4 : 1)) + 255) / 256);
#define GS_FINISH(MODE)                                                                                              \
    do {                                                                                                             \
        if (wide) gemm_stream_finish_kernel<MODE, 4><<<blocks, 256, 0, stream>>>(ws, y, n, N_out, Nw, splits, act);  \
        else gemm_stream_finish_kernel<MODE, 1><<<blocks, 256, 0, stream>>>(ws, y, n, N_out, Nw, splits, act);       \
    } while (0)
    switch (mode) {
        case GS_STORE_BF16: GS_FINISH(GS_STORE_BF16); break;
        case GS_STORE_F32: GS_FINISH(GS_STORE_F32); break;
        case GS_SWIGLU: GS_FINISH(GS_SWIGLU); break;
        default: GS_FINISH(GS_ADD); break;
    }
#undef GS_FINISH
}

static int gs_column_groups(int N_out, bool swiglu, int waves = GS_WAVES) { return swiglu ? pl_ceil_div(N_out, 16 * waves) : pl_ceil_div(N_out, 32 * waves); }

// Into how many stretches K is cut.  A compute unit takes in only so many bytes a microsecond, however many
// workgroups it runs (about 20 GB/s measured, 5 TB/s over the chip), so the pass is as fast as the chip
// only if every compute unit has the same share of it: the workgroups of a launch mostly run at once, and
// with 1.5 of them a compute unit half the chip has twice the work of the other half (51,200 rows of
// 5,120: 400 workgroups, 4.2 TB/s; 65,536 rows: 512 workgroups, 5.0 TB/s).  More stretches make the shares
// more even, but every stretch beyond the first writes and reads its partial tiles, n x (rows of w) floats.
// The count with the smallest estimate of (bytes moved) / (evenness) is taken.
extern "C" int pl_gemm_stream_splits(int n, int N_out, int K, int swiglu) {
    if (n <= 0 || N_out <= 0 || K <= 0) return 1;
    const long long units = pl_compute_units();
    const long long Nw = static_cast<long long>(N_out) * (swiglu ? 2 : 1);
    const int nchunks = pl_ceil_div(K, GS_BK);
    const double weights = static_cast<double>(Nw) * K * 2;
    int best = 1;
    double best_cost = 0;
    for (int splits = 1; splits <= GS_MAX_SPLITS; ++splits) {
        const int per_split = pl_ceil_div(nchunks, splits);
        if (splits > 1 && per_split < 4) break;
        const int parts = pl_ceil_div(nchunks, per_split);
        if (parts != splits) continue;                       // the same launch as a smaller count
        const long long groups = splits > 1 ? (Nw + 32 * GS_WAVES - 1) / (32 * GS_WAVES) : gs_column_groups(N_out, swiglu != 0);
        const long long workgroups = groups * parts;
        const long long rounds = (workgroups + units - 1) / units;
        const double even = static_cast<double>(workgroups) / (static_cast<double>(rounds) * units);
        // (the second kernel's launch counts as the bytes that three microseconds move)
        const double moved = weights + (splits > 1 ? 2.0 * splits * n * static_cast<double>(Nw) * 4 + 1.5e7 : 0.0);
        const double cost = moved / even;
        if (splits == 1 || cost < best_cost) {
            best = splits;
            best_cost = cost;
        }
    }
    return best;
}

template <int MT, int WV>
static int gs_launch(const bf16_t* x, const bf16_t* w, void* y, float* ws, int n, int N_out, int K, int mode, int act,
                     int splits, hipStream_t stream) {
    const bool swiglu = mode == GS_SWIGLU;
    const int Nw = swiglu ? 2 * N_out : N_out;
    const int nchunks = pl_ceil_div(K, GS_BK);
    const int per_split = pl_ceil_div(nchunks, splits);
    const dim3 grid(gs_column_groups(N_out, swiglu && splits == 1, WV), pl_ceil_div(nchunks, per_split));
#define GS_GO(MODE) gemm_stream_kernel<MT, MODE, WV><<<grid, 64 * WV, 0, stream>>>(x, w, y, ws, n, N_out, Nw, K, act, per_split)
    if (splits > 1) {
        // as a plain product over all rows of w; the second kernel pairs gate and up
        gemm_stream_kernel<MT, GS_PARTIAL, WV><<<dim3(pl_ceil_div(Nw, 32 * WV), grid.y), 64 * WV, 0, stream>>>(
            x, w, y, ws, n, Nw, Nw, K, act, per_split);
        PL_CHECK_LAUNCH("gemm_stream");
        gs_finish(ws, y, n, N_out, Nw, static_cast<int>(grid.y), mode, act, stream);
        PL_CHECK_LAUNCH("gemm_stream_finish");
        return 0;
    }
    switch (mode) {
        case GS_STORE_BF16: GS_GO(GS_STORE_BF16); break;
        case GS_STORE_F32: GS_GO(GS_STORE_F32); break;
        case GS_SWIGLU: GS_GO(GS_SWIGLU); break;
        default: GS_GO(GS_ADD); break;
    }
#undef GS_GO
    PL_CHECK_LAUNCH("gemm_stream");
    return 0;
}

// x: bfloat16 [n, K], n <= 64; w: bfloat16 [N_out, K] ([2 N_out, K], gate rows then up rows, for epilogue 1);
// K a multiple of 8.  epilogue 0: y [n, N_out], bfloat16 or (out_f32) 32-bit; 1: y = act(gate) * up, bfloat16;
// 2: y is the 32-bit residual stream and takes the sum.  splits: the stretches of K (pl_gemm_stream_splits
// says how many pay); with more than one, ws holds splits * n * (rows of w) floats.
extern "C" int pl_gemm_stream(const void* x, const void* w, void* y, float* ws, int n, int N_out, int K, int epilogue,
                              int out_f32, int act, int splits, hipStream_t stream) {
    PL_REQUIRE(n > 0 && n <= GS_MAX_ROWS && N_out > 0 && K > 0 && K % 8 == 0,
               "streamed product: %d rows (64 at most), %d columns, a width of %d (a multiple of 8)", n, N_out, K);
    PL_REQUIRE(epilogue >= 0 && epilogue <= 2, "streamed product: epilogue %d", epilogue);
    PL_REQUIRE(splits >= 1 && splits <= GS_MAX_SPLITS && (splits == 1 || ws != nullptr),
               "streamed product: %d stretches of K (%d at most), which need a workspace", splits, GS_MAX_SPLITS);
    PL_REQUIRE(act == PL_ACT_SILU || act == PL_ACT_GELU_TANH || act == PL_ACT_GELU, "streamed product: activation code %d", act);
    PL_REQUIRE(static_cast<long long>(N_out) * (epilogue == 1 ? 2 : 1) <= 0x7fffffffLL / 2, "streamed product: %d columns", N_out);
    const int mode = epilogue == 1 ? GS_SWIGLU : (epilogue == 2 ? GS_ADD : (out_f32 ? GS_STORE_F32 : GS_STORE_BF16));
    const bf16_t* xb = static_cast<const bf16_t*>(x);
    const bf16_t* wb = static_cast<const bf16_t*>(w);
    // (Eight waves a workgroup, 256 rows of w, were no faster at any size measured.)
    if (n <= 16) return gs_launch<1, GS_WAVES>(xb, wb, y, ws, n, N_out, K, mode, act, splits, stream);
    if (n <= 32) return gs_launch<2, GS_WAVES>(xb, wb, y, ws, n, N_out, K, mode, act, splits, stream);
    if (n <= 48) return gs_launch<3, GS_WAVES>(xb, wb, y, ws, n, N_out, K, mode, act, splits, stream);
    return gs_launch<4, GS_WAVES>(xb, wb, y, ws, n, N_out, K, mode, act, splits, stream);
}

// The second kernel alone, for partial products that came from elsewhere (a deep product of some hundred
// rows that the library ran as a batch of stretches of K): ws is 32-bit [splits, n, N_out] (for epilogue 1
// [splits, n, 2 N_out], gate columns then up columns); the partial results are added in their order and
// stored (epilogue 0: bfloat16 or, out_f32, 32-bit; 1: act(gate) * up, bfloat16) or added into the 32-bit
// residual stream y (epilogue 2).  Any number of rows.
extern "C" int pl_gemm_finish(const float* ws, void* y, long long n, int N_out, int splits, int epilogue, int out_f32,
                              int act, hipStream_t stream) {
    PL_REQUIRE(n > 0 && N_out > 0 && splits >= 1 && splits <= 64 && ws != nullptr && y != nullptr,
               "sum of partial products: %lld rows, %d columns, %d parts", n, N_out, splits);
    PL_REQUIRE(epilogue >= 0 && epilogue <= 2, "sum of partial products: epilogue %d", epilogue);
    PL_REQUIRE(act == PL_ACT_SILU || act == PL_ACT_GELU_TANH || act == PL_ACT_GELU, "sum of partial products: activation code %d", act);
    PL_REQUIRE(n * N_out < (1ll << 31) * 256 && n <= 0x7fffffff, "sum of partial products: %lld x %d results", n, N_out);
    const int Nw = epilogue == 1 ? 2 * N_out : N_out;
    const int mode = epilogue == 1 ? GS_SWIGLU : (epilogue == 2 ? GS_ADD : (out_f32 ? GS_STORE_F32 : GS_STORE_BF16));
    gs_finish(ws, y, static_cast<int>(n), N_out, Nw, splits, mode, act, stream);
    PL_CHECK_LAUNCH("gemm_stream_finish");
    return 0;
}

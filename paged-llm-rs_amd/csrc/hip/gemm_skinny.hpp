// y[n, N] = x[n, K] . w[N, K]^T for few rows (n <= 64), bfloat16 weights, 32-bit accumulate,
// on the matrix cores, with what comes before and after the product fused into it.
//
// With few rows the product is a stream of the weight matrix through the chip:
// every weight is read once and the time is the time of that read, which is the
// time of one trip to memory if the whole matrix is asked for at once.  One
// workgroup of four waves owns 16 output columns (16 rows of w); the waves split
// K between them and each asks for its whole share before it multiplies, and
// their partial tiles are added in a fixed order through LDS.  Each wave feeds
// v_mfma_f32_16x16x32_bf16 straight from global memory: both operands are
// contiguous along K, so a lane's 16 bytes are one load.
//
// Before the product (PRO):
//   PRO_BF16  x is bfloat16 [n, K].
//   PRO_NORM  x is the 32-bit residual stream; row r of the product reads row rows[r] of it (or r).
//             The product runs over bf16(x * gain) and the result is scaled by
//             1 / sqrt(mean(x^2) + eps) of its row afterwards: the statistic is summed from the
//             very values the product loads, so the norm costs no pass of its own.
// After the product (EPI):
//   EPI_STORE   y = result (bfloat16 or 32-bit).
//   EPI_SWIGLU  the workgroup owns 16 gate columns and the 16 up columns that belong to
//               them (rows c and N + c of w) and stores silu(gate) * up.
//   EPI_ADD     the 32-bit residual stream takes the result: resid[r, c] += result.  Every
//               element has one owner, so the sum does not depend on timing.
//
// The norm handed forward.  A product that adds into the stream (EPI_ADD) owns whole 16-column stripes of
// the updated stream, so it can leave the next norm's work behind: bf16(stream * gain) for its stripe, and
// for every row the sum of squares over the stripe.  The product behind that norm then loads bfloat16 rows
// (half the bytes of the stream, nothing to convert or square), adds the stripes' sums in a fixed order and
// scales its result by 1 / sqrt(sum / K + eps), which is where PRO_NORM applies the statistic as well.
//
// With more than 16 rows a wave's registers fill with x (every 16 rows are another operand a K step), and
// little of w is on its way at a time.  PANEL then brings the workgroup's 16 (or 32) rows of w into LDS
// first: every wave asks for its share with loads that write LDS themselves (global_load_lds_dwordx4), so
// the whole panel is on its way at once at no cost in registers, and the matrix cores take w from LDS
// (16-byte pieces permuted within a row, piece p of row r at p ^ (r & 15), so that the 16 rows a read
// touches fall on different banks).  K has to be a multiple of 512: a load of one wave fills 1 KB of a row.
#pragma once
#include "common.hpp"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));

#define SK_TILE_N 16
#define SK_KSTEP 32

#define PRO_BF16 0
#define PRO_NORM 1
#define EPI_STORE 0
#define EPI_SWIGLU 1
#define EPI_ADD 2

struct __attribute__((aligned(16))) sk_f32x4 {
    float v[4];
};
struct __attribute__((aligned(16))) sk_u32x4 {
    uint32_t v[4];
};

// What a launch carries beside its operands: a norm handed forward (see above; all null: none is), and how
// the weights are laid out.  (The kernels' parameter of this type is still called `hand`.)
struct sk_extras_t {
    // from a product that adds into the stream: the next norm's gains [N_out]; x [n, N_out] takes
    // bf16(stream * gain) and ssq [n, column tiles] the stripes' sums of squares
    const float* gain;
    bf16_t* x;
    float* ssq;
    // to a product of bfloat16 rows that such a product left: their stripes' sums of squares [n, count]
    const float* parts;
    int count;
    // w holds the weights in strips (see "Weights in strips" below)
    int strips;
    // the K steps a wave of the launch takes (ceil(steps / waves): the launch knows both, and a division by a number
    // the kernel learns only when it runs is some thirty instructions in front of its first loads); 0: not said
    int steps_a_wave;
};

static inline sk_extras_t sk_with_steps(sk_extras_t extras, int K, int waves) {
    extras.steps_a_wave = pl_ceil_div(pl_ceil_div(K, 32), waves);
    return extras;
}

// Weights in strips.  Read as [N][K], a wave's load of a K step fetches 64 bytes from each of 16 rows of w that
// lie K elements apart; the memory gives a pass of such loads less than it gives one that reads front to back
// (a 201 MB matrix at 8 rows: 48.7 us against 42.9, a 50 MB one 16.4 against 14.5, an 8 MB one 4.9 against 4.6).
// So the same weights can be handed over in the order the matrix cores take them: strips of 16 rows of w, a
// strip a run of K/32 tiles of 1 KB, a tile (rows r = 0..15 of the strip, elements 32 t .. 32 t + 31 of K) stored
// as [4 groups of 8 elements][16 rows][8 elements], which is lane g*16 + r of a wave loading its 16 bytes of the
// tile at byte (g*16 + r)*16.  A wave's stretch of K of a strip is then one contiguous stretch of memory.  The
// rows of w (for act(gate) * up: the columns of y, so that the up rows start a strip) have to be a multiple of 16
// and K of 32, and the kernel for one tile of 16 rows of x is the one that reads them (sk_strips_apply).
#define SK_HAND_CHUNK 8      // sums a lane adds up: sixteen lanes a row, so count <= 128 (a stream of 2,048)

__device__ __forceinline__ bf16x8 sk_load8(const bf16_t* p) {
    return *reinterpret_cast<const bf16x8*>(p);
}

__device__ __forceinline__ bf16x8 sk_zero8() {
    bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    return z;
}

// Eight consecutive gains (32-bit floats).
__device__ __forceinline__ void sk_load_gain(const float* gain, int k, float* out) {
    const sk_f32x4 a = *reinterpret_cast<const sk_f32x4*>(gain + k);
    const sk_f32x4 b = *reinterpret_cast<const sk_f32x4*>(gain + k + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        out[e] = a.v[e];
        out[4 + e] = b.v[e];
    }
}

// MT: 16-row tiles of x (n <= 16*MT).  UNR: K steps a wave asks for at once.  WV: the most waves a
// workgroup may have (it is launched with as many as give every wave one round of loads, or WV).
// The gain is 32-bit.
// A workgroup walks the column tiles blockIdx.x, blockIdx.x + gridDim.x, ...; when a wave's share of
// K fits one round of loads, its rows of x are loaded (and normalised) once and stay in registers.
// 16 bytes a lane from global memory straight into LDS (lane l's land at lds_at + 16 l; lds_at, the same
// for the wave, travels in M0).  Assembly, so that the compiler does not count the load and make every
// later read of LDS wait for it; the wait is written by hand where the panel is due.
__device__ __forceinline__ void sk_load_to_lds(const void* from, const void* lds_at) {
    const uint32_t at = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)lds_at));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(at), "v"(from) : "memory", "m0");
}

// HANDS (an adding product): the kernel leaves the next norm's work behind.  It is a kernel of its own because
// what that adds to the last stage costs the product registers that the 16-wave shapes do not have.
template <int MT, int UNR, int WV, int PRO, int EPI, typename OUT, bool PANEL = false, bool AHEAD = false, bool HANDS = false>
__global__ void __launch_bounds__(64 * WV)
gemm_skinny_kernel(const void* __restrict__ x_, const bf16_t* __restrict__ w, OUT* __restrict__ y,
                   const float* __restrict__ gain, float eps, const int* __restrict__ rows, int n, int N_out,
                   int K, int act, sk_extras_t hand) {
    constexpr int BT = EPI == EPI_SWIGLU ? 2 : 1;
    // may be handed the sums of squares of its rows (a product that adds into the stream reads a part's output,
    // never a norm's)
    // (nor a product so deep that it takes sixteen waves: the norm of a stream that wide is not handed forward)
    constexpr bool TAKES = PRO == PRO_BF16 && MT == 1 && EPI != EPI_ADD && WV <= 8;
    const int nwaves = blockDim.x / PL_WAVE;
    extern __shared__ float sk_lds[];
    // PANEL: [BT * 16][K] bfloat16, in the same place as the partial tiles (which are written when it is done with)
    bf16_t* panel = reinterpret_cast<bf16_t*>(sk_lds);
    float* red = sk_lds;                                   // [nwaves][BT][MT][256] partial tiles
    float* ssq_lds = red + nwaves * BT * MT * 256;         // [nwaves][MT * 16] partial sums of squares

    const int lane = threadIdx.x % PL_WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PL_WAVE);
    const int c = lane % 16;  // column of the tile (a row of w), and the row of x inside its tile
    const int g = lane / 16;  // which 8 of the 32 values of a K step
    const int num_tiles = pl_ceil_div(N_out, SK_TILE_N);

    // K is cut into one stretch of whole steps a wave.
    const int steps = (K + SK_KSTEP - 1) / SK_KSTEP;
    const int per_wave = hand.steps_a_wave > 0 ? hand.steps_a_wave : (steps + nwaves - 1) / nwaves;
    const int kbeg = wave * per_wave * SK_KSTEP;
    const int kend = min(K, (wave + 1) * per_wave * SK_KSTEP);
    const bool one_round = per_wave <= UNR;

    const bf16_t* xb = static_cast<const bf16_t*>(x_);
    const float* xf = static_cast<const float*>(x_);
    size_t xrow[MT];
    bool row_ok[MT];
    // (blockIdx.y: with few tiles of columns the rows are dealt to workgroups too, 16 * MT to each)
    const int row0 = blockIdx.y * 16 * MT;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int row = row0 + m * 16 + c;
        row_ok[m] = row < n;
        int src = row_ok[m] ? row : 0;
        if (PRO == PRO_NORM && rows) src = rows[src];
        xrow[m] = static_cast<size_t>(src) * K;
    }

    bf16x8 ax[MT][UNR];
    float ssq[MT];
    sk_f32x4 raw[PRO == PRO_NORM ? MT : 1][UNR][2];
    float gn[PRO == PRO_NORM ? UNR : 1][8];

    // The rows of x for the K steps k0, k0 + 32, ...: asked for from a place that exists in any case
    // (a load inside a branch is waited for at the branch's end) ...
    auto ask_x = [&](int k0) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int at = k0 + u * SK_KSTEP + g * 8;
            const int kk = at < kend ? at : 0;  // K is a multiple of 8, so a chunk is whole or absent
            if (PRO == PRO_NORM) sk_load_gain(gain, kk, gn[u]);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (PRO == PRO_BF16) {
                    ax[m][u] = sk_load8(xb + xrow[m] + kk);
                } else {
                    raw[m][u][0] = *reinterpret_cast<const sk_f32x4*>(xf + xrow[m] + kk);
                    raw[m][u][1] = *reinterpret_cast<const sk_f32x4*>(xf + xrow[m] + kk + 4);
                }
            }
        }
    };
    // ... and, once they are there, masked, summed into the row's statistic and rounded.
    auto take_x = [&](int k0) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const bool k_ok = k0 + u * SK_KSTEP + g * 8 < kend;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const bool ok = k_ok && row_ok[m];
                if (PRO == PRO_BF16) {
                    ax[m][u] = ok ? ax[m][u] : sk_zero8();
                } else {
                    f32x8 v;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float xv = ok ? raw[m][u][e / 4].v[e % 4] : 0.f;
                        ssq[m] = fmaf(xv, xv, ssq[m]);
                        v[e] = xv * gn[u][e];
                    }
                    ax[m][u] = __builtin_convertvector(v, bf16x8);
                }
            }
        }
    };

#pragma unroll
    for (int m = 0; m < MT; ++m) ssq[m] = 0.f;
    // (x before the weights although those come from furthest away: loads are waited for in the order in which they
    // were asked for, and what is done with x, the norm's arithmetic among it, is done while the weights are on
    // their way.)
    bool x_asked = one_round && kbeg < kend;
    if (x_asked) ask_x(kbeg);

    // Handed sums of squares: the sixteen threads that will finish a row's sixteen columns each ask for a
    // run of the row's sums now, with x, and add them up behind the products (inside the loop over K the
    // sum cost the kernel sixty registers).  Asked for from a place that exists in any case, like x.
    float hp[TAKES ? SK_HAND_CHUNK : 1];
    bool hand_pending = false;
    float hand_rinv = 1.f;
    if constexpr (TAKES) {
        hand_pending = hand.parts != nullptr;
        const float* from = hand_pending ? hand.parts : static_cast<const float*>(x_);
        const int ft = threadIdx.x % 256;
        const int frow = row0 + (ft / 64) * 4 + ft % 4, fc = (ft / 4) % 16;
        const int run = pl_ceil_div(hand.count, 16);
#pragma unroll
        for (int j = 0; j < SK_HAND_CHUNK; ++j) {
            const int idx = fc * run + j;
            const bool ok = hand_pending && frow < n && j < run && idx < hand.count;
            const float got = from[ok ? static_cast<size_t>(frow) * hand.count + idx : 0];
            hp[j] = ok ? got : 0.f;
        }
    }
    auto take_hand = [&]() {
        if constexpr (TAKES) {
            if (hand_pending) {
                float s = 0.f;
#pragma unroll
                for (int j = 0; j < SK_HAND_CHUNK; ++j) s += hp[j];
                s += __shfl_xor(s, 4, PL_WAVE);
                s += __shfl_xor(s, 8, PL_WAVE);
                s += __shfl_xor(s, 16, PL_WAVE);
                s += __shfl_xor(s, 32, PL_WAVE);
                hand_rinv = 1.f / sqrtf(s / static_cast<float>(K) + eps);
                hand_pending = false;
            }
        }
    };

    for (int tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
        const int n0 = tile * SK_TILE_N;
        const bool col_ok = n0 + c < N_out;

        const bf16_t* wrow[BT];
        wrow[0] = w + static_cast<size_t>(col_ok ? n0 + c : 0) * K;
        if (BT == 2) wrow[BT - 1] = w + static_cast<size_t>(N_out + (col_ok ? n0 + c : 0)) * K;
        if (!PANEL && hand.strips) {       // the strip of the tile, and the lane's 16 bytes of the strip's first tile
            wrow[0] = w + static_cast<size_t>(tile) * 16 * K + lane * 8;
            if (BT == 2) wrow[BT - 1] = w + static_cast<size_t>(N_out / 16 + tile) * 16 * K + lane * 8;
        }
        // where the lane's 8 values of K step `at` (its own piece at + g*8) stand from wrow
        const int wmul = (!PANEL && hand.strips) ? 16 : 1, wadd = (!PANEL && hand.strips) ? 0 : g * 8;

        if constexpr (PANEL) {
            // the tile's rows of w, 1 KB (64 pieces of a row) a load, dealt to the waves in turn
            const int chunks = K / 512, loads = BT * 16 * chunks;
            for (int j = wave; j < loads; j += nwaves) {
                const int prow = j / chunks, chunk = j - prow * chunks;
                const int r = prow % 16;
                const size_t grow = (prow >= 16 ? N_out : 0) + static_cast<size_t>(n0 + r < N_out ? n0 + r : 0);
                const int piece = (chunk * 64 + lane) ^ r;
                sk_load_to_lds(w + grow * K + piece * 8, panel + static_cast<size_t>(prow) * K + chunk * 512);
            }
        }

        f32x4 acc[BT][MT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int b = 0; b < BT; ++b) acc[b][m] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (!one_round) {
#pragma unroll
            for (int m = 0; m < MT; ++m) ssq[m] = 0.f;
        }
        // AHEAD (a wave's share of K takes several rounds of loads): the weights of a round are asked for
        // while the round before is multiplied, held as they come and masked when they are used.
        bf16x8 ahead[AHEAD ? BT : 1][AHEAD ? UNR : 1];
        auto ask_w = [&](int k0) {
            if constexpr (AHEAD) {
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    const int at = k0 + u * SK_KSTEP;
                    const int kk = at + g * 8 < kend ? at * wmul + wadd : 0;
#pragma unroll
                    for (int b = 0; b < BT; ++b) ahead[b][u] = sk_load8(wrow[b] + kk);
                }
            }
        };
        ask_w(kbeg);
        if constexpr (PANEL) {
            __builtin_amdgcn_s_waitcnt(0x0F70);            // vmcnt(0): this wave's share of the panel has landed
            __syncthreads();                               // and every wave's
        }

        for (int k0 = kbeg; k0 < kend; k0 += SK_KSTEP * UNR) {
            if constexpr (PANEL) {
                // w waits in LDS: x is asked for (if it is not held from the start) and each step's
                // piece of w is read just before its products
                if (!one_round) {
                    ask_x(k0);
                    take_x(k0);
                } else if (x_asked) {
                    take_x(kbeg);
                    x_asked = false;
                }
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    const int at = k0 + u * SK_KSTEP + g * 8;
                    const int kk = at < kend ? at : 0;          // past the end x is zero
#pragma unroll
                    for (int b = 0; b < BT; ++b) {
                        const bf16x8 bw = sk_load8(panel + static_cast<size_t>(b * 16 + c) * K + (((kk >> 3) ^ c) << 3));
#pragma unroll
                        for (int m = 0; m < MT; ++m)
                            acc[b][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[m][u], bw, acc[b][m], 0, 0, 0);
                    }
                }
            } else {
                bf16x8 bw[BT][UNR];
                if constexpr (AHEAD) {
                    // this round's weights were asked for a round ago; the next round's are asked for now
#pragma unroll
                    for (int u = 0; u < UNR; ++u) {
                        const bool k_ok = k0 + u * SK_KSTEP + g * 8 < kend;
#pragma unroll
                        for (int b = 0; b < BT; ++b) bw[b][u] = (k_ok && col_ok) ? ahead[b][u] : sk_zero8();
                    }
                    ask_w(k0 + SK_KSTEP * UNR);
                } else {
#pragma unroll
                    for (int u = 0; u < UNR; ++u) {
                        const int at = k0 + u * SK_KSTEP;
                        const bool k_ok = at + g * 8 < kend;
                        const int kk = k_ok ? at * wmul + wadd : 0;
#pragma unroll
                        for (int b = 0; b < BT; ++b) {
                            const bf16x8 got = sk_load8(wrow[b] + kk);
                            bw[b][u] = (k_ok && col_ok) ? got : sk_zero8();
                        }
                    }
                }
                // the weights are asked for first: they come from furthest away
                if (!one_round) {
                    ask_x(k0);
                    take_x(k0);
                } else if (x_asked) {
                    take_x(kbeg);
                    x_asked = false;
                }
#pragma unroll
                for (int u = 0; u < UNR; ++u)
#pragma unroll
                    for (int m = 0; m < MT; ++m)
#pragma unroll
                        for (int b = 0; b < BT; ++b)
                            acc[b][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[m][u], bw[b][u], acc[b][m], 0, 0, 0);
            }
        }

        take_hand();
        // the next norm's gain of the column this thread will finish (a product that hands forward): asked for
        // here, where the registers of the products are free, and used behind the sums through LDS
        float hand_gain = 1.f;
        if constexpr (HANDS) {
            const int hc = n0 + (threadIdx.x % 256 / 4) % 16;
            hand_gain = hand.gain[hc < N_out ? hc : 0];
        }
        if constexpr (PANEL) __syncthreads();   // every wave has read its last of the panel
        // A lane holds rows (lane/16)*4 + i, i = 0..3, of column lane%16 of its 16x16 tile.
#pragma unroll
        for (int b = 0; b < BT; ++b)
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[((wave * BT + b) * MT + m) * 256 + lane * 4 + i] = acc[b][m][i];
        if (PRO == PRO_NORM) {
            // the four lanes that hold a row's four chunks of a K step, then the four waves
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float s = ssq[m];
                s += __shfl_xor(s, 16, PL_WAVE);
                s += __shfl_xor(s, 32, PL_WAVE);
                if (g == 0) ssq_lds[wave * MT * 16 + m * 16 + c] = s;
            }
        }
        __syncthreads();

        const int t = threadIdx.x % 256;   // with more than four waves the first four finish the tile
        const int src_lane = t / 4, i = t % 4;
        const int row_in_tile = (src_lane / 16) * 4 + i;
        const int col = n0 + src_lane % 16;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int row = row0 + m * 16 + row_in_tile;
            float v[BT];
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                float s = 0.f;
#pragma unroll
                for (int wv = 0; wv < nwaves; ++wv) s += red[((wv * BT + b) * MT + m) * 256 + t];
                v[b] = s;
            }
            if (PRO == PRO_NORM) {
                float total = 0.f;
#pragma unroll
                for (int wv = 0; wv < nwaves; ++wv) total += ssq_lds[wv * MT * 16 + m * 16 + row_in_tile];
                const float rinv = 1.f / sqrtf(total / static_cast<float>(K) + eps);
#pragma unroll
                for (int b = 0; b < BT; ++b) v[b] *= rinv;
            }
            if constexpr (TAKES) {
#pragma unroll
                for (int b = 0; b < BT; ++b) v[b] *= hand_rinv;      // (1 where nothing was handed)
            }
            const bool mine = threadIdx.x < 256 && row < n && col < N_out;
            float updated = 0.f;
            if (mine) {
                float r = v[0];
                if (EPI == EPI_SWIGLU) r = pl_activate<false>(v[0], act) * v[BT - 1];
                const size_t at = static_cast<size_t>(row) * N_out + col;
                if (EPI == EPI_ADD) {
                    updated = to_float(y[at]) + r;
                    y[at] = from_float<OUT>(updated);
                } else {
                    y[at] = from_float<OUT>(r);
                }
            }
            if constexpr (HANDS) {
                {
                    // the stripe of the updated stream, as the next norm's product will want it, and its sum of
                    // squares a row: the sixteen columns of a row are sixteen lanes of one wave, four apart
                    if (mine) hand.x[static_cast<size_t>(row) * N_out + col] = from_float<bf16_t>(updated * hand_gain);
                    float sq = updated * updated;
                    sq += __shfl_xor(sq, 4, PL_WAVE);
                    sq += __shfl_xor(sq, 8, PL_WAVE);
                    sq += __shfl_xor(sq, 16, PL_WAVE);
                    sq += __shfl_xor(sq, 32, PL_WAVE);
                    if (threadIdx.x < 256 && row < n && src_lane % 16 == 0)
                        hand.ssq[static_cast<size_t>(row) * num_tiles + tile] = sq;
                }
            }
        }
        __syncthreads();  // the next tile writes the same LDS
    }
}

// More column tiles than this many workgroups are walked in a loop, which keeps a wave's rows of x
// in its registers from tile to tile: eight workgroups a compute unit are as many as stay resident.
#define SK_MAX_GRID 2048
// Up to this many workgroups (column tiles times row tiles) a product of 17 to 64 rows is dealt out by row tiles too.
#define SK_ROW_TILES_GRID 512

template <int MT, int UNR, int WV, int PRO, int EPI, typename OUT>
static int launch_one(int waves, const void* x, const void* w, void* y, const float* gain, float eps,
                      const int* rows, int n, int N_out, int K, int act, const sk_extras_t& hand, hipStream_t stream) {
    PL_REQUIRE(!hand.parts || (MT == 1 && PRO == PRO_BF16 && EPI != EPI_ADD && WV <= 8), "skinny product: this shape of product takes no handed norm");
    PL_REQUIRE(!hand.strips || MT == 1, "skinny product: this shape of product reads the weights row by row");
    const int row_tiles = pl_ceil_div(n, 16 * MT);   // more than one where launch_mt deals the rows out
    constexpr int BT = EPI == EPI_SWIGLU ? 2 : 1;
    constexpr int UA = (WV == 16 && UNR >= 2) ? UNR / 2 : UNR;   // K steps a round when rounds overlap
    const int grid = min(pl_ceil_div(N_out, SK_TILE_N), SK_MAX_GRID);
    const size_t lds_bytes = static_cast<size_t>(waves) * (BT * MT * 256 + MT * 16) * sizeof(float);
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_skinny_kernel<MT, UNR, WV, PRO, EPI, OUT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
        PL_REQUIRE(e == hipSuccess, "skinny product: %zu bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_skinny_kernel<MT, UA, WV, PRO, EPI, OUT, false, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
        PL_REQUIRE(e == hipSuccess, "skinny product: %zu bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
    }
    // A wave's share of K in more rounds of loads than one: the rounds overlap, two of them on their way at
    // a time (of half the steps each where sixteen waves leave a lane 128 registers).
    const bool several = pl_ceil_div(pl_ceil_div(K, SK_KSTEP), waves) > UNR;
    const dim3 grid3(grid, row_tiles);
    const bf16_t* wb = static_cast<const bf16_t*>(w);
    OUT* yo = static_cast<OUT*>(y);
    PL_REQUIRE(!hand.x || (EPI == EPI_ADD && MT == 1), "skinny product: this shape of product hands nothing forward");
    if constexpr (EPI == EPI_ADD && MT == 1) {
        if (hand.x) {
            // (with 16 waves the last stage's extra work would spill beside eight K steps of loads: six then)
            constexpr int UH = WV == 16 ? (UNR * 3) / 4 : UNR;
            constexpr int UHA = (WV == 16 && UH >= 2) ? UH / 2 : UH;
            const int steps = pl_ceil_div(K, SK_KSTEP);
            const int wh = WV == 16 ? max(9, min(16, pl_ceil_div(steps, UH))) : waves;    // as many waves as cover K in one round
            const size_t lds_h = static_cast<size_t>(wh) * (BT * MT * 256 + MT * 16) * sizeof(float);
            if (pl_ceil_div(steps, wh) > UH)
                gemm_skinny_kernel<MT, UHA, WV, PRO, EPI, OUT, false, true, true><<<grid3, 64 * wh, lds_h, stream>>>(
                    x, wb, yo, gain, eps, rows, n, N_out, K, act, sk_with_steps(hand, K, wh));
            else
                gemm_skinny_kernel<MT, UH, WV, PRO, EPI, OUT, false, false, true><<<grid3, 64 * wh, lds_h, stream>>>(
                    x, wb, yo, gain, eps, rows, n, N_out, K, act, sk_with_steps(hand, K, wh));
            PL_CHECK_LAUNCH("gemm_skinny");
            return 0;
        }
    }
    if (several)
        gemm_skinny_kernel<MT, UA, WV, PRO, EPI, OUT, false, true><<<grid3, 64 * waves, lds_bytes, stream>>>(
            x, wb, yo, gain, eps, rows, n, N_out, K, act, sk_with_steps(hand, K, waves));
    else
        gemm_skinny_kernel<MT, UNR, WV, PRO, EPI, OUT><<<grid3, 64 * waves, lds_bytes, stream>>>(
            x, wb, yo, gain, eps, rows, n, N_out, K, act, sk_with_steps(hand, K, waves));
    PL_CHECK_LAUNCH("gemm_skinny");
    return 0;
}

// ---------------------------------------------------------------------------
// More than 16 rows, K a multiple of 512: every wave takes ONE tile of 16 rows and one stretch of K.
// The workgroup's rows of w come into LDS first (as with PANEL above, and the norm's gains beside
// them), so that w costs the waves no registers; a wave then asks for its whole share of x at once,
// STEPS K steps of 16 bytes a lane (32 with the 32-bit stream), and multiplies as they arrive.  With MT
// tiles of rows there are WV / MT stretches of K.  The partial tiles and sums of squares meet in LDS
// (where the panel was) and every thread finishes one element of one tile.
// ---------------------------------------------------------------------------
template <int MT, int WV, int STEPS, int PRO, int EPI, typename OUT>
__global__ void __launch_bounds__(64 * WV)
gemm_skinny_rows_kernel(const void* __restrict__ x_, const bf16_t* __restrict__ w, OUT* __restrict__ y,
                        const float* __restrict__ gain, float eps, const int* __restrict__ rows, int n, int N_out,
                        int K, int act, sk_extras_t hand) {
    constexpr int BT = EPI == EPI_SWIGLU ? 2 : 1;
    // may be handed the sums of squares of its rows (a stream of up to 2,048: eight steps a wave, or sixteen with four tiles of rows)
    constexpr bool TAKES = PRO == PRO_BF16 && EPI != EPI_ADD && WV * 64 >= MT * 256 && (STEPS <= 8 || MT == 4);
    constexpr int NKS = WV / MT;                                // stretches of K
    extern __shared__ float sk_lds[];
    bf16_t* panel = reinterpret_cast<bf16_t*>(sk_lds);          // [BT * 16][K], pieces permuted
    float* red = sk_lds;                                        // [NKS][MT][BT][256], once the panel is done with
    // The gains are loaded once and read for every tile of columns, the sums of squares are written for
    // every tile: both lie behind the larger of the panel and the partial tiles, which alone share a place.
    float* gain_lds = sk_lds + max(BT * 16 * K / 2, NKS * MT * BT * 256);   // [K] (PRO_NORM)
    float* ssq_lds = gain_lds + (PRO == PRO_NORM ? K : 0);      // [NKS][MT][16]

    const int lane = threadIdx.x % PL_WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PL_WAVE);
    const int c = lane % 16, g = lane / 16;
    const int mt = wave % MT, ks = wave / MT;
    const bool working = ks < NKS;                              // WV need not be a multiple of MT
    const int num_tiles = pl_ceil_div(N_out, SK_TILE_N);
    const int per_slice = K / SK_KSTEP / NKS * SK_KSTEP;        // K is a multiple of 512, NKS of 16 at most... see the launcher
    const int kbeg = ks * per_slice;

    // the wave's rows of x, asked for once: they serve every tile of columns
    const int row = mt * 16 + c;
    const bool row_ok = working && row < n;
    int src = row_ok ? row : 0;
    if (PRO == PRO_NORM && rows) src = rows[src];
    const size_t xrow = static_cast<size_t>(src) * K;
    const bf16_t* xb = static_cast<const bf16_t*>(x_);
    const float* xf = static_cast<const float*>(x_);
    bf16x8 ax[PRO == PRO_BF16 ? STEPS : 1];
    sk_f32x4 raw[PRO == PRO_NORM ? STEPS : 1][2];
#pragma unroll
    for (int u = 0; u < STEPS; ++u) {
        const int at = kbeg + u * SK_KSTEP + g * 8;
        const int kk = (u * SK_KSTEP < per_slice) ? at : 0;
        if (PRO == PRO_BF16) {
            ax[u] = sk_load8(xb + xrow + kk);
        } else {
            raw[u][0] = *reinterpret_cast<const sk_f32x4*>(xf + xrow + kk);
            raw[u][1] = *reinterpret_cast<const sk_f32x4*>(xf + xrow + kk + 4);
        }
    }
    if (PRO == PRO_NORM)
        for (int k = threadIdx.x * 4; k < K; k += blockDim.x * 4)
            *reinterpret_cast<sk_f32x4*>(gain_lds + k) = *reinterpret_cast<const sk_f32x4*>(gain + k);
    // Handed sums of squares (see gemm_skinny_kernel): thread e finishes element e % 256 of tile e / 256, and
    // the sixteen threads of a row each ask for a run of the row's sums, before the panel is asked for.
    float hp[TAKES ? SK_HAND_CHUNK : 1];
    bool hand_pending = false;
    float hand_rinv = 1.f;
    if constexpr (TAKES) {
        hand_pending = hand.parts != nullptr;
        const float* from = hand_pending ? hand.parts : static_cast<const float*>(x_);
        const int ft = threadIdx.x % 256;
        const int frow = (threadIdx.x / 256) * 16 + (ft / 64) * 4 + ft % 4, fc = (ft / 4) % 16;
        const int run = pl_ceil_div(hand.count, 16);
        if (hand.count % 64 == 0) {
            // a lane's run is whole groups of four sums, 16 bytes aligned: one load a group
            static_assert(SK_HAND_CHUNK == 8, "two groups of four");
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const bool ok = hand_pending && frow < n && q * 4 < run;
                const sk_f32x4 got = *reinterpret_cast<const sk_f32x4*>(
                    from + (ok ? static_cast<size_t>(frow) * hand.count + fc * run + q * 4 : 0));
#pragma unroll
                for (int e = 0; e < 4; ++e) hp[q * 4 + e] = ok ? got.v[e] : 0.f;
            }
        } else {
#pragma unroll
            for (int j = 0; j < SK_HAND_CHUNK; ++j) {
                const int idx = fc * run + j;
                const bool ok = hand_pending && frow < n && j < run && idx < hand.count;
                const float got = from[ok ? static_cast<size_t>(frow) * hand.count + idx : 0];
                hp[j] = ok ? got : 0.f;
            }
        }
    }

    for (int tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
        const int n0 = tile * SK_TILE_N;
        {
            const int chunks = K / 512, loads = BT * 16 * chunks;
            for (int j = wave; j < loads; j += WV) {
                const int prow = j / chunks, chunk = j - prow * chunks;
                const int r = prow % 16;
                const size_t grow = (prow >= 16 ? N_out : 0) + static_cast<size_t>(n0 + r < N_out ? n0 + r : 0);
                const int piece = (chunk * 64 + lane) ^ r;
                sk_load_to_lds(w + grow * K + piece * 8, panel + static_cast<size_t>(prow) * K + chunk * 512);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);                     // vmcnt(0): x and this wave's share of the panel
        __syncthreads();
        if constexpr (TAKES) {
            if (hand_pending) {
                float s = 0.f;
#pragma unroll
                for (int j = 0; j < SK_HAND_CHUNK; ++j) s += hp[j];
                s += __shfl_xor(s, 4, PL_WAVE);
                s += __shfl_xor(s, 8, PL_WAVE);
                s += __shfl_xor(s, 16, PL_WAVE);
                s += __shfl_xor(s, 32, PL_WAVE);
                hand_rinv = 1.f / sqrtf(s / static_cast<float>(K) + eps);
                hand_pending = false;
            }
        }

        f32x4 acc[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
        float ssq = 0.f;
        // Rows past n and steps past the stretch are not branched around: a row past n gives outputs that
        // are not stored, and a step past the stretch multiplies by zeros instead of w (x is only looked
        // at here, after the panel has been asked for, so nothing waits for it earlier).
        const int nsteps = per_slice / SK_KSTEP;
        // four steps' pieces of w are read from LDS before their products, so that LDS is waited for once in four
        static_assert(STEPS % 4 == 0, "steps are taken four at a time");
#pragma unroll
        for (int u0 = 0; u0 < STEPS; u0 += 4) {
            bf16x8 bw[4][BT];
            int kk[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool live = u0 + j < nsteps;
                kk[j] = kbeg + (live ? u0 + j : 0) * SK_KSTEP + g * 8;
#pragma unroll
                for (int b = 0; b < BT; ++b) {
                    const bf16x8 got = sk_load8(panel + static_cast<size_t>(b * 16 + c) * K + (((kk[j] >> 3) ^ c) << 3));
                    bw[j][b] = live ? got : sk_zero8();
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int u = u0 + j;
                bf16x8 a;
                if (PRO == PRO_BF16) {
                    a = ax[u];
                } else {
                    const bool live = u < nsteps;
                    const sk_f32x4 g0 = *reinterpret_cast<const sk_f32x4*>(gain_lds + kk[j]);
                    const sk_f32x4 g1 = *reinterpret_cast<const sk_f32x4*>(gain_lds + kk[j] + 4);
                    f32x8 v;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float xv = raw[u][e / 4].v[e % 4];
                        ssq = live ? fmaf(xv, xv, ssq) : ssq;
                        v[e] = xv * (e < 4 ? g0.v[e % 4] : g1.v[e % 4]);
                    }
                    a = __builtin_convertvector(v, bf16x8);
                }
#pragma unroll
                for (int b = 0; b < BT; ++b)
                    acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bw[j][b], acc[b], 0, 0, 0);
            }
        }
        __syncthreads();                                        // every wave has read its last of the panel
        if (working) {
#pragma unroll
            for (int b = 0; b < BT; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[((ks * MT + mt) * BT + b) * 256 + lane * 4 + i] = acc[b][i];
            if (PRO == PRO_NORM) {
                float s = ssq;
                s += __shfl_xor(s, 16, PL_WAVE);
                s += __shfl_xor(s, 32, PL_WAVE);
                if (g == 0) ssq_lds[(ks * MT + mt) * 16 + c] = s;
            }
        }
        __syncthreads();
        // one element of one tile a thread: element t of tile m is row (t/64)*4 + t%4 of the tile, column (t/4)%16
        for (int e = threadIdx.x; e < MT * 256; e += blockDim.x) {
            const int m = e / 256, t = e % 256;
            const int src_lane = t / 4, i = t % 4;
            const int row_in_tile = (src_lane / 16) * 4 + i;
            const int out_row = m * 16 + row_in_tile, col = n0 + src_lane % 16;
            float v[BT];
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                float s = 0.f;
#pragma unroll
                for (int k = 0; k < NKS; ++k) s += red[((k * MT + m) * BT + b) * 256 + t];
                v[b] = s;
            }
            if (PRO == PRO_NORM) {
                float total = 0.f;
#pragma unroll
                for (int k = 0; k < NKS; ++k) total += ssq_lds[(k * MT + m) * 16 + row_in_tile];
                const float rinv = 1.f / sqrtf(total / static_cast<float>(K) + eps);
#pragma unroll
                for (int b = 0; b < BT; ++b) v[b] *= rinv;
            }
            if constexpr (TAKES) {
                // (the launch has a thread for every element, so e is this thread's own index and the
                // statistic it holds is its row's)
#pragma unroll
                for (int b = 0; b < BT; ++b) v[b] *= hand_rinv;
            }
            if (out_row < n && col < N_out) {
                float r = v[0];
                if (EPI == EPI_SWIGLU) r = pl_activate<false>(v[0], act) * v[BT - 1];
                const size_t at = static_cast<size_t>(out_row) * N_out + col;
                if (EPI == EPI_ADD)
                    y[at] = from_float<OUT>(to_float(y[at]) + r);
                else
                    y[at] = from_float<OUT>(r);
            }
        }
        __syncthreads();  // the next tile's panel lands where the partial tiles are
    }
}

// The rows variant's launch: WV waves, MT tiles of rows, WV / MT stretches of K of at most STEPS steps.
template <int MT, int WV, int STEPS, int PRO, int EPI, typename OUT>
static int launch_rows(const void* x, const void* w, void* y, const float* gain, float eps,
                       const int* rows, int n, int N_out, int K, int act, const sk_extras_t& hand, hipStream_t stream) {
    PL_REQUIRE(!hand.x, "skinny product: this shape of product hands nothing forward");
    PL_REQUIRE(!hand.strips, "skinny product: this shape of product reads the weights row by row");
    PL_REQUIRE(!hand.parts || (PRO == PRO_BF16 && EPI != EPI_ADD && WV * 64 >= MT * 256 && (STEPS <= 8 || MT == 4)),
               "skinny product: this shape of product takes no handed norm");
    constexpr int BT = EPI == EPI_SWIGLU ? 2 : 1;
    constexpr int NKS = WV / MT;
    const int grid = min(pl_ceil_div(N_out, SK_TILE_N), SK_MAX_GRID);
    const size_t panel_bytes = static_cast<size_t>(BT) * 16 * K * 2;
    const size_t red_bytes = static_cast<size_t>(NKS) * MT * BT * 256 * sizeof(float);
    const size_t lds_bytes = (panel_bytes > red_bytes ? panel_bytes : red_bytes)
                             + (PRO == PRO_NORM ? static_cast<size_t>(K) * 4 : 0)      // the gains
                             + static_cast<size_t>(NKS) * MT * 16 * sizeof(float);     // the sums of squares
    auto kernel = &gemm_skinny_rows_kernel<MT, WV, STEPS, PRO, EPI, OUT>;
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(lds_bytes));
        PL_REQUIRE(e == hipSuccess, "skinny product: %zu bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
    }
    kernel<<<grid, 64 * WV, lds_bytes, stream>>>(x, static_cast<const bf16_t*>(w), static_cast<OUT*>(y), gain, eps,
                                                rows, n, N_out, K, act, hand);
    PL_CHECK_LAUNCH("gemm_skinny");
    return 0;
}

// The panel variant: 8 waves (256 registers a lane); a wave holds 16 * MT rows of x for UNR K steps.
template <int MT, int UNR, int PRO, int EPI, typename OUT>
static int launch_panel(const void* x, const void* w, void* y, const float* gain, float eps,
                        const int* rows, int n, int N_out, int K, int act, const sk_extras_t& hand, hipStream_t stream) {
    PL_REQUIRE(!hand.parts || (MT == 1 && EPI != EPI_ADD), "skinny product: this shape of product takes no handed norm");
    PL_REQUIRE(!hand.x, "skinny product: this shape of product hands nothing forward");
    PL_REQUIRE(!hand.strips, "skinny product: this shape of product reads the weights row by row");
    constexpr int BT = EPI == EPI_SWIGLU ? 2 : 1;
    constexpr int waves = 8;
    const int grid = min(pl_ceil_div(N_out, SK_TILE_N), SK_MAX_GRID);
    const size_t panel_bytes = static_cast<size_t>(BT) * 16 * K * 2;
    const size_t red_bytes = static_cast<size_t>(waves) * (BT * MT * 256 + MT * 16) * sizeof(float);
    const size_t lds_bytes = panel_bytes > red_bytes ? panel_bytes : red_bytes;
    auto kernel = &gemm_skinny_kernel<MT, UNR, waves, PRO, EPI, OUT, true>;
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(lds_bytes));
        PL_REQUIRE(e == hipSuccess, "skinny product: %zu bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
    }
    kernel<<<grid, 64 * waves, lds_bytes, stream>>>(x, static_cast<const bf16_t*>(w), static_cast<OUT*>(y), gain, eps,
                                                   rows, n, N_out, K, act, sk_with_steps(hand, K, waves));
    PL_CHECK_LAUNCH("gemm_skinny");
    return 0;
}

// Whether a product of MT tiles of rows goes to the rows kernel (launch_unr's choice, also asked by what decides
// on strips and handed norms): 16 waves in 16 / MT stretches of K, each a whole number of K steps that a wave can
// hold at once, the panel (and the norm's gains) within LDS.  steps: the K steps a wave then holds (8 or 16).
static inline bool sk_rows_kernel_takes(int MT, int K, bool two_tiles, bool norm, int* steps = nullptr) {
    if (MT != 2 && MT != 4) return false;
    const int NKS = 16 / MT;
    const size_t panel = static_cast<size_t>(two_tiles ? 2 : 1) * 16 * K * 2 + (norm ? static_cast<size_t>(K) * 4 : 0);
    if (K % 512 != 0 || K / SK_KSTEP % NKS != 0 || panel > 144 * 1024) return false;
    const int need = K / SK_KSTEP / NKS;
    // (the 32-bit stream takes twice the registers a step; 24 steps would fit the registers of 16 waves only with spills)
    if (need > (norm ? 8 : 16)) return false;
    if (steps) *steps = need <= 8 ? 8 : 16;
    return true;
}

// How many waves, and how many K steps each asks for at once.  What a wave holds in flight has to fit
// its registers (512 a lane with four waves, 256 with eight, 128 with sixteen); within that, the
// fewest waves whose one round of loads covers K are taken, so that the whole matrix is asked for at
// once and the kernel's time is one trip to memory.  The numbers are the largest that compile
// without spilling (0: that many waves have no room).
template <int MT, int PRO, int EPI>
struct SkShape {
    static constexpr bool TWO = EPI == EPI_SWIGLU;     // two weight tiles a step
    static constexpr int U4 = PRO == PRO_NORM ? (MT == 1 ? 8 : (MT == 2 ? 4 : 2)) : ((TWO && MT >= 3) ? 4 : 8);
    static constexpr int U8 = PRO == PRO_NORM ? 0 : (TWO ? (MT == 1 ? 8 : (MT <= 3 ? 4 : 2)) : (MT <= 2 ? 8 : 4));
    static constexpr int U16 = PRO == PRO_NORM ? 0 : (TWO ? (MT == 1 ? 4 : (MT <= 3 ? 2 : 1)) : (MT == 1 ? 8 : (MT == 2 ? 4 : 2)));
};

template <int MT, int PRO, int EPI, typename OUT>
static int launch_unr(const void* x, const void* w, void* y, const float* gain, float eps,
                      const int* rows, int n, int N_out, int K, int act, const sk_extras_t& hand, hipStream_t stream) {
    using S = SkShape<MT, PRO, EPI>;
    if constexpr (MT == 2 || MT == 4) {
        int steps = 0;
        if (sk_rows_kernel_takes(MT, K, EPI == EPI_SWIGLU, PRO == PRO_NORM, &steps)) {
            if (steps == 8) return launch_rows<MT, 16, 8, PRO, EPI, OUT>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
            if constexpr (PRO == PRO_BF16)
                return launch_rows<MT, 16, 16, PRO, EPI, OUT>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
        }
    }
    if constexpr (MT >= 2) {
        constexpr int BT = EPI == EPI_SWIGLU ? 2 : 1;
        if (K % 512 == 0 && static_cast<size_t>(BT) * 16 * K * 2 <= 128 * 1024)
            return launch_panel<MT, (PRO == PRO_NORM ? (MT == 4 ? 1 : 2) : (MT == 4 ? 4 : 8)), PRO, EPI, OUT>(
                x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
    }
    const int steps = pl_ceil_div(K, SK_KSTEP);
    const int most = max(4 * S::U4, max(8 * S::U8, 16 * S::U16));
    const int need = min(steps, most);     // beyond that, several rounds
    if (need <= 4 * S::U4)
        return launch_one<MT, S::U4, 4, PRO, EPI, OUT>(4, x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
    if constexpr (S::U8 > 0) {
        if (need <= 8 * S::U8 || S::U16 == 0)
            return launch_one<MT, S::U8, 8, PRO, EPI, OUT>(max(5, min(8, pl_ceil_div(steps, S::U8))), x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
    }
    if constexpr (S::U16 > 0) {
        return launch_one<MT, S::U16, 16, PRO, EPI, OUT>(max(9, min(16, pl_ceil_div(steps, S::U16))), x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
    }
    return launch_one<MT, S::U4, 4, PRO, EPI, OUT>(4, x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
}

template <int PRO, int EPI, typename OUT>
static int launch_mt(const void* x, const void* w, void* y, const float* gain, float eps,
                     const int* rows, int n, int N_out, int K, int act, const sk_extras_t& hand, hipStream_t stream) {
    // Few tiles of columns (a narrow output, as of the projections back into the stream): the tiles of 16 rows
    // go to workgroups of their own, the kernel for up to 16 rows on a grid of (column tiles, row tiles), so that
    // the launch has workgroups for every compute unit; each reads its rows of x only, and w comes from L2
    // from the second row tile on.
    if (n > 16 && pl_ceil_div(N_out, SK_TILE_N) * pl_ceil_div(n, 16) <= SK_ROW_TILES_GRID)
        return launch_unr<1, PRO, EPI, OUT>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
    switch (pl_ceil_div(n, 16)) {
        case 1: return launch_unr<1, PRO, EPI, OUT>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
        case 2: return launch_unr<2, PRO, EPI, OUT>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
        case 3:
            // (a handed norm is taken by the kernel of two or four tiles of rows: three go as four, one of them empty)
            if (hand.parts) return launch_unr<4, PRO, EPI, OUT>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
            return launch_unr<3, PRO, EPI, OUT>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
        default: return launch_unr<4, PRO, EPI, OUT>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
    }
}

// Whether a product of this shape reads its weights in strips: the layout is defined, and launch_mt takes the
// kernel for one tile of rows (the kernels whose weights wait in LDS read the rows: there the strips gained
// nothing that showed, and cost the deepest shapes registers).  N_out: the columns of y.
static inline bool sk_strips_apply(int n, int N_out, int K) {
    if (n <= 0 || n > 64 || N_out <= 0 || N_out % SK_TILE_N || K <= 0 || K % SK_KSTEP) return false;
    return n <= 16 || pl_ceil_div(N_out, SK_TILE_N) * pl_ceil_div(n, 16) <= SK_ROW_TILES_GRID;
}

// Which kernel the launchers above take for a product of bfloat16 rows, as far as the handed norm goes:
// whether the product can take the sums of squares of its rows (taking), or leave them and the normalised
// stripe behind (an adding product, !taking).  The same conditions as in launch_mt and launch_unr.
static inline bool sk_hand_applies(int n, int N_out, int K, int epilogue, bool taking) {
    if (n <= 0 || n > 64 || K % 8 || N_out <= 0) return false;
    if (taking && (epilogue == EPI_ADD || pl_ceil_div(K, SK_TILE_N) > 16 * SK_HAND_CHUNK)) return false;
    if (!taking && epilogue != EPI_ADD) return false;
    const int row_tiles = pl_ceil_div(n, 16);
    if (n <= 16 || pl_ceil_div(N_out, SK_TILE_N) * row_tiles <= SK_ROW_TILES_GRID) return true;   // the kernel for one tile of rows
    const int MT = (taking && row_tiles == 3) ? 4 : row_tiles;
    const bool rows_kernel = sk_rows_kernel_takes(MT, K, epilogue == EPI_SWIGLU, false);
    return taking && rows_kernel;        // (an adding product hands forward from the kernel for one tile of rows only)
}

template <int PRO>
static int sk_launch(int epilogue, int out_f32, const void* x, const void* w, void* y, const float* gain,
                      float eps, const int* rows, int n, int N_out, int K, int act, const sk_extras_t& hand, hipStream_t stream) {
    if (epilogue == EPI_STORE)
        return out_f32 ? launch_mt<PRO, EPI_STORE, float>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream)
                       : launch_mt<PRO, EPI_STORE, bf16_t>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
    if (epilogue == EPI_SWIGLU) return launch_mt<PRO, EPI_SWIGLU, bf16_t>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
    if constexpr (PRO == PRO_NORM) {
        pl_set_error("skinny product: a product that reads the residual stream cannot add into it");
        return -1;
    } else {
        return launch_mt<PRO, EPI_ADD, float>(x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
    }
}


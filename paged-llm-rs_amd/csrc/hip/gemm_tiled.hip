// y[M, N] = x[M, K] . w[N, K]^T for many rows, bfloat16 operands, 32-bit accumulate, on the matrix
// cores, with what comes after the product fused into it: SwiGLU over [gate | up] weights, or the sum
// into the 32-bit residual stream.
//
// One workgroup of four waves owns 128 rows of x and 128 rows of w (for SwiGLU: 64 gate rows and the 64
// up rows that belong to them).  K is walked 32 at a time through four stages of LDS; every stage is
// asked for three steps ahead by loads that write LDS themselves (global_load_lds_dwordx4: lane l of a
// wave puts its 16 bytes at the wave's LDS base + 16 l), so the operands cost no registers on their
// way.  A row of a stage is 64 bytes, four 16-byte pieces; piece p of row r stands at p ^ ((r >> 2) & 3),
// so that the 16 rows a read of the matrix cores' operands touches at once fall on every bank once.
//
// Wave (wm, wn) computes rows 64 wm .. + 63 against w rows 32 wn .. + 31 of either half of the tile:
//   D^T = W . X^T   v_mfma_f32_32x32x16_bf16, A = 32 rows of w, B = 32 rows of x: a lane then holds, for ONE
//                   row of x (lane % 32), 16 columns of the output in groups of four neighbours, which is what
//                   the epilogue stores.
#include "common.hpp"

typedef __bf16 gt_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gt_f32x16 __attribute__((ext_vector_type(16)));
typedef float gt_f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 gt_bf16x2 __attribute__((ext_vector_type(2)));
typedef float gt_f32x2 __attribute__((ext_vector_type(2)));

#define GT_BM 128          // rows of x a workgroup
#define GT_BN 128          // rows of w a workgroup
#define GT_BK 32           // K a stage
#define GT_STAGES 4
#define GT_STAGE_ELEMS ((GT_BM + GT_BN) * GT_BK)

#define GT_STORE 0
#define GT_SWIGLU 1
#define GT_ADD 2

// 16 bytes a lane from global memory straight into LDS (see attention_prefill.hip: assembly, so that
// the compiler does not count the load and make every later read of LDS wait for all of them).
__device__ __forceinline__ void gt_load_to_lds(const void* from, const uint16_t* lds_at) {
    const uint32_t at = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)lds_at));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(at), "v"(from) : "memory", "m0");
}

__device__ __forceinline__ uint32_t gt_pack2(float lo, float hi) {
    const gt_f32x2 pair = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, gt_bf16x2));
}

// EPI: GT_STORE y = result (bfloat16).  GT_SWIGLU: w is [gate rows | up rows], N counts the gate rows, and
// y = silu(gate) * up (bfloat16).  GT_ADD: y is the 32-bit residual stream and takes the result.
// M any; N a multiple of 128 (64 for SwiGLU); K a multiple of 32.
template <int EPI>
__global__ void __launch_bounds__(256, 2)
gemm_tiled_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ y_, int M, int N, int K,
                  int row_tiles, int total, int act) {
    extern __shared__ __attribute__((aligned(16))) uint16_t gt_lds[];   // [stage][x rows 0..127 | w rows 0..127][32]

    // Workgroups are dealt round-robin to the eight XCDs; consecutive tiles (the row tiles of one column
    // tile first) go to one XCD, whose L2 then holds the rows of w they share.
    int work = blockIdx.x;
    if ((total & 7) == 0) work = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
    const int m0 = (work % row_tiles) * GT_BM;
    const int col_tile = work / row_tiles;
    constexpr int COLS = EPI == GT_SWIGLU ? GT_BN / 2 : GT_BN;   // output columns a workgroup
    const int n0 = col_tile * COLS;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int r32 = lane & 31, h = lane >> 5;

    // The loads of a stage: 16 chunks of 16 rows (eight of x, eight of w), four a wave.  Lane l of a chunk
    // brings piece (l % 4) ^ ((row >> 2) & 3) of row l / 4, which lands in slot l % 4 of that row.
    const char* from[4];
    int lds_chunk[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int chunk = wave + 4 * i;              // 0..7: x, 8..15: w
        const int row = (chunk & 7) * 16 + (lane >> 2);
        const int piece = (lane & 3) ^ ((row >> 2) & 3);
        size_t grow;
        if (chunk < 8) {
            grow = static_cast<size_t>(min(m0 + row, M - 1));
            from[i] = reinterpret_cast<const char*>(x) + (grow * K + piece * 8) * 2;
        } else {
            // SwiGLU: rows 0..63 of the tile are gate rows n0.., rows 64..127 the up rows N + n0..
            grow = EPI == GT_SWIGLU ? static_cast<size_t>(row < 64 ? n0 + row : N + n0 + row - 64) : static_cast<size_t>(n0 + row);
            from[i] = reinterpret_cast<const char*>(w) + (grow * K + piece * 8) * 2;
        }
        lds_chunk[i] = chunk * 16 * GT_BK;           // elements from the stage's start
    }
    const int steps = K / GT_BK;
    auto ask = [&](int step) {                       // past the end the last step is asked for again: the count of
        const int s = min(step, steps - 1);          // loads on their way stays the same for every step
        uint16_t* stage = gt_lds + (step % GT_STAGES) * GT_STAGE_ELEMS;
#pragma unroll
        for (int i = 0; i < 4; ++i) gt_load_to_lds(from[i] + static_cast<size_t>(s) * GT_BK * 2, stage + lds_chunk[i]);
    };

    // where this lane's operands stand in a stage: row and, for either 16 of the 32 K, the slot of its 8
    int a_at[2][2], b_at[2][2];                      // [which 32 rows][K half]
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int wrow = (EPI == GT_SWIGLU ? 64 * t + 32 * wn : 64 * wn + 32 * t) + r32;
        const int xrow = 64 * wm + 32 * t + r32;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            a_at[t][kk] = (GT_BM + wrow) * GT_BK + (((2 * kk + h) ^ ((wrow >> 2) & 3)) * 8);
            b_at[t][kk] = xrow * GT_BK + (((2 * kk + h) ^ ((xrow >> 2) & 3)) * 8);
        }
    }

    gt_f32x16 acc[2][2];                             // [w rows t][x rows mb]
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][mb][r] = 0.f;

    // The operands of a step are read out of LDS one step early, while the step before is multiplied:
    // two sets of registers that take turns.
    gt_bf16x8 a[2][2][2], b[2][2][2];               // [set][which 32 rows][K half]
    auto read_operands = [&](int set, int step) {
        const uint16_t* stage = gt_lds + (step % GT_STAGES) * GT_STAGE_ELEMS;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                a[set][t][kk] = *reinterpret_cast<const gt_bf16x8*>(stage + a_at[t][kk]);
                b[set][t][kk] = *reinterpret_cast<const gt_bf16x8*>(stage + b_at[t][kk]);
            }
    };
    auto multiply = [&](int set) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
                    acc[t][mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[set][t][kk], b[set][mb][kk], acc[t][mb], 0, 0, 0);
    };
    // One step: the loads of the step after this one have landed in this wave (two later steps, eight loads,
    // may be on their way); after the barrier every wave's have, and every wave has read this step's operands,
    // whose stage is the one asked for next.
    auto one_step = [&](int set, int step) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        ask(step + 4);
        read_operands(set ^ 1, step + 1);            // (past the last step: the stage holds the last step again)
        multiply(set);
    };
    ask(0);
    ask(1);
    ask(2);
    ask(3);
    __builtin_amdgcn_s_waitcnt(0x0F70 | 12);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_operands(0, 0);
    int step = 0;
    for (; step + 1 < steps; step += 2) {
        one_step(0, step);
        one_step(1, step + 1);
    }
    if (step < steps) one_step(0, step);
    __builtin_amdgcn_s_waitcnt(0x0F70);              // nothing may still be on its way into LDS when the workgroup ends

    // The last stage goes through LDS: a lane holds, for one row, groups of four neighbouring columns, and
    // stored from there a wave's store would touch 32 rows with 8 or 16 bytes each (a product of 2,048 rows
    // against 4,096 columns spent 8.7 us of its 29 storing 16 MB so).  The tile is laid down in LDS as rows
    // (a pitch of the row plus 16 bytes, so that the rows a store of LDS touches fall on different banks)
    // and leaves in whole rows, 16 bytes a lane.
    // acc[t][mb][4 j + i]: output column (of the wave's 32 of half t) 8 j + 4 h + i, row 64 wm + 32 mb + r32
    __syncthreads();                                 // every wave has read its last operands
    constexpr int OUT_COLS = EPI == GT_SWIGLU ? GT_BN / 2 : GT_BN;
    constexpr int OUT_BYTES = EPI == GT_ADD ? 4 : 2;
    constexpr int PITCH = OUT_COLS * OUT_BYTES + 16;      // bytes (a multiple of 16: rows are read 16 bytes a lane)
    char* staged = reinterpret_cast<char*>(gt_lds);
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
        char* at_row = staged + (64 * wm + 32 * mb + r32) * PITCH;
        if constexpr (EPI == GT_SWIGLU) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float g = acc[0][mb][4 * j + i];
                    v[i] = pl_activate<false>(g, act) * acc[1][mb][4 * j + i];
                }
                uint2 packed;
                packed.x = gt_pack2(v[0], v[1]);
                packed.y = gt_pack2(v[2], v[3]);
                *reinterpret_cast<uint2*>(at_row + (32 * wn + 4 * h + 8 * j) * 2) = packed;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int col = 64 * wn + 32 * t + 4 * h + 8 * j;
                    if constexpr (EPI == GT_ADD) {
                        gt_f32x4 v;
#pragma unroll
                        for (int i = 0; i < 4; ++i) v[i] = acc[t][mb][4 * j + i];
                        *reinterpret_cast<gt_f32x4*>(at_row + col * 4) = v;
                    } else {
                        uint2 packed;
                        packed.x = gt_pack2(acc[t][mb][4 * j], acc[t][mb][4 * j + 1]);
                        packed.y = gt_pack2(acc[t][mb][4 * j + 2], acc[t][mb][4 * j + 3]);
                        *reinterpret_cast<uint2*>(at_row + col * 2) = packed;
                    }
                }
        }
    }
    __syncthreads();
    constexpr int LANES_A_ROW = OUT_COLS * OUT_BYTES / 16;       // 8, 16 or 32
    constexpr int ROWS_A_PASS = 256 / LANES_A_ROW;
    const int piece = tid % LANES_A_ROW;
#pragma unroll 4
    for (int r = tid / LANES_A_ROW; r < GT_BM; r += ROWS_A_PASS) {
        const int row = m0 + r;
        if (row >= M) break;
        const gt_f32x4 got = *reinterpret_cast<const gt_f32x4*>(staged + r * PITCH + piece * 16);
        char* out = static_cast<char*>(y_) + (static_cast<size_t>(row) * N + n0) * OUT_BYTES + piece * 16;
        if constexpr (EPI == GT_ADD) {
            gt_f32x4 old = *reinterpret_cast<const gt_f32x4*>(out);
#pragma unroll
            for (int i = 0; i < 4; ++i) old[i] += got[i];
            *reinterpret_cast<gt_f32x4*>(out) = old;
        } else {
            *reinterpret_cast<gt_f32x4*>(out) = got;
        }
    }
}

template <int EPI>
static int gt_launch(const void* x, const void* w, void* y, int M, int N, int K, int act, hipStream_t stream) {
    constexpr int COLS = EPI == GT_SWIGLU ? GT_BN / 2 : GT_BN;
    const int row_tiles = pl_ceil_div(M, GT_BM);
    const long long total = static_cast<long long>(row_tiles) * (N / COLS);
    PL_REQUIRE(total > 0 && total < (1ll << 30), "tiled product: %lld workgroups", total);
    // the stages of operands, or the tile on its way out (32-bit rows of 128 with their pitch), whichever is more
    constexpr size_t out_bytes = static_cast<size_t>(GT_BM) * (EPI == GT_ADD ? GT_BN * 4 + 16 : (EPI == GT_SWIGLU ? GT_BN + 16 : GT_BN * 2 + 16));
    constexpr size_t stage_bytes = static_cast<size_t>(GT_STAGES) * GT_STAGE_ELEMS * 2;
    const size_t lds_bytes = out_bytes > stage_bytes ? out_bytes : stage_bytes;
    static bool raised = false;
    if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tiled_kernel<EPI>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
        PL_REQUIRE(e == hipSuccess, "tiled product: %zu bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
        raised = true;
    }
    gemm_tiled_kernel<EPI><<<static_cast<int>(total), 256, lds_bytes, stream>>>(
        static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), y, M, N, K, row_tiles, static_cast<int>(total), act);
    PL_CHECK_LAUNCH("gemm_tiled");
    return 0;
}

// Whether a shape is served: K a multiple of 32, N (output columns) of 128, or of 64 for SwiGLU.
extern "C" int pl_gemm_tiled_applies(int M, int N, int K, int epilogue) {
    if (M <= 0 || N <= 0 || K <= 0 || K % GT_BK) return 0;
    if (epilogue == GT_SWIGLU) return N % (GT_BN / 2) == 0;
    return (epilogue == GT_STORE || epilogue == GT_ADD) && N % GT_BN == 0;
}

// x: bfloat16 [M, K].  w: bfloat16 [N, K], or [2 N, K] with the gate rows first for epilogue 1.
// epilogue 0: y (bfloat16 [M, N]) = result.  1: y = act(gate) * up (act: PL_ACT_*).  2: y (32-bit [M, N]) += result.
extern "C" int pl_gemm_tiled(const void* x, const void* w, void* y, int M, int N, int K, int epilogue, int act, hipStream_t stream) {
    PL_REQUIRE(act >= PL_ACT_SILU && act <= PL_ACT_GELU, "tiled product: activation code %d", act);
    PL_REQUIRE(pl_gemm_tiled_applies(M, N, K, epilogue), "tiled product: %d rows, %d columns, inner width %d, epilogue %d", M, N,
               K, epilogue);
    if (epilogue == GT_SWIGLU) return gt_launch<GT_SWIGLU>(x, w, y, M, N, K, act, stream);
    if (epilogue == GT_ADD) return gt_launch<GT_ADD>(x, w, y, M, N, K, act, stream);
    return gt_launch<GT_STORE>(x, w, y, M, N, K, act, stream);
}

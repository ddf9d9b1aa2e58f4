// The entry point of the product for few rows, and its instantiations for bfloat16 rows
// (those that start with a norm are in gemm_skinny_norm.hip: two files compile side by side).
#include "gemm_skinny.hpp"

int sk_launch_norm(int epilogue, int out_f32, const void* x, const void* w, void* y, const float* gain, float eps, const int* rows, int n, int N_out, int K, int act, hipStream_t stream);

static int sk_launch_plain(int epilogue, int out_f32, const void* x, const void* w, void* y, const float* gain,
                           float eps, const int* rows, int n, int N_out, int K, int act, hipStream_t stream) {
    return sk_launch<PRO_BF16>(epilogue, out_f32, x, w, y, gain, eps, rows, n, N_out, K, act, stream);
}

// x: bfloat16 [n, K], or with a gain the 32-bit residual stream [*, K] whose rows rows[0..n) (or 0..n) are
// normalised on the way in (the gain is 32-bit).  w: bfloat16 [N_out, K], or [2*N_out, K] with gate rows first for epilogue 1.
// epilogue 0: y = result, bfloat16 or (out_f32) 32-bit.  1: y = act(gate) * up (act: PL_ACT_*).  2: y, 32-bit, += result.
extern "C" int pl_gemm_skinny(const void* x, const void* w, void* y, const float* gain, float eps,
                              const int* rows, int n, int N_out, int K, int epilogue, int out_f32, int act,
                              hipStream_t stream) {
    PL_REQUIRE(n >= 0 && n <= 64, "skinny product: %d rows, it takes up to 64", n);
    PL_REQUIRE(N_out > 0 && K > 0 && K % 8 == 0, "skinny product: %d columns, inner width %d (a multiple of 8 is needed)", N_out, K);
    PL_REQUIRE(epilogue >= EPI_STORE && epilogue <= EPI_ADD, "skinny product: epilogue code %d", epilogue);
    PL_REQUIRE(epilogue != EPI_ADD || out_f32, "skinny product: the residual stream is 32-bit");
    PL_REQUIRE(gain || !rows, "skinny product: a row list without a norm");
    PL_REQUIRE(epilogue != EPI_SWIGLU || !out_f32, "skinny product: the activation is stored in bfloat16");
    PL_REQUIRE(!(gain && epilogue == EPI_ADD), "skinny product: a product that reads the residual stream cannot add into it");
    PL_REQUIRE(act >= PL_ACT_SILU && act <= PL_ACT_GELU, "skinny product: activation code %d", act);
    if (n == 0) return 0;
    if (gain) return sk_launch_norm(epilogue, out_f32, x, w, y, gain, eps, rows, n, N_out, K, act, stream);
    return sk_launch_plain(epilogue, out_f32, x, w, y, gain, eps, rows, n, N_out, K, act, stream);
}

// The entry point of the product for few rows, and its instantiations for bfloat16 rows
// (those that start with a norm are in gemm_skinny_norm.hip: two files compile side by side).
#include "gemm_skinny.hpp"

int sk_launch_norm(int epilogue, int out_f32, const void* x, const void* w, void* y, const float* gain, float eps, const int* rows, int n, int N_out, int K, int act, int strips, hipStream_t stream);

static int sk_launch_plain(int epilogue, int out_f32, const void* x, const void* w, void* y, const float* gain,
                           float eps, const int* rows, int n, int N_out, int K, int act, const sk_extras_t& hand,
                           hipStream_t stream) {
    return sk_launch<PRO_BF16>(epilogue, out_f32, x, w, y, gain, eps, rows, n, N_out, K, act, hand, stream);
}

// x: bfloat16 [n, K], or with a gain the 32-bit residual stream [*, K] whose rows rows[0..n) (or 0..n) are
// normalised on the way in (the gain is 32-bit).  w: bfloat16 [N_out, K], or [2*N_out, K] with gate rows first for epilogue 1.
// epilogue 0: y = result, bfloat16 or (out_f32) 32-bit.  1: y = act(gate) * up (act: PL_ACT_*).  2: y, 32-bit, += result.
// strips: w holds the same weights in strips (gemm_skinny.hpp has the layout; pl_gemm_skinny_strips_apply says for
// which products that is read).
extern "C" int pl_gemm_skinny_strips_apply(int n, int N_out, int K) { return sk_strips_apply(n, N_out, K) ? 1 : 0; }

extern "C" int pl_gemm_skinny(const void* x, const void* w, void* y, const float* gain, float eps,
                              const int* rows, int n, int N_out, int K, int epilogue, int out_f32, int act,
                              int strips, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && n <= 64, "skinny product: %d rows, it takes up to 64", n);
    PL_REQUIRE(N_out > 0 && K > 0 && K % 8 == 0, "skinny product: %d columns, inner width %d (a multiple of 8 is needed)", N_out, K);
    PL_REQUIRE(epilogue >= EPI_STORE && epilogue <= EPI_ADD, "skinny product: epilogue code %d", epilogue);
    PL_REQUIRE(epilogue != EPI_ADD || out_f32, "skinny product: the residual stream is 32-bit");
    PL_REQUIRE(gain || !rows, "skinny product: a row list without a norm");
    PL_REQUIRE(epilogue != EPI_SWIGLU || !out_f32, "skinny product: the activation is stored in bfloat16");
    PL_REQUIRE(!(gain && epilogue == EPI_ADD), "skinny product: a product that reads the residual stream cannot add into it");
    PL_REQUIRE(act >= PL_ACT_SILU && act <= PL_ACT_GELU, "skinny product: activation code %d", act);
    if (n == 0) return 0;
    PL_REQUIRE(!strips || sk_strips_apply(n, N_out, K),
               "skinny product: %d rows, %d columns, width %d are not read from weights in strips", n, N_out, K);
    if (gain) return sk_launch_norm(epilogue, out_f32, x, w, y, gain, eps, rows, n, N_out, K, act, strips ? 1 : 0, stream);
    sk_extras_t with{};
    with.strips = strips ? 1 : 0;
    return sk_launch_plain(epilogue, out_f32, x, w, y, gain, eps, rows, n, N_out, K, act, with, stream);
}

// Whether a product of n bfloat16 rows of this shape can take a handed norm (taking != 0), or, for an adding
// product (epilogue 2), hand one forward (taking == 0).
extern "C" int pl_gemm_skinny_hand_applies(int n, int N_out, int K, int epilogue, int taking) {
    return sk_hand_applies(n, N_out, K, epilogue, taking != 0) ? 1 : 0;
}

// The same product of bfloat16 rows with a norm handed forward, on either side or both:
//   taken: ssq_parts [n, parts] holds sums of squares whose sum over a row is that of the K values the row was
//     normalised from; the result is scaled by 1 / sqrt(sum / K + eps) of its row (x is bf16(stream * gain)).
//   handed (epilogue 2 only): with hand_gain [N_out], bf16((y + result) * hand_gain) goes to hand_x [n, N_out]
//     and the sums of squares of the updated stream over each 16-column stripe to hand_ssq [n, ceil(N_out / 16)].
extern "C" int pl_gemm_skinny_hand(const void* x, const void* w, void* y, int n, int N_out, int K, int epilogue,
                                   int out_f32, int act, const float* ssq_parts, int parts, float eps,
                                   const float* hand_gain, void* hand_x, float* hand_ssq, int strips, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && n <= 64, "skinny product: %d rows, it takes up to 64", n);
    PL_REQUIRE(N_out > 0 && K > 0 && K % 8 == 0, "skinny product: %d columns, inner width %d (a multiple of 8 is needed)", N_out, K);
    PL_REQUIRE(epilogue >= EPI_STORE && epilogue <= EPI_ADD, "skinny product: epilogue code %d", epilogue);
    PL_REQUIRE(epilogue != EPI_ADD || out_f32, "skinny product: the residual stream is 32-bit");
    PL_REQUIRE(epilogue != EPI_SWIGLU || !out_f32, "skinny product: the activation is stored in bfloat16");
    PL_REQUIRE(act >= PL_ACT_SILU && act <= PL_ACT_GELU, "skinny product: activation code %d", act);
    PL_REQUIRE(!ssq_parts || (parts > 0 && sk_hand_applies(n, N_out, K, epilogue, true)),
               "skinny product: %d rows, %d columns, width %d take no handed norm (%d sums a row)", n, N_out, K, parts);
    PL_REQUIRE((hand_x != nullptr) == (hand_ssq != nullptr) && (hand_x != nullptr) == (hand_gain != nullptr),
               "skinny product: a norm is handed forward with its gains, rows and sums, or not at all");
    PL_REQUIRE(!hand_x || sk_hand_applies(n, N_out, K, epilogue, false),
               "skinny product: %d rows, %d columns, width %d hand no norm forward", n, N_out, K);
    if (n == 0) return 0;
    PL_REQUIRE(!strips || sk_strips_apply(n, N_out, K),
               "skinny product: %d rows, %d columns, width %d are not read from weights in strips", n, N_out, K);
    sk_extras_t hand{hand_gain, static_cast<bf16_t*>(hand_x), hand_ssq, ssq_parts, ssq_parts ? parts : 0, strips ? 1 : 0};
    return sk_launch_plain(epilogue, out_f32, x, w, y, nullptr, eps, nullptr, n, N_out, K, act, hand, stream);
}

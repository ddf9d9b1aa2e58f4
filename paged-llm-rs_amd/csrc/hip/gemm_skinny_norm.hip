// The products for few rows that start with a norm of the 32-bit residual stream.
#include "gemm_skinny.hpp"

int sk_launch_norm(int epilogue, int out_f32, const void* x, const void* w, void* y, const float* gain, float eps, const int* rows, int n, int N_out, int K, int act, int strips, hipStream_t stream) {
    sk_extras_t with{};
    with.strips = strips;
    return sk_launch<PRO_NORM>(epilogue, out_f32, x, w, y, gain, eps, rows, n, N_out, K, act, with, stream);
}

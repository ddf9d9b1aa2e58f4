// Paged attention, one wave per (token, query head), everything in 32-bit.
//
// This kernel serves every kind of row alike: a decoded token, a token of a
// prompt portion, a token of a whole prompt.  A token at position p of its
// request reads the keys 0..p (or the last `window` of them) of that request
// through the block table; the keys of its own step are already in the cache,
// because the cache write precedes attention inside a layer.  Keys are walked
// in ascending order in tiles of 64 with a running maximum and sum, so the
// result for a position does not depend on how the request was cut into steps
// or on what else is in the batch.  It is the attention of the true 32-bit
// path and the fallback for shapes the matrix-core kernels refuse.
#include "common.hpp"

#define PL_MAX_HEAD_DIM 256

template <typename T>
__global__ void __launch_bounds__(PL_WAVE)
paged_attention_plain_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out,
                             const int* __restrict__ positions, const int* __restrict__ seq_of,
                             const int* __restrict__ block_table, int max_blocks, int block_size,
                             const T* __restrict__ k_pool, const T* __restrict__ v_pool, int nq,
                             int nkv, int d, float scale, int window) {
    __shared__ float qs[PL_MAX_HEAD_DIM];
    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const int pos = positions[t];
    if (pos < 0) return;  // padding row

    const int kvh = h / (nq / nkv);
    const T* qrow = q + static_cast<size_t>(t) * q_stride + static_cast<size_t>(h) * d;
    for (int i = lane; i < d; i += PL_WAVE) qs[i] = to_float(qrow[i]);
    __syncthreads();

    const int* table = block_table + static_cast<size_t>(seq_of[t]) * max_blocks;
    const int first = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
    const int regs = (d + PL_WAVE - 1) / PL_WAVE;  // output elements per lane, at most 4

    float m = -INFINITY, l = 0.f;
    float acc[PL_MAX_HEAD_DIM / PL_WAVE] = {0.f, 0.f, 0.f, 0.f};

    for (int j0 = first; j0 <= pos; j0 += PL_WAVE) {
        const int j = j0 + lane;
        float s = -INFINITY;
        int slot = -1;
        if (j <= pos) {
            const int blk = table[j / block_size];
            if (blk >= 0) {
                slot = blk * block_size + j % block_size;
                const T* krow = k_pool + (static_cast<size_t>(slot) * nkv + kvh) * d;
                float dot = 0.f;
                for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_float(krow[i]), dot);
                s = dot * scale;
            }
        }
        const float tile_max = wave_max(s);
        const float m_new = fmaxf(m, tile_max);
        if (m_new == -INFINITY) continue;  // nothing visible yet (the same for every lane)
        const float corr = expf(m - m_new);  // exp(-inf) = 0 on the first tile
        const float p = (slot >= 0) ? expf(s - m_new) : 0.f;
        l = l * corr + wave_sum(p);
        for (int r = 0; r < regs; ++r) acc[r] *= corr;
        const int count = min(PL_WAVE, pos - j0 + 1);
        for (int jj = 0; jj < count; ++jj) {
            const float pj = __shfl(p, jj, PL_WAVE);
            const int sj = __shfl(slot, jj, PL_WAVE);
            if (sj < 0) continue;
            const T* vrow = v_pool + (static_cast<size_t>(sj) * nkv + kvh) * d;
            for (int r = 0; r < regs; ++r) {
                const int i = lane + r * PL_WAVE;
                if (i < d) acc[r] = fmaf(pj, to_float(vrow[i]), acc[r]);
            }
        }
        m = m_new;
    }
    T* orow = out + (static_cast<size_t>(t) * nq + h) * d;
    for (int r = 0; r < regs; ++r) {
        const int i = lane + r * PL_WAVE;
        if (i < d) orow[i] = from_float<T>(l > 0.f ? acc[r] / l : 0.f);
    }
}

extern "C" int pl_paged_attention_plain(const void* q, int q_stride, void* out, const int* positions,
                                        const int* seq_of, const int* block_table, int max_blocks,
                                        int block_size, const void* k_pool, const void* v_pool, int n,
                                        int nq, int nkv, int d, float scale, int window, int dtype,
                                        hipStream_t stream) {
    PL_REQUIRE(d > 0 && d <= PL_MAX_HEAD_DIM, "attention: head size %d, which has to be between 1 and %d", d, PL_MAX_HEAD_DIM);
    PL_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "attention: %d query heads over %d key heads", nq, nkv);
    PL_REQUIRE(block_size > 0 && max_blocks > 0 && q_stride >= nq * d && window >= 0,
               "attention: block size %d, %d blocks a row, query stride %d, window %d", block_size, max_blocks, q_stride, window);
    PL_REQUIRE(nq <= 65535, "attention: %d query heads are more than one launch covers", nq);
    if (n <= 0) return 0;
    dim3 grid(n, nq);
    if (dtype == PL_DTYPE_F32)
        paged_attention_plain_kernel<float><<<grid, PL_WAVE, 0, stream>>>(
            static_cast<const float*>(q), q_stride, static_cast<float*>(out), positions, seq_of, block_table, max_blocks,
            block_size, static_cast<const float*>(k_pool), static_cast<const float*>(v_pool), nq, nkv, d, scale, window);
    else if (dtype == PL_DTYPE_BF16)
        paged_attention_plain_kernel<bf16_t><<<grid, PL_WAVE, 0, stream>>>(
            static_cast<const bf16_t*>(q), q_stride, static_cast<bf16_t*>(out), positions, seq_of, block_table, max_blocks,
            block_size, static_cast<const bf16_t*>(k_pool), static_cast<const bf16_t*>(v_pool), nq, nkv, d, scale, window);
    else
        PL_REQUIRE(false, "attention: dtype code %d", dtype);
    PL_CHECK_LAUNCH("paged_attention_plain");
    return 0;
}

// Plain, sequential versions of what the GPU kernels compute, one short function each, in double
// precision over 32-bit inputs: the oracles that the kernel tests hold the kernels against, beside the
// kernels as the reference keeps its scalar oracle beside its attention kernel
// (crates/pagedllm/src/kernels/paged_attention.rs:150-210).  Nothing here is on the product path.
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <limits>
#include <vector>

extern "C" {

// out[r, :] = x[r, :] / sqrt(mean(x[r, :]^2) + eps) * gain  (model/layers.rs:58-64)
void plh_oracle_rms_norm(const float* x, const float* gain, double eps, long rows, long width, float* out) {
    for (long r = 0; r < rows; ++r) {
        double ssq = 0.0;
        for (long i = 0; i < width; ++i) ssq += static_cast<double>(x[r * width + i]) * x[r * width + i];
        const double inv = 1.0 / std::sqrt(ssq / static_cast<double>(width) + eps);
        for (long i = 0; i < width; ++i) out[r * width + i] = static_cast<float>(x[r * width + i] * inv * gain[i]);
    }
}

// Rotation of the first `rot` elements of every head of x [rows, heads, d] by the angles of each row's position:
// pairs (i, i + rot/2) (model/rope.rs:38-56), or with `neighbours` pairs (2i, 2i + 1); angle i of position p is
// p * theta^(-2i/rot).
void plh_oracle_rotate(float* x, const int* positions, long rows, long heads, long d, long rot, double theta, int neighbours) {
    const long half = rot / 2;
    for (long r = 0; r < rows; ++r)
        for (long h = 0; h < heads; ++h) {
            float* v = x + (r * heads + h) * d;
            for (long i = 0; i < half; ++i) {
                const double angle = static_cast<double>(positions[r]) * std::pow(theta, -2.0 * static_cast<double>(i) / static_cast<double>(rot));
                const double c = std::cos(angle), s = std::sin(angle);
                const long a = neighbours ? 2 * i : i, b = neighbours ? 2 * i + 1 : i + half;
                const double xa = v[a], xb = v[b];
                v[a] = static_cast<float>(xa * c - xb * s);
                v[b] = static_cast<float>(xb * c + xa * s);
            }
        }
}

// y[M, N] = x[M, K] . w[N, K]^T
void plh_oracle_product(const float* x, const float* w, long M, long N, long K, float* y) {
    for (long m = 0; m < M; ++m)
        for (long n = 0; n < N; ++n) {
            double sum = 0.0;
            for (long k = 0; k < K; ++k) sum += static_cast<double>(x[m * K + k]) * w[n * K + k];
            y[m * N + n] = static_cast<float>(sum);
        }
}

// out[r, j] = silu(gu[r, j]) * gu[r, I + j] over rows [gate | up]  (model/layers.rs:104-121)
void plh_oracle_swiglu(const float* gu, long rows, long inter, float* out) {
    for (long r = 0; r < rows; ++r)
        for (long j = 0; j < inter; ++j) {
            const double g = gu[r * 2 * inter + j], u = gu[r * 2 * inter + inter + j];
            out[r * inter + j] = static_cast<float>(g / (1.0 + std::exp(-g)) * u);
        }
}

// Attention of single rows over a paged cache.  Row t is a query [nq, d] of request seq_of[t] at position
// positions[t]; it sees the keys j <= position (and, with a window, j > position - window) of its request, whose
// key j lies in row block_table[seq, j / block_size] * block_size + j % block_size of the pools [rows, nkv, d];
// query head h reads key head h / (nq / nkv).  Scores, softmax and the weighted sum are taken in double.
// (kernels/paged_attention.rs:150-210 is the reference's oracle of the same.)  A negative position is a
// padding row and gives zeros.
void plh_oracle_paged_attention(const float* q, const float* k_pool, const float* v_pool, const int* block_table,
                                const int* positions, const int* seq_of, long rows, long nq, long nkv, long d,
                                long block_size, long max_blocks, double scale, long window, float* out) {
    const long group = nq / nkv;
    std::vector<double> score, acc(static_cast<size_t>(d));
    for (long t = 0; t < rows; ++t) {
        const long pos = positions[t];
        for (long h = 0; h < nq; ++h) {
            float* o = out + (t * nq + h) * d;
            if (pos < 0) {
                for (long e = 0; e < d; ++e) o[e] = 0.f;
                continue;
            }
            const long first = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
            const long kvh = h / group;
            const int* table = block_table + static_cast<long>(seq_of[t]) * max_blocks;
            score.assign(static_cast<size_t>(pos + 1 - first), 0.0);
            double largest = -std::numeric_limits<double>::infinity();
            for (long j = first; j <= pos; ++j) {
                const long row = static_cast<long>(table[j / block_size]) * block_size + j % block_size;
                const float* key = k_pool + (row * nkv + kvh) * d;
                double dot = 0.0;
                for (long e = 0; e < d; ++e) dot += static_cast<double>(q[(t * nq + h) * d + e]) * key[e];
                score[static_cast<size_t>(j - first)] = dot * scale;
                if (dot * scale > largest) largest = dot * scale;
            }
            double total = 0.0;
            for (double& s : score) {
                s = std::exp(s - largest);
                total += s;
            }
            for (long e = 0; e < d; ++e) acc[static_cast<size_t>(e)] = 0.0;
            for (long j = first; j <= pos; ++j) {
                const long row = static_cast<long>(table[j / block_size]) * block_size + j % block_size;
                const float* value = v_pool + (row * nkv + kvh) * d;
                const double p = score[static_cast<size_t>(j - first)] / total;
                for (long e = 0; e < d; ++e) acc[static_cast<size_t>(e)] += p * value[e];
            }
            for (long e = 0; e < d; ++e) o[e] = static_cast<float>(acc[static_cast<size_t>(e)]);
        }
    }
}

// The first largest of every row.
void plh_oracle_argmax(const float* logits, long rows, long vocab, int* out) {
    for (long r = 0; r < rows; ++r) {
        long best = 0;
        for (long i = 1; i < vocab; ++i)
            if (logits[r * vocab + i] > logits[r * vocab + best]) best = i;
        out[r] = static_cast<int>(best);
    }
}

}  // extern "C"

// Embedding gather, residual add + RMSNorm, per-head q/k norm + rotation + cache
// write, SwiGLU.  Statistics, rotation and the residual sum are 32-bit whatever
// the activation type is; a result is rounded once, when it is stored.
#include "common.hpp"

// ---------------------------------------------------------------------------
// Embedding: out[t, :] = table[ids[t], :] as the 32-bit residual stream.
// A negative id marks a padding row and gives zeros.  With `src` and `fed`, a
// row t whose src[t] is not negative takes its id from fed[src[t]] instead: the
// token that the step before chose on the device, which the host has not read
// when it launches this step.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const int* __restrict__ src,
                             const int* __restrict__ fed, const T* __restrict__ table,
                             float* __restrict__ out, int H, int V) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (src != nullptr) {
        const int from = src[t];
        if (from >= 0) id = fed[from];
    }
    float* o = out + static_cast<size_t>(t) * H;
    if (id < 0 || id >= V) {
        for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = 0.f;
        return;
    }
    const T* row = table + static_cast<size_t>(id) * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_float(row[i]);
}

// `src` and `fed` come together or not at all (both null: every id is ids[t]).
// The caller has checked that every src[t] is a row of `fed`.
extern "C" int pl_embed_fed(const int* ids, const int* src, const int* fed, const void* table, int dtype,
                            float* out, int n, int H, int V, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && H > 0 && V > 0, "embed: n %d, width %d, vocabulary %d", n, H, V);
    PL_REQUIRE((src == nullptr) == (fed == nullptr), "embed: rows fed from the step before need both the rows and the tokens");
    if (n == 0) return 0;
    const int threads = H >= 256 ? 256 : 64;
    if (dtype == PL_DTYPE_F32)
        embed_kernel<float><<<n, threads, 0, stream>>>(ids, src, fed, static_cast<const float*>(table), out, H, V);
    else if (dtype == PL_DTYPE_BF16)
        embed_kernel<bf16_t><<<n, threads, 0, stream>>>(ids, src, fed, static_cast<const bf16_t*>(table), out, H, V);
    else
        PL_REQUIRE(false, "embed: dtype code %d", dtype);
    PL_CHECK_LAUNCH("embed");
    return 0;
}

extern "C" int pl_embed(const int* ids, const void* table, int dtype, float* out, int n, int H,
                        int V, hipStream_t stream) {
    return pl_embed_fed(ids, nullptr, nullptr, table, dtype, out, n, H, V, stream);
}

// ---------------------------------------------------------------------------
// Residual add + RMSNorm.
//   x = resid[r] (+ delta[r]);  if write_resid: resid[r] = x
//   out[i] = x / sqrt(mean(x^2) + eps) * gain
// r = rows[i] when a row list is given (then nothing is written back), else i.
// One workgroup per output row; the sum of squares is reduced in a fixed order.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const T* __restrict__ delta,
                                   const void* __restrict__ gain, int gain_dtype, float eps,
                                   T* __restrict__ out, const int* __restrict__ rows, int H,
                                   int write_resid) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    float* x = resid + static_cast<size_t>(r) * H;
    const T* d = delta ? delta + static_cast<size_t>(r) * H : nullptr;
    T* o = out + static_cast<size_t>(i) * H;

    // A thread keeps up to NORM_KEEP of its elements in registers between the sum and the output, so
    // that a row is read once (wider rows read the rest again).
    constexpr int NORM_KEEP = 8;
    float kept[NORM_KEEP];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NORM_KEEP; ++k) {
        const int c = threadIdx.x + k * blockDim.x;
        float v = 0.f;
        if (c < H) {
            v = x[c];
            if (d) v += to_float(d[c]);
            if (write_resid) x[c] = v;
        }
        kept[k] = v;
        ss += v * v;
    }
    for (int c = threadIdx.x + NORM_KEEP * blockDim.x; c < H; c += blockDim.x) {
        float v = x[c];
        if (d) v += to_float(d[c]);
        if (write_resid) x[c] = v;
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float denom = sqrtf(ss / static_cast<float>(H) + eps);
#pragma unroll
    for (int k = 0; k < NORM_KEEP; ++k) {
        const int c = threadIdx.x + k * blockDim.x;
        if (c < H) o[c] = from_float<T>(kept[k] / denom * load_as_float(gain, gain_dtype, c));
    }
    for (int c = threadIdx.x + NORM_KEEP * blockDim.x; c < H; c += blockDim.x) {
        float v = x[c];
        if (d && !write_resid) v += to_float(d[c]);
        o[c] = from_float<T>(v / denom * load_as_float(gain, gain_dtype, c));
    }
}

// The same for widths that are a multiple of four, four neighbouring elements a thread and load (16 bytes of
// the 32-bit stream, 8 of bfloat16): VPT such groups a thread hold the whole row in registers.
template <typename T>
struct norm_quad;
template <>
struct norm_quad<float> {
    static __device__ __forceinline__ void load(const float* p, float* v) {
        const float4 q = *reinterpret_cast<const float4*>(p);
        v[0] = q.x, v[1] = q.y, v[2] = q.z, v[3] = q.w;
    }
    static __device__ __forceinline__ void store(float* p, const float* v) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
};
template <>
struct norm_quad<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float* v) {
        const uint2 q = *reinterpret_cast<const uint2*>(p);
        v[0] = __uint_as_float(q.x << 16), v[1] = __uint_as_float(q.x & 0xffff0000u);
        v[2] = __uint_as_float(q.y << 16), v[3] = __uint_as_float(q.y & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float* v) {
        uint2 q;
        q.x = static_cast<uint32_t>(bf16_bits_from_float(v[0])) | (static_cast<uint32_t>(bf16_bits_from_float(v[1])) << 16);
        q.y = static_cast<uint32_t>(bf16_bits_from_float(v[2])) | (static_cast<uint32_t>(bf16_bits_from_float(v[3])) << 16);
        *reinterpret_cast<uint2*>(p) = q;
    }
};

template <typename T, int VPT>
__global__ void add_rmsnorm_quads_kernel(float* __restrict__ resid, const T* __restrict__ delta,
                                         const void* __restrict__ gain, int gain_dtype, float eps,
                                         T* __restrict__ out, const int* __restrict__ rows, int H, int write_resid) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    float* x = resid + static_cast<size_t>(r) * H;
    const T* d = delta ? delta + static_cast<size_t>(r) * H : nullptr;
    T* o = out + static_cast<size_t>(i) * H;
    float kept[VPT][4];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int c = (threadIdx.x + k * blockDim.x) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) kept[k][e] = 0.f;
        if (c < H) {
            norm_quad<float>::load(x + c, kept[k]);
            if (d) {
                float dv[4];
                norm_quad<T>::load(d + c, dv);
#pragma unroll
                for (int e = 0; e < 4; ++e) kept[k][e] += dv[e];
            }
            if (write_resid) norm_quad<float>::store(x + c, kept[k]);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) ss += kept[k][e] * kept[k][e];
    }
    ss = block_sum(ss, scratch);
    const float denom = sqrtf(ss / static_cast<float>(H) + eps);
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int c = (threadIdx.x + k * blockDim.x) * 4;
        if (c < H) {
            float g[4], v[4];
            if (gain_dtype == PL_DTYPE_F32)
                norm_quad<float>::load(static_cast<const float*>(gain) + c, g);
            else
                norm_quad<bf16_t>::load(static_cast<const bf16_t*>(gain) + c, g);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = kept[k][e] / denom * g[e];
            norm_quad<T>::store(o + c, v);
        }
    }
}

template <typename T>
static bool launch_add_rmsnorm_quads(float* resid, const void* delta, const void* gain, int gain_dtype, float eps, void* out,
                                     const int* rows, int n_out, int H, int write_resid, hipStream_t stream) {
    if (H % 4) return false;
    const int quads = H / 4;
    const int threads = quads >= 512 ? 512 : (quads >= 128 ? 256 : 64);
    const int each = (quads + threads - 1) / threads;
#define NORM_QUADS(V)                                                                                                  \
    add_rmsnorm_quads_kernel<T, V><<<n_out, threads, 0, stream>>>(resid, static_cast<const T*>(delta), gain, gain_dtype, eps, \
                                                                  static_cast<T*>(out), rows, H, write_resid)
    if (each == 1) NORM_QUADS(1);
    else if (each == 2) NORM_QUADS(2);
    else if (each <= 4) NORM_QUADS(4);
    else return false;
#undef NORM_QUADS
    return true;
}

extern "C" int pl_add_rmsnorm(float* resid, const void* delta, const void* gain, int gain_dtype,
                              float eps, void* out, int dtype, const int* rows, int n_out, int H,
                              int write_resid, hipStream_t stream) {
    PL_REQUIRE(n_out >= 0 && H > 0, "add_rmsnorm: rows %d, width %d", n_out, H);
    PL_REQUIRE(!(rows && write_resid), "add_rmsnorm: a gathered call cannot write the residual back");
    PL_REQUIRE(gain_dtype == PL_DTYPE_F32 || gain_dtype == PL_DTYPE_BF16, "add_rmsnorm: gain dtype code %d", gain_dtype);
    if (n_out == 0) return 0;
    PL_REQUIRE(dtype == PL_DTYPE_F32 || dtype == PL_DTYPE_BF16, "add_rmsnorm: dtype code %d", dtype);
    const bool done = dtype == PL_DTYPE_F32
        ? launch_add_rmsnorm_quads<float>(resid, delta, gain, gain_dtype, eps, out, rows, n_out, H, write_resid, stream)
        : launch_add_rmsnorm_quads<bf16_t>(resid, delta, gain, gain_dtype, eps, out, rows, n_out, H, write_resid, stream);
    if (done) {
        PL_CHECK_LAUNCH("add_rmsnorm");
        return 0;
    }
    const int threads = H >= 2048 ? 512 : (H >= 512 ? 256 : 64);
    if (dtype == PL_DTYPE_F32)
        add_rmsnorm_kernel<float><<<n_out, threads, 0, stream>>>(
            resid, static_cast<const float*>(delta), gain, gain_dtype, eps, static_cast<float*>(out), rows, H, write_resid);
    else if (dtype == PL_DTYPE_BF16)
        add_rmsnorm_kernel<bf16_t><<<n_out, threads, 0, stream>>>(
            resid, static_cast<const bf16_t*>(delta), gain, gain_dtype, eps, static_cast<bf16_t*>(out), rows, H, write_resid);
    else
        PL_REQUIRE(false, "add_rmsnorm: dtype code %d", dtype);
    PL_CHECK_LAUNCH("add_rmsnorm");
    return 0;
}

// A projection's bias: y[r, c] += bias[c], in y's own type (the sum in 32-bit).
template <typename T, typename B>
__global__ void add_bias_kernel(T* __restrict__ y, const B* __restrict__ bias, int N, size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) y[i] = from_float<T>(to_float(y[i]) + to_float(bias[i % N]));
}

extern "C" int pl_add_bias(void* y, const void* bias, int dtype, int bias_dtype, int n, int N, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && N > 0, "add_bias: rows %d, width %d", n, N);
    const size_t count = static_cast<size_t>(n) * N;
    if (count == 0) return 0;
    const int blocks = static_cast<int>((count + 255) / 256);
    if (dtype == PL_DTYPE_F32 && bias_dtype == PL_DTYPE_F32)
        add_bias_kernel<float, float><<<blocks, 256, 0, stream>>>(static_cast<float*>(y), static_cast<const float*>(bias), N, count);
    else if (dtype == PL_DTYPE_BF16 && bias_dtype == PL_DTYPE_BF16)
        add_bias_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>(static_cast<bf16_t*>(y), static_cast<const bf16_t*>(bias), N, count);
    else if (dtype == PL_DTYPE_BF16 && bias_dtype == PL_DTYPE_F32)
        add_bias_kernel<bf16_t, float><<<blocks, 256, 0, stream>>>(static_cast<bf16_t*>(y), static_cast<const float*>(bias), N, count);
    else if (dtype == PL_DTYPE_F32 && bias_dtype == PL_DTYPE_BF16)
        add_bias_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>(static_cast<float*>(y), static_cast<const bf16_t*>(bias), N, count);
    else
        PL_REQUIRE(false, "add_bias: dtype codes %d and %d", dtype, bias_dtype);
    PL_CHECK_LAUNCH("add_bias");
    return 0;
}

// A plain residual add for blocks whose next step is not a norm: resid += delta.
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ resid, const T* __restrict__ delta, size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) resid[i] += to_float(delta[i]);
}

extern "C" int pl_residual_add(float* resid, const void* delta, int dtype, int n, int H, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && H > 0, "residual_add: rows %d, width %d", n, H);
    const size_t count = static_cast<size_t>(n) * H;
    if (count == 0) return 0;
    const int blocks = static_cast<int>((count + 255) / 256);
    if (dtype == PL_DTYPE_F32)
        residual_add_kernel<float><<<blocks, 256, 0, stream>>>(resid, static_cast<const float*>(delta), count);
    else if (dtype == PL_DTYPE_BF16)
        residual_add_kernel<bf16_t><<<blocks, 256, 0, stream>>>(resid, static_cast<const bf16_t*>(delta), count);
    else
        PL_REQUIRE(false, "residual_add: dtype code %d", dtype);
    PL_CHECK_LAUNCH("residual_add");
    return 0;
}

// ---------------------------------------------------------------------------
// Per-head RMSNorm on q and k, rotation of q and k, and the write of k and v
// into their cache slots.  One wave per (token, head) over the nq + 2*nkv heads
// of the fused projection row [q | k | v].  q is rewritten in place.
//
//   slot(t) = block_table[seq_of[t], pos / bs] * bs + pos % bs
//
// A token with a negative position is padding and is skipped.  The rotation
// pairs element i with i + rot/2 (the two halves of the head) or, told so,
// element 2 i with 2 i + 1, and uses 32-bit cos/sin tables of [max_pos, rot/2].
// ---------------------------------------------------------------------------
#define PL_MAX_HEAD_DIM 256

template <typename T>
__global__ void qk_norm_rope_kv_write_kernel(
    T* __restrict__ qkv, const void* __restrict__ q_gain, const void* __restrict__ k_gain,
    int gain_dtype, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rot, const int* __restrict__ positions,
    const int* __restrict__ seq_of, const int* __restrict__ block_table, int max_blocks,
    int block_size, T* __restrict__ k_pool, T* __restrict__ v_pool, int nq, int nkv, int d, int neighbours) {
    __shared__ float head[PL_MAX_HEAD_DIM];
    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const int pos = positions[t];
    if (pos < 0) return;

    const int row_width = (nq + 2 * nkv) * d;
    T* src = qkv + static_cast<size_t>(t) * row_width + static_cast<size_t>(h) * d;
    const bool is_q = h < nq;
    const bool is_k = !is_q && h < nq + nkv;

    T* dst = src;
    if (!is_q) {
        const int blk = block_table[static_cast<size_t>(seq_of[t]) * max_blocks + pos / block_size];
        if (blk < 0) return;  // the host refuses such a batch; never write through a hole
        const size_t slot = static_cast<size_t>(blk) * block_size + pos % block_size;
        const int kvh = is_k ? h - nq : h - nq - nkv;
        dst = (is_k ? k_pool : v_pool) + (slot * nkv + kvh) * d;
    }

    if (!is_q && !is_k) {  // v: a copy
        for (int i = lane; i < d; i += PL_WAVE) dst[i] = src[i];
        return;
    }

    const void* gain = is_q ? q_gain : k_gain;
    float ss = 0.f;
    for (int i = lane; i < d; i += PL_WAVE) {
        const float v = to_float(src[i]);
        head[i] = v;
        ss += v * v;
    }
    if (gain) {
        ss = wave_sum(ss);
        const float rinv = 1.f / sqrtf(ss / static_cast<float>(d) + eps);   // one division a head (the decode attention kernel does the same)
        __syncthreads();
        for (int i = lane; i < d; i += PL_WAVE) head[i] = head[i] * rinv * load_as_float(gain, gain_dtype, i);
    }
    __syncthreads();
    const int half = rot / 2;
    if (cos_table) {
        const float* c = cos_table + static_cast<size_t>(pos) * half;
        const float* s = sin_table + static_cast<size_t>(pos) * half;
        for (int i = lane; i < half; i += PL_WAVE) {
            // the pair that angle i turns: the two halves' elements i, or the neighbours 2 i and 2 i + 1
            const int a = neighbours ? 2 * i : i, b = neighbours ? 2 * i + 1 : i + half;
            const float x1 = head[a], x2 = head[b];
            dst[a] = from_float<T>(x1 * c[i] - x2 * s[i]);
            dst[b] = from_float<T>(x2 * c[i] + x1 * s[i]);
        }
        for (int i = rot + lane; i < d; i += PL_WAVE) dst[i] = from_float<T>(head[i]);
    } else {
        for (int i = lane; i < d; i += PL_WAVE) dst[i] = from_float<T>(head[i]);
    }
}

// The same for the common case that the rotated width is a multiple of 16: a lane holds eight
// consecutive elements of a head (one 16-byte load in bfloat16), d/8 lanes a head, so a wave works
// on several heads at once and the partner of an element in the rotation lies whole in another
// lane, d/16 lanes away.  A workgroup of four waves takes 4 * (64 / (d/8)) heads of one token.
template <typename T>
struct qk_vec;
template <>
struct qk_vec<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float* out) {
        struct __attribute__((aligned(16))) raw_t { uint32_t v[4]; };
        const raw_t raw = *reinterpret_cast<const raw_t*>(p);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            out[2 * e] = __uint_as_float(raw.v[e] << 16);
            out[2 * e + 1] = __uint_as_float(raw.v[e] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float* in) {
        struct __attribute__((aligned(16))) raw_t { uint32_t v[4]; };
        raw_t raw;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            raw.v[e] = static_cast<uint32_t>(bf16_bits_from_float(in[2 * e])) |
                       (static_cast<uint32_t>(bf16_bits_from_float(in[2 * e + 1])) << 16);
        *reinterpret_cast<raw_t*>(p) = raw;
    }
};
template <>
struct qk_vec<float> {
    struct __attribute__((aligned(16))) raw_t { float v[4]; };
    static __device__ __forceinline__ void load(const float* p, float* out) {
        const raw_t a = *reinterpret_cast<const raw_t*>(p), b = *reinterpret_cast<const raw_t*>(p + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            out[e] = a.v[e];
            out[4 + e] = b.v[e];
        }
    }
    static __device__ __forceinline__ void store(float* p, const float* in) {
        raw_t a, b;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            a.v[e] = in[e];
            b.v[e] = in[4 + e];
        }
        *reinterpret_cast<raw_t*>(p) = a;
        *reinterpret_cast<raw_t*>(p + 4) = b;
    }
};

template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_kv_write_wide_kernel(
    T* __restrict__ qkv, const void* __restrict__ q_gain, const void* __restrict__ k_gain,
    int gain_dtype, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rot, const int* __restrict__ positions,
    const int* __restrict__ seq_of, const int* __restrict__ block_table, int max_blocks,
    int block_size, T* __restrict__ k_pool, T* __restrict__ v_pool, int nq, int nkv, int d, int heads) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x % PL_WAVE;
    const int wave = threadIdx.x / PL_WAVE;
    const int pos = positions[t];
    if (pos < 0) return;

    const int lph = d / 8;                  // lanes a head
    const int hpw = PL_WAVE / lph;          // heads a wave
    const int hw = lane / lph, chunk = lane - hw * lph;
    const int row_width = (nq + 2 * nkv) * d;
    const int blk = block_table[static_cast<size_t>(seq_of[t]) * max_blocks + pos / block_size];
    const size_t slot = static_cast<size_t>(blk < 0 ? 0 : blk) * block_size + pos % block_size;

    // What does not depend on the head is fetched once: the lane's eight gains of either norm and its
    // eight angles (the partner in the rotation is the element rot/2 further on, or back).
    const int half = rot / 2, hc = half / 8;
    const bool low = chunk < hc;
    const int partner = min(max(lane + (low ? hc : -hc), 0), PL_WAVE - 1);
    const bool rotates = cos_table && chunk * 8 < rot;
    float qg[8], kg[8], c[8], sn[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        qg[e] = q_gain ? load_as_float(q_gain, gain_dtype, chunk * 8 + e) : 1.f;
        kg[e] = k_gain ? load_as_float(k_gain, gain_dtype, chunk * 8 + e) : 1.f;
        c[e] = 1.f;
        sn[e] = 0.f;
    }
    if (rotates) {
        const size_t at = static_cast<size_t>(pos) * half + (low ? chunk : chunk - hc) * 8;
        qk_vec<float>::load(cos_table + at, c);
        qk_vec<float>::load(sin_table + at, sn);
    }

    // The workgroups of a token share its heads: 4 * hpw heads make a group, a workgroup takes two
    // groups at a time (both asked for before either is worked on), gridDim.y pairs apart.
    const int per_group = 4 * hpw;
    for (int first = blockIdx.y * 2 * per_group; first < heads; first += gridDim.y * 2 * per_group) {
        T* src[2];
        T* dst[2];
        bool writes[2], plain_copy[2], normed[2], is_q[2];
        float x[2][8];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int hd = first + u * per_group + wave * hpw + hw;
            const bool active = hw < hpw && hd < heads;
            const int hh = active ? hd : 0;
            is_q[u] = hh < nq;
            const bool is_k = !is_q[u] && hh < nq + nkv;
            src[u] = qkv + static_cast<size_t>(t) * row_width + static_cast<size_t>(hh) * d + chunk * 8;
            dst[u] = src[u];
            if (!is_q[u]) {
                const int kvh = is_k ? hh - nq : hh - nq - nkv;
                dst[u] = (is_k ? k_pool : v_pool) + (slot * nkv + kvh) * d + chunk * 8;
            }
            writes[u] = active && (is_q[u] || blk >= 0);   // never write through a hole in the table
            plain_copy[u] = !is_q[u] && !is_k;             // v
            normed[u] = !plain_copy[u] && (is_q[u] ? q_gain != nullptr : k_gain != nullptr);
            qk_vec<T>::load(src[u], x[u]);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            // the sum of squares over the lanes of the head (every lane takes part in the exchange)
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) ss = fmaf(x[u][e], x[u][e], ss);
            float total = 0.f;
            const int base = hw * lph;
            for (int j = 0; j < lph; ++j) total += __shfl(ss, min(base + j, PL_WAVE - 1), PL_WAVE);
            if (normed[u]) {
                const float rinv = 1.f / sqrtf(total / static_cast<float>(d) + eps);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[u][e] = x[u][e] * rinv * (is_q[u] ? qg[e] : kg[e]);
            }
            float px[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) px[e] = __shfl(x[u][e], partner, PL_WAVE);
            if (rotates && !plain_copy[u]) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    x[u][e] = low ? x[u][e] * c[e] - px[e] * sn[e] : x[u][e] * c[e] + px[e] * sn[e];
            }
            if (writes[u]) qk_vec<T>::store(dst[u], x[u]);
        }
    }
}

// Heads of 128 elements that are rotated whole: a head is a row of 16 lanes, so the sum of squares
// and the exchange with the rotation's partner (8 lanes further on or back) go through the lanes'
// own data paths (DPP) instead of LDS.  One wave works on four heads of a token, a workgroup on 16.
__device__ __forceinline__ float qk_dpp_quad_xor1(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));   // quad_perm [1,0,3,2]
}
__device__ __forceinline__ float qk_dpp_quad_xor2(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
}
__device__ __forceinline__ float qk_dpp_half_mirror(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true));  // lane i of 8 takes 7-i
}
__device__ __forceinline__ float qk_dpp_mirror(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true));  // lane i of 16 takes 15-i
}
__device__ __forceinline__ float qk_dpp_ror8(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, true));  // lane i of 16 takes i^8
}

template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_kv_write_128_kernel(
    T* __restrict__ qkv, const void* __restrict__ q_gain, const void* __restrict__ k_gain,
    int gain_dtype, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, const int* __restrict__ positions,
    const int* __restrict__ seq_of, const int* __restrict__ block_table, int max_blocks,
    int block_size, T* __restrict__ k_pool, T* __restrict__ v_pool, int nq, int nkv, int heads) {
    constexpr int D = 128;
    const int t = blockIdx.x;
    const int pos = positions[t];
    if (pos < 0) return;
    const int hd = blockIdx.y * 16 + threadIdx.x / 16;     // this lane's head
    const int chunk = threadIdx.x % 16;                    // its eight elements of the head
    const bool active = hd < heads;
    const int hh = active ? hd : 0;
    const bool is_q = hh < nq, is_k = !is_q && hh < nq + nkv;
    T* src = qkv + static_cast<size_t>(t) * (nq + 2 * nkv) * D + static_cast<size_t>(hh) * D + chunk * 8;
    float x[8];
    qk_vec<T>::load(src, x);
    const int blk = block_table[static_cast<size_t>(seq_of[t]) * max_blocks + pos / block_size];

    const bool low = chunk < 8;
    const void* gain = is_q ? q_gain : k_gain;
    float g[8], c[8], sn[8];
    if (gain && !(!is_q && !is_k)) {
        if (gain_dtype == PL_DTYPE_F32) qk_vec<float>::load(static_cast<const float*>(gain) + chunk * 8, g);
        else qk_vec<bf16_t>::load(static_cast<const bf16_t*>(gain) + chunk * 8, g);
    }
    if (cos_table) {
        const size_t at = static_cast<size_t>(pos) * (D / 2) + (chunk & 7) * 8;
        qk_vec<float>::load(cos_table + at, c);
        qk_vec<float>::load(sin_table + at, sn);
    }

    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(x[e], x[e], ss);
    ss += qk_dpp_quad_xor1(ss);
    ss += qk_dpp_quad_xor2(ss);
    ss += qk_dpp_half_mirror(ss);
    ss += qk_dpp_mirror(ss);
    const bool is_v = !is_q && !is_k;
    if (gain && !is_v) {
        const float rinv = 1.f / sqrtf(ss / static_cast<float>(D) + eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = x[e] * rinv * g[e];
    }
    if (cos_table) {
        float px[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) px[e] = qk_dpp_ror8(x[e]);
        if (!is_v) {
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = low ? x[e] * c[e] - px[e] * sn[e] : x[e] * c[e] + px[e] * sn[e];
        }
    }
    T* dst = src;
    if (!is_q) {
        const size_t slot = static_cast<size_t>(blk < 0 ? 0 : blk) * block_size + pos % block_size;
        const int kvh = is_k ? hh - nq : hh - nq - nkv;
        dst = (is_k ? k_pool : v_pool) + (slot * nkv + kvh) * D + chunk * 8;
    }
    if (active && (is_q || blk >= 0)) qk_vec<T>::store(dst, x);   // never write through a hole in the table
}

extern "C" int pl_qk_norm_rope_kv_write(
    void* qkv, const void* q_gain, const void* k_gain, int gain_dtype, float eps,
    const float* cos_table, const float* sin_table, int rot, const int* positions,
    const int* seq_of, const int* block_table, int max_blocks, int block_size, void* k_pool,
    void* v_pool, int n, int nq, int nkv, int d, int write_kv, int dtype, int neighbours, hipStream_t stream) {
    // (any head size: the kernels that work on eight elements a lane take multiples of 16, one wave a head takes the rest)
    PL_REQUIRE(d > 0 && d <= PL_MAX_HEAD_DIM, "qk_norm_rope: head size %d, which has to be between 1 and %d", d, PL_MAX_HEAD_DIM);
    PL_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "qk_norm_rope: rotated width %d of a head of %d", rot, d);
    PL_REQUIRE(nq > 0 && nkv > 0 && block_size > 0 && max_blocks > 0,
               "qk_norm_rope: %d query heads, %d key heads, block size %d, %d blocks a row", nq, nkv, block_size, max_blocks);
    PL_REQUIRE((q_gain == nullptr) == (k_gain == nullptr), "qk_norm_rope: one of the two gains is missing");
    if (n <= 0) return 0;
    // Without the cache write (a layer that reads another layer's pages) only the query heads run.
    const int heads = write_kv ? nq + 2 * nkv : nq;
    // (neighbours: the rotation pairs elements 2 i and 2 i + 1 instead of i and i + rot/2; the kernel of one wave a
    // head takes that, the others are written for the halves)
    if (neighbours && cos_table) {
        // falls through to the last kernel
    } else if (d == 128 && (rot == 128 || !cos_table)) {
        dim3 rows(n, pl_ceil_div(heads, 16));
        if (dtype == PL_DTYPE_F32)
            qk_norm_rope_kv_write_128_kernel<float><<<rows, 256, 0, stream>>>(
                static_cast<float*>(qkv), q_gain, k_gain, gain_dtype, eps, cos_table, sin_table, positions, seq_of,
                block_table, max_blocks, block_size, static_cast<float*>(k_pool), static_cast<float*>(v_pool), nq, nkv, heads);
        else if (dtype == PL_DTYPE_BF16)
            qk_norm_rope_kv_write_128_kernel<bf16_t><<<rows, 256, 0, stream>>>(
                static_cast<bf16_t*>(qkv), q_gain, k_gain, gain_dtype, eps, cos_table, sin_table, positions, seq_of,
                block_table, max_blocks, block_size, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), nq, nkv, heads);
        else
            PL_REQUIRE(false, "qk_norm_rope: dtype code %d", dtype);
        PL_CHECK_LAUNCH("qk_norm_rope_kv_write");
        return 0;
    }
    if (rot % 16 == 0 && d % 16 == 0 && !(neighbours && cos_table)) {
        // a workgroup takes two groups of 4 * (64 / (d/8)) heads of a token at a time
        const int per_group = 4 * (PL_WAVE / (d / 8));
        dim3 wide(n, pl_ceil_div(heads, 2 * per_group));
        if (dtype == PL_DTYPE_F32)
            qk_norm_rope_kv_write_wide_kernel<float><<<wide, 256, 0, stream>>>(
                static_cast<float*>(qkv), q_gain, k_gain, gain_dtype, eps, cos_table, sin_table, rot, positions, seq_of,
                block_table, max_blocks, block_size, static_cast<float*>(k_pool), static_cast<float*>(v_pool), nq, nkv, d, heads);
        else if (dtype == PL_DTYPE_BF16)
            qk_norm_rope_kv_write_wide_kernel<bf16_t><<<wide, 256, 0, stream>>>(
                static_cast<bf16_t*>(qkv), q_gain, k_gain, gain_dtype, eps, cos_table, sin_table, rot, positions, seq_of,
                block_table, max_blocks, block_size, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), nq, nkv, d, heads);
        else
            PL_REQUIRE(false, "qk_norm_rope: dtype code %d", dtype);
        PL_CHECK_LAUNCH("qk_norm_rope_kv_write");
        return 0;
    }
    dim3 grid(n, heads);
    if (dtype == PL_DTYPE_F32)
        qk_norm_rope_kv_write_kernel<float><<<grid, PL_WAVE, 0, stream>>>(
            static_cast<float*>(qkv), q_gain, k_gain, gain_dtype, eps, cos_table, sin_table, rot, positions, seq_of,
            block_table, max_blocks, block_size, static_cast<float*>(k_pool), static_cast<float*>(v_pool), nq, nkv, d, neighbours);
    else if (dtype == PL_DTYPE_BF16)
        qk_norm_rope_kv_write_kernel<bf16_t><<<grid, PL_WAVE, 0, stream>>>(
            static_cast<bf16_t*>(qkv), q_gain, k_gain, gain_dtype, eps, cos_table, sin_table, rot, positions, seq_of,
            block_table, max_blocks, block_size, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), nq, nkv, d, neighbours);
    else
        PL_REQUIRE(false, "qk_norm_rope: dtype code %d", dtype);
    PL_CHECK_LAUNCH("qk_norm_rope_kv_write");
    return 0;
}

// ---------------------------------------------------------------------------
// The gated activation on the fused projection row [gate | up]: out = act(gate) * up (SiLU, or a GELU).
// ---------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t count, int act) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= count) return;
    const size_t row = idx / I;
    const int c = static_cast<int>(idx % I);
    const float g = to_float(gu[row * 2 * I + c]);
    const float u = to_float(gu[row * 2 * I + I + c]);
    out[idx] = from_float<T>(pl_activate<true>(g, act) * u);
}

// The same, eight consecutive elements a thread (one 16-byte load of each half in bfloat16), for
// widths that are a multiple of eight.
template <typename T>
__global__ void __launch_bounds__(256)
swiglu_wide_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t chunks, int act) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= chunks) return;
    const int per_row = I / 8;
    const size_t row = idx / per_row;
    const int c = static_cast<int>(idx - row * per_row) * 8;
    float g[8], u[8], r[8];
    qk_vec<T>::load(gu + row * 2 * I + c, g);
    qk_vec<T>::load(gu + row * 2 * I + I + c, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = pl_activate<true>(g[e], act) * u[e];
    qk_vec<T>::store(out + row * I + c, r);
}

extern "C" int pl_swiglu(const void* gu, void* out, int n, int I, int dtype, int act, hipStream_t stream) {
    PL_REQUIRE(n >= 0 && I > 0, "swiglu: rows %d, width %d", n, I);
    PL_REQUIRE(act >= PL_ACT_SILU && act <= PL_ACT_GELU, "swiglu: activation code %d", act);
    const size_t count = static_cast<size_t>(n) * I;
    if (count == 0) return 0;
    if (I % 8 == 0 && (dtype == PL_DTYPE_F32 || dtype == PL_DTYPE_BF16)) {
        const size_t chunks = count / 8;
        const int wide_blocks = static_cast<int>((chunks + 255) / 256);
        if (dtype == PL_DTYPE_F32)
            swiglu_wide_kernel<float><<<wide_blocks, 256, 0, stream>>>(static_cast<const float*>(gu), static_cast<float*>(out), I, chunks, act);
        else
            swiglu_wide_kernel<bf16_t><<<wide_blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(gu), static_cast<bf16_t*>(out), I, chunks, act);
        PL_CHECK_LAUNCH("swiglu");
        return 0;
    }
    const int blocks = static_cast<int>((count + 255) / 256);
    if (dtype == PL_DTYPE_F32)
        swiglu_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(gu), static_cast<float*>(out), I, count, act);
    else if (dtype == PL_DTYPE_BF16)
        swiglu_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(gu), static_cast<bf16_t*>(out), I, count, act);
    else
        PL_REQUIRE(false, "swiglu: dtype code %d", dtype);
    PL_CHECK_LAUNCH("swiglu");
    return 0;
}

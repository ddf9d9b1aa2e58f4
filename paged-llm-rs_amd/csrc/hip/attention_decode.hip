// Paged attention for single tokens in bfloat16: a decoded token, or a token of
// a short prompt portion, reading the keys 0..position of its request through
// the block table.  The work is a stream of the request's keys and values
// through the chip, so the kernel is built around 16-byte loads that are all in
// flight together:
//
//   grid (kv head x query-head tile, token, split).  A workgroup of four waves
//   owns one stretch of the context (split-KV) of one kv head and serves up to
//   GT of the query heads that share it, so keys and values are read once per
//   kv head, not once per query head.
//   A group of LPK lanes owns one key: each lane holds 8 of its values.  A wave
//   handles 64/LPK keys with one load instruction and four or eight such
//   instructions are issued back to back for keys and for values.
//   Softmax is online (running maximum and sum in 32-bit, base-2 exponentials
//   with log2(e) folded into the query scale).  The lane groups and waves keep
//   separate running states that are merged through LDS at the end; with more
//   than one split the partial results go to a workspace and a second kernel
//   merges them.
#include "common.hpp"

#define AD_WAVES 4

struct __attribute__((aligned(16))) u32x4 {
    uint32_t v[4];
};

__device__ __forceinline__ void unpack8(const u32x4& p, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __uint_as_float(p.v[i] << 16);
        f[2 * i + 1] = __uint_as_float(p.v[i] & 0xffff0000u);
    }
}

template <int LPK>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int off = LPK / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PL_WAVE);
    return v;
}

// What the kernel needs to normalise and rotate queries and the new key itself (a step in which every
// request brings one token): then no kernel of its own runs for that before attention.
struct ad_fuse_t {
    const void* q_gain;       // per-head norm gains, or null
    const void* k_gain;
    int gain_dtype;
    float eps;
    const float* cos_table;   // [max_pos, rot/2], or null
    const float* sin_table;
    int rot;                  // a multiple of 16
    int mode;                 // 0: q, k and v are ready; 1: q is raw; 2: q is raw, and the token's key and value
                              //    are taken raw from its row, used, and written into the cache
};

__device__ __forceinline__ void ad_load_gain8(const void* gain, int dtype, int at, float* out) {
    if (dtype == PL_DTYPE_F32) {
        struct __attribute__((aligned(16))) f4 { float v[4]; };
        const f4 a = *reinterpret_cast<const f4*>(static_cast<const float*>(gain) + at);
        const f4 b = *reinterpret_cast<const f4*>(static_cast<const float*>(gain) + at + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[i] = a.v[i];
            out[4 + i] = b.v[i];
        }
    } else {
        unpack8(*reinterpret_cast<const u32x4*>(static_cast<const bf16_t*>(gain) + at), out);
    }
}

// One head spread over LPK lanes, eight elements a lane: RMSNorm over the head, rotation by the
// token's position (the partner of an element lies rot/16 lanes away), rounding to bfloat16 as the
// stand-alone kernel stores it.  Every lane of the wave takes part in the exchanges.
template <int LPK>
__device__ __forceinline__ void ad_norm_rope8(float* x, const void* gain, const ad_fuse_t& f, int d, int dl, int pos) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss = fmaf(x[i], x[i], ss);
    ss = group_sum<LPK>(ss);
    const int at = min(dl * 8, d - 8);
    if (gain) {
        float gn[8];
        ad_load_gain8(gain, f.gain_dtype, at, gn);
        const float denom = sqrtf(ss / static_cast<float>(d) + f.eps);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = x[i] / denom * gn[i];
    }
    const int half = f.rot / 2, hc = half / 8;
    const bool low = dl < hc;
    const int lane = threadIdx.x % PL_WAVE;
    const int partner = min(max(lane + (low ? hc : -hc), 0), PL_WAVE - 1);
    float px[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) px[i] = __shfl(x[i], partner, PL_WAVE);
    if (f.cos_table && dl * 8 < f.rot) {
        const int ta = (low ? dl : dl - hc) * 8;
        float c[8], s[8];
        ad_load_gain8(f.cos_table + static_cast<size_t>(pos) * half, PL_DTYPE_F32, ta, c);
        ad_load_gain8(f.sin_table + static_cast<size_t>(pos) * half, PL_DTYPE_F32, ta, s);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = low ? x[i] * c[i] - px[i] * s[i] : x[i] * c[i] + px[i] * s[i];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = to_float(from_float<bf16_t>(x[i]));
}

// The tokens of the requests with fewer than `short_limit` tokens, counted through the requests in their
// order: which row of the step is number `slot`?  (The requests' rows follow each other.)  A step of a long
// portion beside single tokens then has workgroups for the single tokens only: one for every row of the
// portion as well, each of which would leave at once, costs the launch some 7 ns apiece.  Every thread of the
// workgroup calls this with all lanes of its wave; false: there is no such token.
__device__ __forceinline__ bool ad_find_row(int slot, const int* __restrict__ q_len, int num_seqs, int short_limit,
                                            int& row) {
    const int lane = threadIdx.x % PL_WAVE;
    int rows_before = 0, short_before = 0;
    for (int base = 0; base < num_seqs; base += PL_WAVE) {
        const int s = base + lane;
        const int count = s < num_seqs ? q_len[s] : 0;
        const int few = count < short_limit ? count : 0;
        int rows_through = count, short_through = few;
#pragma unroll
        for (int off = 1; off < PL_WAVE; off <<= 1) {
            const int a = __shfl_up(rows_through, off, PL_WAVE), b = __shfl_up(short_through, off, PL_WAVE);
            if (lane >= off) {
                rows_through += a;
                short_through += b;
            }
        }
        // (uniform, and said to be: what follows from them stays in scalar registers)
        const int rows_here = __builtin_amdgcn_readfirstlane(__shfl(rows_through, PL_WAVE - 1, PL_WAVE));
        const int short_here = __builtin_amdgcn_readfirstlane(__shfl(short_through, PL_WAVE - 1, PL_WAVE));
        if (slot < short_before + short_here) {
            const bool mine = few > 0 && slot >= short_before + short_through - few && slot < short_before + short_through;
            const int l = __ffsll(static_cast<unsigned long long>(__ballot(mine))) - 1;   // one lane says so
            row = __builtin_amdgcn_readfirstlane(rows_before + __shfl(rows_through - count, l, PL_WAVE) +
                                                 (slot - short_before - __shfl(short_through - few, l, PL_WAVE)));
            return true;
        }
        rows_before += rows_here;
        short_before += short_here;
    }
    return false;
}

// LPK: lanes a key (a power of two, LPK*8 >= d).  GT: query heads a workgroup serves.
// U: keys a lane group asks for at once.
// num_seqs > 0: blockIdx.y counts the tokens of the short requests (ad_find_row) and not the step's rows.
template <int LPK, int GT, int U>
__global__ void __launch_bounds__(256)
paged_attention_decode_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
                              float* __restrict__ part_acc, float* __restrict__ part_ml,
                              const int* __restrict__ positions, const int* __restrict__ seq_of,
                              const int* __restrict__ q_len, int short_limit, int num_seqs,
                              const int* __restrict__ block_table, int max_blocks, int block_size,
                              bf16_t* __restrict__ k_pool, bf16_t* __restrict__ v_pool, int nq,
                              int nkv, int d, float scale_log2e, int window, int splits, int tiles, ad_fuse_t fuse) {
    constexpr int KPW = PL_WAVE / LPK;  // keys a wave handles with one load
    constexpr int GROUPS = AD_WAVES * KPW;
    extern __shared__ float lds[];  // [GROUPS][GT][2] running max and sum, then [GROUPS][GT][d] accumulators

    int t = blockIdx.y;
    if (num_seqs > 0 && !ad_find_row(blockIdx.y, q_len, num_seqs, short_limit, t)) return;
    const int pos = positions[t];
    if (pos < 0) return;
    const int seq = seq_of[t];
    if (q_len && q_len[seq] >= short_limit) return;  // a long portion: the tiled kernel's

    const int g = nq / nkv;
    const int kvh = blockIdx.x / tiles;
    const int tile = blockIdx.x % tiles;
    const int h0 = kvh * g + tile * GT;               // first query head of this workgroup
    const int heads = min(GT, g - tile * GT);         // how many of the GT are real
    const int split = blockIdx.z;

    const int lane = threadIdx.x % PL_WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PL_WAVE);  // the same for the whole wave: kept scalar
    const int sub = lane / LPK;   // which of the wave's keys
    const int dl = lane % LPK;    // which 8 values of the head
    const bool d_ok = dl * 8 < d;

    // the stretch of keys of this split, in whole rounds of the workgroup
    const int first = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
    const int limit = fuse.mode == 2 ? pos : pos + 1;   // the token's own key is not in the cache yet
    const int total = max(limit - first, 0);
    constexpr int ROUND = AD_WAVES * KPW * U;
    const int per_split = pl_ceil_div(pl_ceil_div(total, splits), ROUND) * ROUND;
    const int s_begin = first + split * per_split;
    const int s_end = min(limit, s_begin + per_split);

    float qf[GT][8];
#pragma unroll
    for (int hq = 0; hq < GT; ++hq) {
        if (hq < heads && d_ok) {
            const u32x4 raw = *reinterpret_cast<const u32x4*>(q + static_cast<size_t>(t) * q_stride +
                                                              static_cast<size_t>(h0 + hq) * d + dl * 8);
            unpack8(raw, qf[hq]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) qf[hq][i] = 0.f;
        }
    }
    // The queries are normalised, rotated and scaled once the first keys and values have been asked
    // for, so that this work passes while they are on their way.
    bool q_ready = false;
    auto prepare_q = [&]() {
#pragma unroll
        for (int hq = 0; hq < GT; ++hq) {
            if (fuse.mode != 0) ad_norm_rope8<LPK>(qf[hq], fuse.q_gain, fuse, d, dl, pos);
#pragma unroll
            for (int i = 0; i < 8; ++i) qf[hq][i] *= scale_log2e;
        }
        q_ready = true;
    };

    float m[GT], l[GT], acc[GT][8];
#pragma unroll
    for (int hq = 0; hq < GT; ++hq) {
        m[hq] = -INFINITY;
        l[hq] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[hq][i] = 0.f;
    }

    const int* table = block_table + static_cast<size_t>(seq) * max_blocks;
    const size_t row_stride = static_cast<size_t>(nkv) * d;
    const size_t head_off = static_cast<size_t>(kvh) * d + min(dl * 8, d - 8);
    // floor(2^32 / block_size): the high half of j * bs_magic is j / block_size or one less
    const uint32_t bs_magic = block_size == 1 ? 0xffffffffu : static_cast<uint32_t>(0x100000000ull / static_cast<uint32_t>(block_size));

    // Loads are unconditional, from an address that is valid in any case, and masked afterwards:
    // a load inside a branch is waited for at the branch's end, one after the other.  The pages
    // of a round are looked up during the round before, so that no load waits for another.
    int blk[U], within[U];
    auto lookup = [&](int base) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = base + u * KPW + sub;
            const bool in = j < s_end;
            const int jj = in ? j : pos;                          // the token's own place always has a page
            int bi = static_cast<int>(__umulhi(static_cast<uint32_t>(jj), bs_magic));
            int w = jj - bi * block_size;
            const int low = w >= block_size ? 1 : 0;              // the estimate is the quotient or one less
            bi += low;
            w -= low * block_size;
            const int got = table[bi];
            blk[u] = in ? got : -1;
            within[u] = w;
        }
    };
    const int first_base = s_begin + wave * KPW * U;
    lookup(first_base);
    // The keys and values of a round are asked for a round ahead, while those of the round before are
    // worked on: what comes back is held raw and masked only where it is used, so nothing waits early.
    u32x4 knext[U], vnext[U];
    bool oknext[U];
    auto ask = [&]() {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            oknext[u] = blk[u] >= 0;
            const size_t off = (static_cast<size_t>(max(blk[u], 0)) * block_size + within[u]) * row_stride + head_off;
            knext[u] = *reinterpret_cast<const u32x4*>(k_pool + off);
            vnext[u] = *reinterpret_cast<const u32x4*>(v_pool + off);
        }
    };
    ask();
    lookup(first_base + ROUND);

    for (int base = first_base; base < s_end; base += ROUND) {
        u32x4 kraw[U], vraw[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            ok[u] = oknext[u];
            kraw[u] = knext[u];
            vraw[u] = vnext[u];
        }
        ask();
        lookup(base + 2 * ROUND);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t keep = (ok[u] && d_ok) ? 0xffffffffu : 0u;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                kraw[u].v[w] &= keep;
                vraw[u].v[w] &= keep;
            }
        }
        if (!q_ready) prepare_q();
        float s[U][GT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float kf[8];
            unpack8(kraw[u], kf);
#pragma unroll
            for (int hq = 0; hq < GT; ++hq) {
                float dot = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) dot = fmaf(qf[hq][i], kf[i], dot);
                dot = group_sum<LPK>(dot);
                s[u][hq] = ok[u] ? dot : -INFINITY;
            }
        }
#pragma unroll
        for (int hq = 0; hq < GT; ++hq) {
            float m_new = m[hq];
#pragma unroll
            for (int u = 0; u < U; ++u) m_new = fmaxf(m_new, s[u][hq]);
            if (m_new == -INFINITY) continue;  // nothing seen yet by this lane group
            const float corr = exp2f(m[hq] - m_new);
            float p[U];
            float psum = 0.f;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                p[u] = exp2f(s[u][hq] - m_new);
                psum += p[u];
            }
            l[hq] = l[hq] * corr + psum;
            m[hq] = m_new;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[hq][i] *= corr;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float vf[8];
                unpack8(vraw[u], vf);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[hq][i] = fmaf(p[u], vf[i], acc[hq][i]);
            }
        }
    }

    // The token's own key and value, raw in its row: normalised and rotated here, taken into the
    // running state of one lane group of the last split, and written into the cache by one workgroup.
    if (!q_ready) prepare_q();
    if (fuse.mode == 2 && split == splits - 1 && wave == 0) {
        const bf16_t* row = q + static_cast<size_t>(t) * q_stride;
        const int at = min(dl * 8, d - 8);
        const u32x4 kraw = *reinterpret_cast<const u32x4*>(row + static_cast<size_t>(nq + kvh) * d + at);
        const u32x4 vraw = *reinterpret_cast<const u32x4*>(row + static_cast<size_t>(nq + nkv + kvh) * d + at);
        float kf[8], vf[8];
        unpack8(kraw, kf);
        unpack8(vraw, vf);
        if (!d_ok) {
#pragma unroll
            for (int i = 0; i < 8; ++i) kf[i] = vf[i] = 0.f;
        }
        ad_norm_rope8<LPK>(kf, fuse.k_gain, fuse, d, dl, pos);
        int bi = static_cast<int>(__umulhi(static_cast<uint32_t>(pos), bs_magic));
        int w = pos - bi * block_size;
        if (w >= block_size) {
            bi += 1;
            w -= block_size;
        }
        const int page = table[bi];
        if (tile == 0 && sub == 0 && d_ok && page >= 0) {
            const size_t off = (static_cast<size_t>(page) * block_size + w) * row_stride + static_cast<size_t>(kvh) * d + dl * 8;
            u32x4 packed;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                packed.v[i] = static_cast<uint32_t>(bf16_bits_from_float(kf[2 * i])) |
                              (static_cast<uint32_t>(bf16_bits_from_float(kf[2 * i + 1])) << 16);
            *reinterpret_cast<u32x4*>(k_pool + off) = packed;
            *reinterpret_cast<u32x4*>(v_pool + off) = vraw;
        }
#pragma unroll
        for (int hq = 0; hq < GT; ++hq) {
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) dot = fmaf(qf[hq][i], kf[i], dot);
            dot = group_sum<LPK>(dot);
            const float sc = (sub == 0 && page >= 0) ? dot : -INFINITY;
            const float m_new = fmaxf(m[hq], sc);
            if (m_new == -INFINITY) continue;
            const float corr = exp2f(m[hq] - m_new);
            const float p = exp2f(sc - m_new);
            l[hq] = l[hq] * corr + p;
            m[hq] = m_new;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[hq][i] = fmaf(p, vf[i], acc[hq][i] * corr);
        }
    }

    // merge the lane groups of the four waves
    float* ml = lds;                              // [GROUPS][GT][2]
    float* accs = lds + GROUPS * GT * 2;          // [GROUPS][GT][d]
    const int group = wave * KPW + sub;
#pragma unroll
    for (int hq = 0; hq < GT; ++hq) {
        if (dl == 0) {
            ml[(group * GT + hq) * 2] = m[hq];
            ml[(group * GT + hq) * 2 + 1] = l[hq];
        }
        if (d_ok) {
#pragma unroll
            for (int i = 0; i < 8; ++i) accs[(static_cast<size_t>(group) * GT + hq) * d + dl * 8 + i] = acc[hq][i];
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < heads * d; idx += blockDim.x) {
        const int hq = idx / d, dd = idx % d;
        float big = -INFINITY;
        for (int gr = 0; gr < GROUPS; ++gr) big = fmaxf(big, ml[(gr * GT + hq) * 2]);
        float sum = 0.f, a = 0.f;
        if (big != -INFINITY) {
            for (int gr = 0; gr < GROUPS; ++gr) {
                const float mg = ml[(gr * GT + hq) * 2];
                if (mg == -INFINITY) continue;
                const float w = exp2f(mg - big);
                sum += ml[(gr * GT + hq) * 2 + 1] * w;
                a += accs[(static_cast<size_t>(gr) * GT + hq) * d + dd] * w;
            }
        }
        const int h = h0 + hq;
        if (splits == 1) {
            out[(static_cast<size_t>(t) * nq + h) * d + dd] = from_float<bf16_t>(sum > 0.f ? a / sum : 0.f);
        } else {
            const size_t pi = (static_cast<size_t>(t) * nq + h) * splits + split;
            part_acc[pi * d + dd] = a;
            if (dd == 0) {
                part_ml[pi * 2] = big;
                part_ml[pi * 2 + 1] = sum;
            }
        }
    }
}

// Merges the splits of one (token, query head): out = sum_s a_s 2^(m_s - M) / sum_s l_s 2^(m_s - M).
// (The merge is a kernel of its own because the end of a kernel is the cheapest way on this chip to make
// one workgroup's results visible to another: a device-wide fence inside a kernel writes back and
// invalidates a whole L2.)  One thread an output element; every load is asked for before any is used.
#define AD_MAX_SPLITS 64

template <int SP>
__global__ void __launch_bounds__(256)
paged_attention_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                             bf16_t* __restrict__ out, const int* __restrict__ positions,
                             const int* __restrict__ seq_of, const int* __restrict__ q_len, int short_limit,
                             int nq, int d, int splits, int n, int num_seqs) {
    const int per_token = nq * d;
    int t, rest;
    bool inside;
    if (num_seqs > 0) {      // blockIdx.y counts the tokens of the short requests, blockIdx.x a token's elements
        if (!ad_find_row(blockIdx.y, q_len, num_seqs, short_limit, t)) return;
        rest = blockIdx.x * blockDim.x + threadIdx.x;
        inside = rest < per_token;
        rest = min(rest, per_token - 1);
    } else {
        const int idx = blockIdx.x * blockDim.x + threadIdx.x;
        t = min(idx / per_token, n - 1);
        rest = idx - t * per_token;
        inside = idx < n * per_token;
    }
    const int h = rest / d, dd = rest - h * d;
    const size_t base = (static_cast<size_t>(t) * nq + h) * splits;
    const int pos = positions[t];
    const int len = q_len ? q_len[seq_of[t]] : 0;
    float ms[SP], ls[SP], as[SP];
#pragma unroll
    for (int s = 0; s < SP; ++s) {
        const int sc = min(s, splits - 1);
        ms[s] = part_ml[(base + sc) * 2];
        ls[s] = part_ml[(base + sc) * 2 + 1];
        as[s] = part_acc[(base + sc) * d + dd];
    }
    if (!inside || pos < 0 || (q_len && len >= short_limit)) return;
    float big = -INFINITY;
#pragma unroll
    for (int s = 0; s < SP; ++s) big = fmaxf(big, s < splits ? ms[s] : -INFINITY);
    float sum = 0.f, a = 0.f;
#pragma unroll
    for (int s = 0; s < SP; ++s) {
        const float w = (s < splits && ms[s] != -INFINITY) ? exp2f(ms[s] - big) : 0.f;
        sum = fmaf(ls[s], w, sum);
        a = fmaf(as[s], w, a);
    }
    out[(static_cast<size_t>(t) * nq + h) * d + dd] = from_float<bf16_t>(sum > 0.f ? a / sum : 0.f);
}

template <int LPK, int GT>
static int launch_decode(const void* q, int q_stride, void* out, float* part_acc, float* part_ml,
                         const int* positions, const int* seq_of, const int* q_len, int short_limit, int num_seqs,
                         int short_rows, const int* block_table, int max_blocks, int block_size, void* k_pool,
                         void* v_pool, int n, int nq, int nkv, int d, float scale, int window, int splits,
                         const ad_fuse_t& fuse, hipStream_t stream) {
    constexpr int KPW = PL_WAVE / LPK;
    constexpr int GROUPS = AD_WAVES * KPW;
    constexpr int U = GT <= 2 ? 4 : 2;   // keys a round; as many again are in flight for the round after
    const int g = nq / nkv;
    const int tiles = pl_ceil_div(g, GT);
    const size_t lds_bytes = (static_cast<size_t>(GROUPS) * GT * 2 + static_cast<size_t>(GROUPS) * GT * d) * sizeof(float);
    PL_REQUIRE(lds_bytes <= 160 * 1024, "decode attention: %zu bytes of LDS for head size %d", lds_bytes, d);
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&paged_attention_decode_kernel<LPK, GT, U>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
        PL_REQUIRE(e == hipSuccess, "decode attention: %zu bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
    }
    // rows of the grid: the step's rows, or, where fewer, the tokens that the short requests can bring
    const bool compact = q_len != nullptr && num_seqs > 0 && short_rows > 0 && short_rows < n;
    dim3 grid(nkv * tiles, compact ? short_rows : n, splits);
    PL_REQUIRE(n <= 65535 && splits <= 65535, "decode attention: %d tokens or %d splits are more than one launch covers", n, splits);
    paged_attention_decode_kernel<LPK, GT, U><<<grid, 256, lds_bytes, stream>>>(
        static_cast<const bf16_t*>(q), q_stride, static_cast<bf16_t*>(out), part_acc, part_ml, positions, seq_of,
        q_len, short_limit, compact ? num_seqs : 0, block_table, max_blocks, block_size, static_cast<bf16_t*>(k_pool),
        static_cast<bf16_t*>(v_pool), nq, nkv, d, scale * 1.4426950408889634f, window, splits, tiles, fuse);
    PL_CHECK_LAUNCH("paged_attention_decode");
    if (splits > 1) {
        const dim3 mgrid = compact ? dim3(pl_ceil_div(nq * d, 256), short_rows) : dim3(pl_ceil_div(n * nq * d, 256));
#define AD_MERGE(SP)                                                                                              \
    paged_attention_merge_kernel<SP><<<mgrid, 256, 0, stream>>>(part_acc, part_ml, static_cast<bf16_t*>(out),     \
                                                                positions, seq_of, q_len, short_limit, nq, d,     \
                                                                splits, n, compact ? num_seqs : 0)
        if (splits <= 4) AD_MERGE(4);
        else if (splits <= 8) AD_MERGE(8);
        else if (splits <= 16) AD_MERGE(16);
        else AD_MERGE(AD_MAX_SPLITS);
#undef AD_MERGE
        PL_CHECK_LAUNCH("paged_attention_merge");
    }
    return 0;
}

template <int LPK>
static int dispatch_gt(int gt, const void* q, int q_stride, void* out, float* part_acc, float* part_ml,
                       const int* positions, const int* seq_of, const int* q_len, int short_limit, int num_seqs,
                       int short_rows, const int* block_table, int max_blocks, int block_size, void* k_pool,
                       void* v_pool, int n, int nq, int nkv, int d, float scale, int window, int splits,
                       const ad_fuse_t& fuse, hipStream_t stream) {
#define AD_CALL(G)                                                                                              \
    return launch_decode<LPK, G>(q, q_stride, out, part_acc, part_ml, positions, seq_of, q_len, short_limit,   \
                                 num_seqs, short_rows, block_table, max_blocks, block_size, k_pool, v_pool, n, nq, nkv, d, scale,    \
                                 window, splits, fuse, stream)
    switch (gt) {
        case 1: AD_CALL(1);
        case 2: AD_CALL(2);
        case 4: AD_CALL(4);
        default: AD_CALL(8);
    }
#undef AD_CALL
}

// bfloat16 only.  With splits > 1 the workspace needs n*nq*splits*d floats (part_acc) and n*nq*splits*2 (part_ml).
// q_len (may be null) and short_limit leave the tokens of requests with q_len >= short_limit to the tiled kernel.
// With q_len: num_seqs, the requests whose rows follow each other in q from row 0 on, and short_rows, the most
// tokens that the other requests bring together (0: not known); where that is fewer than the step's rows the
// launch has workgroups for those tokens only.
// fuse_mode 0: the rows of q are ready and the cache holds every key up to each token's own.  1: the rows of q are
// the raw projection and are normalised (gains, eps) and rotated (tables, rot a multiple of 16) here.  2: as 1, and
// each token's key and value are taken raw from its row [q | k | v], used, and written into the cache; every
// request then has to bring exactly one token.
extern "C" int pl_paged_attention_decode(const void* q, int q_stride, void* out, float* part_acc, float* part_ml,
                                         const int* positions, const int* seq_of, const int* q_len, int short_limit,
                                         int num_seqs, int short_rows,
                                         const int* block_table, int max_blocks, int block_size, void* k_pool,
                                         void* v_pool, int n, int nq, int nkv, int d, float scale, int window,
                                         int splits, int fuse_mode, const void* q_gain, const void* k_gain,
                                         int gain_dtype, float eps, const float* cos_table, const float* sin_table,
                                         int rot, hipStream_t stream) {
    PL_REQUIRE(d > 0 && d <= 256 && d % 16 == 0, "decode attention: head size %d, which has to be a multiple of 16 up to 256", d);
    PL_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "decode attention: %d query heads over %d key heads", nq, nkv);
    PL_REQUIRE(block_size > 0 && max_blocks > 0 && q_stride >= nq * d && q_stride % 8 == 0 && window >= 0 && splits >= 1 && splits <= AD_MAX_SPLITS,
               "decode attention: block size %d, %d blocks a row, query stride %d, window %d, %d splits", block_size,
               max_blocks, q_stride, window, splits);
    PL_REQUIRE(splits == 1 || (part_acc && part_ml), "decode attention: %d splits without a workspace", splits);
    PL_REQUIRE(fuse_mode >= 0 && fuse_mode <= 2, "decode attention: fuse mode %d", fuse_mode);
    if (fuse_mode != 0) {
        PL_REQUIRE(rot >= 0 && rot <= d && rot % 16 == 0, "decode attention: a rotated width of %d of a head of %d is not fused", rot, d);
        PL_REQUIRE((q_gain == nullptr) == (k_gain == nullptr), "decode attention: one of the two gains is missing");
        PL_REQUIRE(!q_gain || gain_dtype == PL_DTYPE_F32 || gain_dtype == PL_DTYPE_BF16, "decode attention: gain dtype code %d", gain_dtype);
        PL_REQUIRE((cos_table == nullptr) == (sin_table == nullptr) && (cos_table || rot == 0), "decode attention: rotation tables");
        PL_REQUIRE(fuse_mode != 2 || (q_len == nullptr && q_stride >= (nq + 2 * nkv) * d),
                   "decode attention: the fused cache write is for steps of one token a request over rows [q | k | v]");
    }
    const ad_fuse_t fuse{q_gain, k_gain, gain_dtype, eps, cos_table, sin_table, rot, fuse_mode};
    if (n <= 0) return 0;
    const int g = nq / nkv;
    const int gt = g >= 8 ? 8 : (g > 2 ? 4 : g);   // 1, 2, 4 or 8 query heads a workgroup; the rest are more tiles
    const int chunks = d / 8;
#define AD_LPK(L)                                                                                                  \
    return dispatch_gt<L>(gt, q, q_stride, out, part_acc, part_ml, positions, seq_of, q_len, short_limit,        \
                          num_seqs, short_rows, block_table, max_blocks, block_size, k_pool, v_pool, n, nq, nkv, d, scale, window,      \
                          splits, fuse, stream)
    if (chunks <= 2) AD_LPK(2);
    if (chunks <= 4) AD_LPK(4);
    if (chunks <= 8) AD_LPK(8);
    if (chunks <= 16) AD_LPK(16);
    AD_LPK(32);
#undef AD_LPK
}

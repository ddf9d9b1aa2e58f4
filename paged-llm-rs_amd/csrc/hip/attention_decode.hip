// Paged attention for single tokens in bfloat16: a decoded token, or a token of
// a short prompt portion, reading the keys 0..position of its request through
// the block table.  The work is a stream of the request's keys and values
// through the chip, so the kernel is built around 16-byte loads that are all in
// flight together:
//
//   grid (kv head x query-head tile, token, split).  A workgroup of four or eight
//   waves owns one stretch of the context (split-KV) of one kv head and serves up to
//   GT of the query heads that share it, so keys and values are read once per
//   kv head, not once per query head.
//   A group of LPK lanes owns one key: each lane holds 8 of its values.  A wave
//   handles 64/LPK keys with one load instruction and four or eight such
//   instructions are issued back to back for keys and for values.
//   Softmax is online (running maximum and sum in 32-bit, base-2 exponentials
//   with log2(e) folded into the query scale).  The lane groups and waves keep
//   separate running states; a wave's are merged in its registers and the waves'
//   through LDS at the end; with more than one split the partial results go to a
//   workspace and a second kernel merges them.
#include "common.hpp"


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

// Sum over the LPK lanes of a key.  Sixteen lanes are a row of the wave's data-parallel primitives: the
// sum then runs on the vector unit alone (four rotations within the row), without a trip through LDS.
template <int LPK>
__device__ __forceinline__ float key_sum(float v) {
    if constexpr (LPK == 16) {
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));  // row_ror:8
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));  // row_ror:4
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));  // row_ror:2
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));  // row_ror:1
        return v;
    } else {
        return group_sum<LPK>(v);
    }
}

// What a lane needs of the norm's gains and the rotation's angles for its eight elements of a head, asked
// for before anything else so that the norm waits for no load of its own.
struct ad_prep_t {
    float gain[8];
    float c[8], s[8];
};

__device__ __forceinline__ void ad_load_prep(ad_prep_t& p, const void* gain, const ad_fuse_t& f, int d, int dl, int pos) {
    const int at = min(dl * 8, d - 8);
    if (gain) ad_load_gain8(gain, f.gain_dtype, at, p.gain);
    const int half = f.rot / 2, hc = half / 8;
    if (f.cos_table && dl * 8 < f.rot) {
        const int ta = (dl < hc ? dl : dl - hc) * 8;
        ad_load_gain8(f.cos_table + static_cast<size_t>(pos) * half, PL_DTYPE_F32, ta, p.c);
        ad_load_gain8(f.sin_table + static_cast<size_t>(pos) * half, PL_DTYPE_F32, ta, p.s);
    }
}

// One head spread over LPK lanes, eight elements a lane: RMSNorm over the head, rotation by the
// token's position (the partner of an element lies rot/16 lanes away), rounding to bfloat16 as the
// stand-alone kernel stores it.  Every lane of the wave takes part in the exchanges.
template <int LPK>
__device__ __forceinline__ void ad_norm_rope8(float* x, bool with_gain, const ad_prep_t& p, const ad_fuse_t& f, int d, int dl) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss = fmaf(x[i], x[i], ss);
    ss = key_sum<LPK>(ss);
    if (with_gain) {
        const float rinv = 1.f / sqrtf(ss / static_cast<float>(d) + f.eps);   // (as the stand-alone kernel computes it)
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = x[i] * rinv * p.gain[i];
    }
    const int half = f.rot / 2, hc = half / 8;
    const bool low = dl < hc;
    float px[8];
    if (LPK == 16 && hc == 8) {
        // a head of 128 rotated whole: the partner lies eight lanes on in the row of sixteen
#pragma unroll
        for (int i = 0; i < 8; ++i)
            px[i] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x[i]), 0x128, 0xf, 0xf, false));
    } else {
        const int lane = threadIdx.x % PL_WAVE;
        const int partner = min(max(lane + (low ? hc : -hc), 0), PL_WAVE - 1);
#pragma unroll
        for (int i = 0; i < 8; ++i) px[i] = __shfl(x[i], partner, PL_WAVE);
    }
    if (f.cos_table && dl * 8 < f.rot) {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = low ? x[i] * p.c[i] - px[i] * p.s[i] : x[i] * p.c[i] + px[i] * p.s[i];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = to_float(from_float<bf16_t>(x[i]));
}

typedef __bf16 ad_bf16x2 __attribute__((ext_vector_type(2)));

// a . b over two bfloat16 pairs held in one word each, added to c in 32-bit (v_dot2c_f32_bf16)
__device__ __forceinline__ float ad_dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(ad_bf16x2, a), __builtin_bit_cast(ad_bf16x2, b), c, false);
}

__device__ __forceinline__ uint32_t ad_pack2(float lo, float hi) {
    return static_cast<uint32_t>(bf16_bits_from_float(lo)) | (static_cast<uint32_t>(bf16_bits_from_float(hi)) << 16);
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

// The pages of a workgroup's stretch of keys are copied into LDS first, this many at most; a longer
// stretch looks its pages up in the table itself.
#define AD_PAGES_LDS 2048

// LPK: lanes a key (a power of two, LPK*8 >= d).  GT: query heads a workgroup serves.
// U: keys a lane group asks for at once.  WV: waves a workgroup.
// num_seqs > 0: blockIdx.y counts the tokens of the short requests (ad_find_row) and not the step's rows.
//
// The kernel's time with few tokens is the length of its chain of dependent trips to memory and the
// number of instructions a wave issues (four cycles each).  The chain is kept at three: the token's position and request (scalar loads); then, together, the pages of the
// workgroup's stretch (into LDS), the query row, the norm's gains, the rotation's angles and, when it is
// to be written, the token's own raw key and value; then keys and values, two rounds of them in flight
// at all times with nothing else between them in the queue of loads (page numbers come from LDS, so no
// round waits behind a table lookup).  Queries and the own key are normalised and rotated while the
// first two rounds are on their way.
template <int LPK, int GT, int U, int WV>
__global__ void __launch_bounds__(64 * WV)
paged_attention_decode_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
                              float* __restrict__ part_acc, float* __restrict__ part_ml,
                              const int* __restrict__ positions, const int* __restrict__ seq_of,
                              const int* __restrict__ q_len, int short_limit, int num_seqs,
                              const int* __restrict__ block_table, int max_blocks, int block_size,
                              bf16_t* __restrict__ k_pool, bf16_t* __restrict__ v_pool, int nq,
                              int nkv, int d, float scale_log2e, int window, int splits, int tiles, int g,
                              uint32_t splits_magic, ad_fuse_t fuse) {
    constexpr int KPW = PL_WAVE / LPK;  // keys a wave handles with one load
    constexpr int ROUND = WV * KPW * U;
    extern __shared__ float lds[];      // [AD_PAGES_LDS] page numbers, then [WV][GT][2] running max and sum, [WV][GT][d] accumulators
    int* pages_lds = reinterpret_cast<int*>(lds);
    float* ml = lds + AD_PAGES_LDS;               // [WV][GT][2]
    float* accs = ml + WV * GT * 2;               // [WV][GT][d]

    int t = blockIdx.y;
    if (num_seqs > 0 && !ad_find_row(blockIdx.y, q_len, num_seqs, short_limit, t)) return;
    const int pos = positions[t];
    if (pos < 0) return;
    const int seq = seq_of[t];
    if (q_len && q_len[seq] >= short_limit) return;  // a long portion: the tiled kernel's

    // (g = nq / nkv and splits_magic = ceil(2^32 / splits) come from the launch: a division by a number that the
    // kernel learns only when it runs is some thirty instructions, and these stood in front of its first loads)
    const int kvh = tiles == 1 ? static_cast<int>(blockIdx.x) : static_cast<int>(blockIdx.x) / tiles;
    const int tile = tiles == 1 ? 0 : static_cast<int>(blockIdx.x) % tiles;
    const int h0 = kvh * g + tile * GT;               // first query head of this workgroup
    const int heads = min(GT, g - tile * GT);         // how many of the GT are real
    const int split = blockIdx.z;

    const int lane = threadIdx.x % PL_WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PL_WAVE);  // the same for the whole wave: kept scalar
    const int sub = lane / LPK;   // which of the wave's keys
    const int dl = lane % LPK;    // which 8 values of the head
    const bool d_ok = dl * 8 < d;
    const int at8 = min(dl * 8, d - 8);

    // the stretch of keys of this split, in whole rounds of the workgroup
    const int first = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
    const int limit = fuse.mode == 2 ? pos : pos + 1;   // the token's own key is not in the cache yet
    const int total = max(limit - first, 0);
    // ceil(total / splits): the high half of (total + splits - 1) * ceil(2^32 / splits), exact below 2^32 / splits
    const int share = splits == 1 ? total : static_cast<int>(__umulhi(static_cast<uint32_t>(total + splits - 1), splits_magic));
    const int per_split = pl_ceil_div(share, ROUND) * ROUND;
    const int s_begin = first + split * per_split;
    const int s_end = min(limit, s_begin + per_split);
    const int rounds = s_end > s_begin ? pl_ceil_div(s_end - s_begin, ROUND) : 0;

    const int* table = block_table + static_cast<size_t>(seq) * max_blocks;
    const size_t row_stride = static_cast<size_t>(nkv) * d;
    const size_t head_off = static_cast<size_t>(kvh) * d + at8;
    // floor(2^32 / block_size): the high half of j * bs_magic is j / block_size or one less
    const uint32_t bs_magic = block_size == 1 ? 0xffffffffu : static_cast<uint32_t>(0x100000000ull / static_cast<uint32_t>(block_size));
    auto page_of = [&](int j, int& w) -> int {          // which entry of the table holds key j, and its place in the page
        int bi = static_cast<int>(__umulhi(static_cast<uint32_t>(j), bs_magic));
        w = j - bi * block_size;
        const int low = w >= block_size ? 1 : 0;        // the estimate is the quotient or one less
        w -= low * block_size;
        return bi + low;
    };

    // ---- everything that does not wait for anything but the position, asked for at once ----
    int unused;
    const int page_first = rounds > 0 ? page_of(s_begin, unused) : 0;
    const int page_count = rounds > 0 ? page_of(s_end - 1, unused) - page_first + 1 : 0;
    const bool pages_in_lds = page_count <= AD_PAGES_LDS;
    int page_got[AD_PAGES_LDS / (64 * WV) > 0 ? AD_PAGES_LDS / (64 * WV) : 1];
    constexpr int PAGE_TURNS = AD_PAGES_LDS / (64 * WV) > 0 ? AD_PAGES_LDS / (64 * WV) : 1;
    if (pages_in_lds) {
#pragma unroll
        for (int i = 0; i < PAGE_TURNS; ++i) {
            const int e = static_cast<int>(threadIdx.x) + i * 64 * WV;
            page_got[i] = table[page_first + min(e, max(page_count - 1, 0))];
        }
    }
    u32x4 qraw[GT];
#pragma unroll
    for (int hq = 0; hq < GT; ++hq)
        qraw[hq] = *reinterpret_cast<const u32x4*>(q + static_cast<size_t>(t) * q_stride +
                                                   static_cast<size_t>(h0 + min(hq, heads - 1)) * d + at8);
    // the token's own key and value (taken raw from its row by the first wave of the last split), and its page
    const bool own = fuse.mode == 2 && split == splits - 1 && wave == 0;
    u32x4 own_k = {{0u, 0u, 0u, 0u}}, own_v = {{0u, 0u, 0u, 0u}};
    int own_page = -1, own_within = 0;
    if (own) {
        const bf16_t* row = q + static_cast<size_t>(t) * q_stride;
        own_k = *reinterpret_cast<const u32x4*>(row + static_cast<size_t>(nq + kvh) * d + at8);
        own_v = *reinterpret_cast<const u32x4*>(row + static_cast<size_t>(nq + nkv + kvh) * d + at8);
        own_page = table[page_of(pos, own_within)];
    }
    ad_prep_t prep_q, prep_k;
    if (fuse.mode != 0) {
        ad_load_prep(prep_q, fuse.q_gain, fuse, d, dl, pos);
        if (own) {
            prep_k = prep_q;                                   // the same angles
            if (fuse.k_gain) ad_load_gain8(fuse.k_gain, fuse.gain_dtype, at8, prep_k.gain);
        }
    }
    if (pages_in_lds) {
#pragma unroll
        for (int i = 0; i < PAGE_TURNS; ++i) {
            const int e = static_cast<int>(threadIdx.x) + i * 64 * WV;
            if (e < page_count) pages_lds[e] = page_got[i];
        }
        __syncthreads();
    }

    // ---- keys and values: a round is U keys a lane group, two rounds are in flight ----
    auto ask = [&](int round, u32x4* kk, u32x4* vv, bool* ok) {
        const int base = s_begin + round * ROUND + wave * KPW * U;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = base + u * KPW + sub;
            const bool in = j < s_end;
            int w;
            const int bi = page_of(in ? j : s_begin, w);                // a key that exists in any case
            const int page = pages_in_lds ? pages_lds[bi - page_first] : table[bi];
            ok[u] = in && page >= 0;
            const size_t off = (static_cast<size_t>(max(page, 0)) * block_size + w) * row_stride + head_off;
            kk[u] = *reinterpret_cast<const u32x4*>(k_pool + off);
            vv[u] = *reinterpret_cast<const u32x4*>(v_pool + off);
        }
    };
    u32x4 ka[U], va[U], kb[U], vb[U];
    bool oka[U], okb[U];
    if (rounds > 0) ask(0, ka, va, oka);
    if (rounds > 1) ask(1, kb, vb, okb);

    // ---- while they are on their way: the queries, and the token's own key ----
    // The queries stay bfloat16 pairs (as the stand-alone kernel would have stored them): a score is four
    // two-element dot products a lane, and the scale multiplies the sum.
    u32x4 qp[GT];
#pragma unroll
    for (int hq = 0; hq < GT; ++hq) {
        const bool real = hq < heads && d_ok;
        if (fuse.mode != 0) {
            float x[8];
            unpack8(qraw[hq], x);
            if (!real) {
#pragma unroll
                for (int i = 0; i < 8; ++i) x[i] = 0.f;
            }
            ad_norm_rope8<LPK>(x, fuse.q_gain != nullptr, prep_q, fuse, d, dl);
#pragma unroll
            for (int w = 0; w < 4; ++w) qp[hq].v[w] = ad_pack2(x[2 * w], x[2 * w + 1]);
        } else {
#pragma unroll
            for (int w = 0; w < 4; ++w) qp[hq].v[w] = real ? qraw[hq].v[w] : 0u;
        }
    }
    float m[GT], l[GT], acc[GT][8];
#pragma unroll
    for (int hq = 0; hq < GT; ++hq) {
        m[hq] = -INFINITY;
        l[hq] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[hq][i] = 0.f;
    }
    if (own) {
        // normalised and rotated here, written into the cache by one workgroup, and the first thing that
        // the running state of one lane group holds
        float kf[8], vf[8];
        unpack8(own_k, kf);
        unpack8(own_v, vf);
        if (!d_ok) {
#pragma unroll
            for (int i = 0; i < 8; ++i) kf[i] = vf[i] = 0.f;
        }
        ad_norm_rope8<LPK>(kf, fuse.k_gain != nullptr, prep_k, fuse, d, dl);
        u32x4 own_kp;
#pragma unroll
        for (int w = 0; w < 4; ++w) own_kp.v[w] = ad_pack2(kf[2 * w], kf[2 * w + 1]);
        if (tile == 0 && sub == 0 && d_ok && own_page >= 0) {
            const size_t off = (static_cast<size_t>(own_page) * block_size + own_within) * row_stride + static_cast<size_t>(kvh) * d + dl * 8;
            *reinterpret_cast<u32x4*>(k_pool + off) = own_kp;
            *reinterpret_cast<u32x4*>(v_pool + off) = own_v;
        }
#pragma unroll
        for (int hq = 0; hq < GT; ++hq) {
            float dot = 0.f;
#pragma unroll
            for (int w = 0; w < 4; ++w) dot = ad_dot2(qp[hq].v[w], own_kp.v[w], dot);
            dot = key_sum<LPK>(dot) * scale_log2e;
            if (sub == 0 && own_page >= 0) {
                m[hq] = dot;
                l[hq] = 1.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[hq][i] = vf[i];
            }
        }
    }

    // A key that does not exist (or whose page the request no longer holds) gets a score of minus
    // infinity by selection, whatever its row holds; its value is cleared, since a probability of zero
    // times a value that is not finite would not be zero.  Lanes past the head's width hold zero queries.
    // Values are taken two keys at a time: element i of both keys in one word against both probabilities
    // (rounded to bfloat16, as the matrix-core kernels round them), one instruction an element and head.
    static_assert(U % 2 == 0, "values are taken two keys at a time");
    auto consume = [&](u32x4* kraw, u32x4* vraw, const bool* ok) {
        float s[U][GT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int hq = 0; hq < GT; ++hq) {
                float dot = 0.f;
#pragma unroll
                for (int w = 0; w < 4; ++w) dot = ad_dot2(qp[hq].v[w], kraw[u].v[w], dot);
                dot = key_sum<LPK>(dot) * scale_log2e;
                s[u][hq] = ok[u] ? dot : -INFINITY;
            }
            const uint32_t keep = ok[u] ? 0xffffffffu : 0u;
#pragma unroll
            for (int w = 0; w < 4; ++w) vraw[u].v[w] &= keep;
        }
        float p[U][GT], corr[GT];
#pragma unroll
        for (int hq = 0; hq < GT; ++hq) {
            float m_new = m[hq];
#pragma unroll
            for (int u = 0; u < U; ++u) m_new = fmaxf(m_new, s[u][hq]);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;   // nothing seen yet by this lane group: all weights zero
            corr[hq] = exp2f(m[hq] - m_use);
            float psum = 0.f;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                p[u][hq] = exp2f(s[u][hq] - m_use);
                psum += p[u][hq];
            }
            l[hq] = l[hq] * corr[hq] + psum;
            m[hq] = m_new;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[hq][i] *= corr[hq];
        }
#pragma unroll
        for (int u = 0; u < U; u += 2) {
            uint32_t pp[GT];
#pragma unroll
            for (int hq = 0; hq < GT; ++hq) pp[hq] = ad_pack2(p[u][hq], p[u + 1][hq]);
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                // (bytes 0..3 of the selector's second operand, 4..7 of its first)
                const uint32_t even = __builtin_amdgcn_perm(vraw[u + 1].v[w], vraw[u].v[w], 0x05040100u);
                const uint32_t odd = __builtin_amdgcn_perm(vraw[u + 1].v[w], vraw[u].v[w], 0x07060302u);
#pragma unroll
                for (int hq = 0; hq < GT; ++hq) {
                    acc[hq][2 * w] = ad_dot2(even, pp[hq], acc[hq][2 * w]);
                    acc[hq][2 * w + 1] = ad_dot2(odd, pp[hq], acc[hq][2 * w + 1]);
                }
            }
        }
    };
    for (int r = 0; r < rounds; r += 2) {
        consume(ka, va, oka);
        if (r + 2 < rounds) ask(r + 2, ka, va, oka);
        if (r + 1 < rounds) {
            consume(kb, vb, okb);
            if (r + 3 < rounds) ask(r + 3, kb, vb, okb);
        }
    }

    // merge the lane groups of a wave in registers, then the waves through LDS
#pragma unroll
    for (int off = LPK; off < PL_WAVE; off <<= 1) {
#pragma unroll
        for (int hq = 0; hq < GT; ++hq) {
            const float mo = __shfl_xor(m[hq], off, PL_WAVE), lo = __shfl_xor(l[hq], off, PL_WAVE);
            const float mn = fmaxf(m[hq], mo);
            const float ca = mn == -INFINITY ? 0.f : exp2f(m[hq] - mn), cb = mn == -INFINITY ? 0.f : exp2f(mo - mn);
            l[hq] = l[hq] * ca + lo * cb;
            m[hq] = mn;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[hq][i] = acc[hq][i] * ca + __shfl_xor(acc[hq][i], off, PL_WAVE) * cb;
        }
    }
    if (sub == 0) {
#pragma unroll
        for (int hq = 0; hq < GT; ++hq) {
            if (dl == 0) {
                ml[(wave * GT + hq) * 2] = m[hq];
                ml[(wave * GT + hq) * 2 + 1] = l[hq];
            }
            if (d_ok) {
#pragma unroll
                for (int i = 0; i < 8; ++i) accs[(static_cast<size_t>(wave) * GT + hq) * d + dl * 8 + i] = acc[hq][i];
            }
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < heads * d; idx += blockDim.x) {
        const int hq = idx / d, dd = idx % d;
        float mw[WV], big = -INFINITY;
#pragma unroll
        for (int w = 0; w < WV; ++w) {
            mw[w] = ml[(w * GT + hq) * 2];
            big = fmaxf(big, mw[w]);
        }
        float sum = 0.f, a = 0.f;
#pragma unroll
        for (int w = 0; w < WV; ++w) {
            const float wt = mw[w] == -INFINITY ? 0.f : exp2f(mw[w] - big);
            sum = fmaf(ml[(w * GT + hq) * 2 + 1], wt, sum);
            a = fmaf(accs[(static_cast<size_t>(w) * GT + hq) * d + dd], wt, a);
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
    } else {                 // blockIdx.y is the token
        t = blockIdx.y;
        rest = blockIdx.x * blockDim.x + threadIdx.x;
        inside = rest < per_token;
        rest = min(rest, per_token - 1);
    }
    // (a head size that is a power of two spares the kernel a division in front of its loads)
    const int h = (d & (d - 1)) == 0 ? rest >> (31 - __builtin_clz(static_cast<unsigned>(d))) : rest / d;
    const int dd = rest - h * d;
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

#define AD_WAVES 4

template <int LPK, int GT, int U>
static int launch_decode_keys(const void* q, int q_stride, void* out, float* part_acc, float* part_ml,
                              const int* positions, const int* seq_of, const int* q_len, int short_limit, int num_seqs,
                              int short_rows, const int* block_table, int max_blocks, int block_size, void* k_pool,
                              void* v_pool, int n, int nq, int nkv, int d, float scale, int window, int splits,
                              const ad_fuse_t& fuse, hipStream_t stream) {
    constexpr int WV = AD_WAVES;
    const int g = nq / nkv;
    const int tiles = pl_ceil_div(g, GT);
    const size_t lds_bytes = (AD_PAGES_LDS + static_cast<size_t>(WV) * GT * 2 + static_cast<size_t>(WV) * GT * d) * sizeof(float);
    PL_REQUIRE(lds_bytes <= 160 * 1024, "decode attention: %zu bytes of LDS for head size %d", lds_bytes, d);
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&paged_attention_decode_kernel<LPK, GT, U, WV>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
        PL_REQUIRE(e == hipSuccess, "decode attention: %zu bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
    }
    // rows of the grid: the step's rows, or, where fewer, the tokens that the short requests can bring
    const bool compact = q_len != nullptr && num_seqs > 0 && short_rows > 0 && short_rows < n;
    dim3 grid(nkv * tiles, compact ? short_rows : n, splits);
    PL_REQUIRE(n <= 65535 && splits <= 65535, "decode attention: %d tokens or %d splits are more than one launch covers", n, splits);
    paged_attention_decode_kernel<LPK, GT, U, WV><<<grid, 64 * WV, lds_bytes, stream>>>(
        static_cast<const bf16_t*>(q), q_stride, static_cast<bf16_t*>(out), part_acc, part_ml, positions, seq_of,
        q_len, short_limit, compact ? num_seqs : 0, block_table, max_blocks, block_size, static_cast<bf16_t*>(k_pool),
        static_cast<bf16_t*>(v_pool), nq, nkv, d, scale * 1.4426950408889634f, window, splits, tiles, g,
        static_cast<uint32_t>((0x100000000ull + splits - 1) / static_cast<unsigned>(splits)), fuse);
    PL_CHECK_LAUNCH("paged_attention_decode");
    if (splits > 1) {
        const dim3 mgrid = dim3(pl_ceil_div(nq * d, 256), compact ? short_rows : n);
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

// Keys a lane group asks for a round (as many again are in flight for the round after).  With at most a
// workgroup a compute unit, what one workgroup has in flight has to keep its compute unit's path to memory
// busy: eight keys a round, which the registers of a lone wave a SIMD hold.  With more workgroups, four (two
// where a workgroup serves many query heads), so that several workgroups fit a compute unit.  The choice
// goes by the step's rows, not by the rows that get workgroups, so that a step computes the same bits
// however its launch is sized.

template <int LPK, int GT>
static int launch_decode(const void* q, int q_stride, void* out, float* part_acc, float* part_ml,
                         const int* positions, const int* seq_of, const int* q_len, int short_limit, int num_seqs,
                         int short_rows, const int* block_table, int max_blocks, int block_size, void* k_pool,
                         void* v_pool, int n, int nq, int nkv, int d, float scale, int window, int splits,
                         const ad_fuse_t& fuse, hipStream_t stream) {
    const long long workgroups = static_cast<long long>(nkv) * pl_ceil_div(nq / nkv, GT) * n * splits;
#define AD_KEYS_CALL(U)                                                                                            \
    return launch_decode_keys<LPK, GT, U>(q, q_stride, out, part_acc, part_ml, positions, seq_of, q_len,          \
                                          short_limit, num_seqs, short_rows, block_table, max_blocks, block_size,  \
                                          k_pool, v_pool, n, nq, nkv, d, scale, window, splits, fuse, stream)
    if constexpr (GT <= 2) {
        if (workgroups <= pl_compute_units()) AD_KEYS_CALL(8);
        AD_KEYS_CALL(4);
    } else {
        AD_KEYS_CALL(2);
    }
#undef AD_KEYS_CALL
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

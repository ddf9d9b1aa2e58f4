// Paged attention for portions of prompts in bfloat16 on the matrix cores.
//
// A request brings q_len consecutive tokens to the step; the first stands at
// position start = ctx_len - q_len.  Token i reads the keys 0..start+i (or the
// last `window` of them) of its request through the block table; the keys of
// its own step are already in the cache.  Requests that bring fewer than
// `short_limit` tokens are left to the kernel for single tokens.
//
// One workgroup of NW waves owns 32*NW consecutive tokens of one request and
// one query head; each wave owns 32 of them.  Keys are walked in tiles of 64:
//
//   S^T = K . Q^T     v_mfma_f32_32x32x16_bf16, A = a tile of keys from LDS,
//                     B = the wave's queries, held in registers for the whole
//                     kernel.  A lane then holds, for ONE query (lane % 32), 16
//                     scores of each 32-key tile, so the softmax statistics are
//                     a reduction inside the lane and one exchange with lane^32.
//   O^T += V^T . P^T  the lane's probabilities, rounded to bfloat16, are the B
//                     operand as they stand: the contraction index of a matrix
//                     product may be permuted freely, so V^T is read from LDS in
//                     the order in which the scores lie in the registers.
//
// V lies in LDS as it lies in the cache, a row a key; the transposing read of
// gfx950 (ds_read_b64_tr_b16) hands a lane four keys of one head element.
// Maximum, sum and the output are 32-bit; exponentials are base 2 with log2(e)
// folded into the scale.
#include "common.hpp"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#ifndef AP_OCC
#define AP_OCC 2  // waves a SIMD that the registers are kept within (the second launch bound counts waves a SIMD)
#endif
#ifndef AP_SMALL_KS
#define AP_SMALL_KS 2
#endif
#ifndef AP_KS
#define AP_KS 2    // waves a block of 32 tokens in the large tile
#endif
#ifndef AP_FEED
#define AP_FEED 2  // how tiles reach LDS where pages are uniform and heads are 64 or 128 wide (see the kernel)
#endif
#define AP_BN 64   // keys a tile
#define AP_KPAD 8  // padding of a row of keys in LDS, in elements

struct __attribute__((aligned(16))) ap_u32x4 {
    uint32_t v[4];
};
struct __attribute__((aligned(8))) ap_u32x2 {
    uint32_t v[2];
};

union ap_frag {
    bf16x8 vec;
    ap_u32x4 raw;
    ap_u32x2 half[2];
    uint32_t w[4];
};

typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 ap_bf16x4;
typedef __attribute__((address_space(3))) ap_bf16x4 ap_lds_bf16x4;

// The transposing read.  Among 16 neighbouring lanes, lane 4e + q gives the address of four
// elements; lane i receives, as its element e, element i % 4 of what lane 4e + i / 4 pointed at.
// With lane 4e + q pointing at row e, columns 4q .. 4q+3 of a row-major block, lane i gets
// column i of the rows 0 .. 3.
__device__ __forceinline__ ap_u32x2 ap_read_transposed(const uint16_t* at) {
    const ap_bf16x4 got = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((ap_lds_bf16x4*)(at));
    return __builtin_bit_cast(ap_u32x2, got);
}

// 16 bytes a lane from global memory straight into LDS: lane l's land at `lds_at` + 16 l (`lds_at`, the
// same for the whole wave, travels in M0).  Written as assembly so that the compiler does not count
// the load: it would make every later read of LDS wait for all such loads, the ones just issued for a
// tile two rounds ahead included.  The waits are placed by hand (s_waitcnt vmcnt) where a tile is due.
__device__ __forceinline__ void ap_load_to_lds(const void* from, const uint16_t* lds_at) {
    const uint32_t at = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)lds_at));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(at), "v"(from) : "memory", "m0");
}

typedef uint32_t ap_vec4 __attribute__((ext_vector_type(4)));   // 16 bytes on their way through registers
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Two floats rounded to nearest-even bfloat16 in one word (the hardware's packed conversion).
__device__ __forceinline__ uint32_t ap_pack2(float lo, float hi) {
    const f32x2 pair = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
}

// DT: the head is padded to 32*DT elements.  NW: blocks of 32 tokens a workgroup.  KS: waves a block
// of tokens (1, or 2: then one wave takes the first 32 keys of every tile and the other the last 32,
// each with a running state of its own, merged at the end; twice the waves overlap more of the
// softmax with the products; heads of more than 128 elements have no registers for it).  A workgroup
// has NW * KS waves.
// Padding of a row of values in LDS, in elements: a row is then 16 banks (of 32) further than the one
// before, and the four rows of 64 bytes that 32 lanes read transposed fall on every bank twice.
__host__ __device__ constexpr int ap_vpad(int dt) { return dt % 2 == 0 ? 32 : 0; }
__host__ __device__ constexpr int ap_value_buffers(int ks) { return ks == 2 ? 3 : 2; }
__host__ __device__ constexpr int ap_direct_ahead(bool grouped) { return grouped ? 1 : 2; }

// The direct feed's permutation of the 16-byte pieces of an unpadded row in LDS (64 banks of 4 bytes: a row
// of 128 elements covers them all once, of 64 elements half).  Piece c of the key with row number r (mod 16)
// stands at c ^ shift.  Keys are read 16 rows at a time, one piece each: 16 different places.  Values are read
// (transposed) four rows at a time, four neighbouring pieces each: four different groups of four.
__device__ __forceinline__ int ap_key_shift(int r, int pieces) { return (pieces == 16 ? r : r >> 1) & (pieces - 1); }
__device__ __forceinline__ int ap_value_shift(int r, int pieces) { return 4 * ((pieces == 16 ? r : r >> 1) & (pieces / 4 - 1)); }

// UP (uniform pages): the 64 / (4*DT) keys whose pieces one wave loads with one instruction lie in one
// page (the page size is a power of two and at least as many keys).  Page numbers then come through
// the scalar unit and an address is a scalar base plus a lane's constant: no vector arithmetic a tile.
// What is loaded is not masked on this path.  Scores of keys that do not exist are replaced, not
// multiplied, so whatever their rows of the key pool hold is never seen.  Their values are multiplied by
// a probability of exactly zero, which only gives zero for a finite value: a page keeps what its last
// owner left there, and that may be anything.  So a lane whose value row lies past the last key that the
// tile's queries see, or before the first (a window's pages may have been given back), reads the last
// key's row instead, a row that this request wrote; only the first and the last tile of keys of a
// workgroup have such rows, and only there the addresses are chosen lane by lane.
//
// FEED 0: any page size, tiles travel through registers and are masked.  1: uniform pages, through
// registers.  2: uniform pages, and the loads write LDS themselves (global_load_lds_dwordx4: lane l of
// a wave puts its 16 bytes at the wave's LDS base + 16 l), three tiles ahead of their use and with no
// register or LDS write instruction spent on them.  Rows then lie unpadded in LDS, so their 16-byte
// pieces are permuted instead (ap_key_shift, ap_value_shift: the reads of the matrix cores' operands
// fall on every bank once); heads of 64 and 128.
//
// GR (grouped): the 32*NW rows of a workgroup are not consecutive tokens of one query head but the query
// heads of ONE token that share a key head (rows past the group's size stand idle): a single token, or
// each token of a short portion, then reads its keys once for the whole group, on the matrix cores.
// The token tile of the work index is then a token, its head a key head, and requests with
// short_limit or more tokens are the ones left out.
// Token tiles counted over the requests that a launch serves (those with `short_limit` tokens or more, and a
// context; grouped: those with fewer, a tile being one token), one request after the other: which request and
// which of its tiles is number `slot`?  Late tiles, which read the most keys, come first within a request.  A step of one long portion beside many single
// tokens then has workgroups for the portion's tiles only, and not tiles-of-the-longest times requests of
// them, nearly all of which would find nothing to do.  Every thread of the workgroup calls this, with all
// lanes of its wave; false: there is no such tile.
__device__ __forceinline__ bool ap_find_tile(int slot, const int* __restrict__ q_len, const int* __restrict__ ctx_len,
                                             int num_seqs, int short_limit, int bm, bool grouped, int& seq, int& tile) {
    const int lane = threadIdx.x & 63;
    int before = 0;                                             // tiles of the requests before this stretch of 64
    for (int base = 0; base < num_seqs; base += 64) {
        const int s = base + lane;
        int mine = 0;
        if (s < num_seqs) {
            const int c = q_len[s];
            const bool served = grouped ? (short_limit <= 0 || c < short_limit) : c >= short_limit;
            if (c > 0 && served && ctx_len[s] > 0) mine = (c + bm - 1) / bm;
        }
        int through = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int other = __shfl_up(through, off, 64);
            if (lane >= off) through += other;
        }
        const int total = __builtin_amdgcn_readfirstlane(__shfl(through, 63, 64));   // uniform, and known to be
        if (slot < before + total) {
            const bool here = mine > 0 && slot >= before + through - mine && slot < before + through;
            const int l = __ffsll(static_cast<unsigned long long>(__ballot(here))) - 1;   // one lane says so
            // (the same in every lane: said so to the compiler, which keeps what follows from them in scalar registers)
            seq = __builtin_amdgcn_readfirstlane(base + l);
            tile = __builtin_amdgcn_readfirstlane(__shfl(mine, l, 64) - 1 - (slot - before - __shfl(through - mine, l, 64)));
            return true;
        }
        before += total;
    }
    return false;
}

template <int DT, int NW, int KS, int FEED, bool GR = false>
__global__ void __launch_bounds__(64 * NW * KS, DT <= 4 ? AP_OCC : 1)
paged_attention_prefill_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out,
                               const int* __restrict__ q_start, const int* __restrict__ q_len,
                               const int* __restrict__ ctx_len, int short_limit, int tiles_a_request,
                               int num_seqs, const int* __restrict__ block_table, int max_blocks,
                               int block_size, const bf16_t* __restrict__ k_pool,
                               const bf16_t* __restrict__ v_pool, int nq, int nkv, int d, float scale_log2e,
                               int window, int total_work, int splits, float* __restrict__ part_acc,
                               float* __restrict__ part_ml, int compact) {
    constexpr int DP = 32 * DT;
    constexpr int BM = 32 * NW;
    constexpr int NT = 64 * NW * KS;
    constexpr int KT = 2 / KS;             // 32-key tiles of a 64-key tile a wave takes
    constexpr bool UP = FEED >= 1, DIRECT = FEED == 2;
    static_assert(!DIRECT || ((DT == 2 || DT == 4) && KS == 2), "the direct feed is written for heads of 64 and 128");
    constexpr int KROW = DIRECT ? DP : DP + AP_KPAD;       // elements a row of Ks
    constexpr int VROW = DIRECT ? DP : DP + ap_vpad(DT);   // elements a row of Vs
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    // Two tiles of keys [AP_BN][KROW], then NVB tiles of values [AP_BN][VROW].  The values of a tile
    // are read one round after its keys, and with two groups of waves half a round apart they live
    // for three rounds.
    // (The direct feed asks for a tile AHEAD rounds before its keys are read: AHEAD - 1 buffers more of each.
    // Grouped, a workgroup is two waves with a round of some 2 us, far more than a trip to memory; what it
    // lacks is company on its compute unit, and with one round ahead instead of two its tiles take 80 KB
    // instead of 112, so that two workgroups share a compute unit.)
    constexpr int AHEAD = ap_direct_ahead(GR);
    constexpr int NKB = DIRECT ? AHEAD + 1 : 2;
    constexpr int NVB = DIRECT ? AHEAD + 2 : ap_value_buffers(KS);
    constexpr int KTILE = AP_BN * KROW, VTILE = AP_BN * VROW;
    uint16_t* const Kbase = lds;
    uint16_t* const Vbase = lds + NKB * KTILE;

    // Workgroups are dealt round-robin to the eight XCDs; consecutive pieces of
    // work (the token tiles of one head) go to one XCD, whose L2 then holds the
    // keys and values they share.
    int work = blockIdx.x;
    // (compact: only the first slots have tiles, and a stretch of them must not fall to one XCD; workgroups
    // that follow each other go to XCDs that follow each other, so with heads times splits a multiple of eight
    // a head's tiles still meet in one XCD.)
    if (!compact && (total_work & 7) == 0) work = (blockIdx.x & 7) * (total_work >> 3) + (blockIdx.x >> 3);
    // work = ((request * nq + head) * tiles + (tiles - 1 - tile)) * splits + split: late tiles, which read
    // the most keys, first.  With splits > 1 the key tiles of a token tile are dealt to that many
    // workgroups (few token tiles over a long context would leave compute units idle, and the last
    // token tiles of a prompt hold the others up); each leaves its unnormalised output, maximum and sum
    // in the workspace and a second kernel puts them together.
    // (compact: work = (slot * heads + head) * splits + split, the slot being a token tile as ap_find_tile counts them)
    const int split = work % splits;
    work /= splits;
    const int heads_n = GR ? nkv : nq;
    int tile = tiles_a_request - 1 - work % tiles_a_request;
    int head = (work / tiles_a_request) % heads_n;
    int seq = work / (tiles_a_request * heads_n);
    if (compact) {
        head = work % heads_n;
        if (!ap_find_tile(work / heads_n, q_len, ctx_len, num_seqs, short_limit, GR ? 1 : 32 * NW, GR, seq, tile)) return;
    }
    if (seq >= num_seqs) return;

    const int count = q_len[seq];
    if (ctx_len[seq] <= 0) return;                           // a request of padding rows has no context
    if (GR ? (short_limit > 0 && count >= short_limit) : count < short_limit) return;
    const int q0 = GR ? tile : tile * BM;                    // the tile's first token
    if (q0 >= count) return;
    const int start = ctx_len[seq] - count;  // position of the request's first token in this step
    const int row0 = q_start[seq];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave_id = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same for the whole wave: kept scalar
    // waves w and w + 4 share a SIMD: with NW == 4 a SIMD holds one wave of either group of keys
    const int wave = wave_id % NW;                               // which block of 32 tokens
    const int kt0 = (wave_id / NW) * KT;                         // the wave's first 32-key tile of a 64-key tile
    const int r32 = lane & 31;
    const int h = lane >> 5;
    const int group = nq / nkv;
    const int kvh = GR ? head : head / group;

    // the wave's queries: lane holds query wq = q0 + wave*32 + r32, elements 16*kk + 8*h .. +8
    // (grouped: the lane's query is head kvh * group + wave*32 + r32 of token q0)
    const int wq = GR ? q0 : q0 + wave * 32 + r32;
    const int q_head = GR ? kvh * group + min(wave * 32 + r32, group - 1) : head;
    const bool q_ok = GR ? wave * 32 + r32 < group : wq < count;
    ap_frag qf[2 * DT];
#pragma unroll
    for (int kk = 0; kk < 2 * DT; ++kk) {
        const int e0 = 16 * kk + 8 * h;
        if (q_ok && e0 < d)
            qf[kk].raw = *reinterpret_cast<const ap_u32x4*>(q + static_cast<size_t>(row0 + wq) * q_stride +
                                                            static_cast<size_t>(q_head) * d + e0);
        else
            qf[kk].raw = ap_u32x4{{0u, 0u, 0u, 0u}};
    }
    const int q_pos = start + wq;                               // position of this lane's query
    const int wave_first = GR ? q_pos : start + q0 + wave * 32; // position of the wave's first query
    const int wave_last = GR ? q_pos : start + min(q0 + wave * 32 + 31, count - 1);
    const bool wave_active = GR ? wave * 32 < group : q0 + wave * 32 < count;

    f32x16 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;

    const int last_pos = GR ? start + q0 : start + min(q0 + BM, count) - 1;   // the last key any query of the tile sees
    const int first_pos = (window > 0 && start + q0 + 1 > window) ? start + q0 + 1 - window : 0;
    const int* table = block_table + static_cast<size_t>(seq) * max_blocks;
    const size_t row_stride = static_cast<size_t>(nkv) * d;
    const size_t head_off = static_cast<size_t>(kvh) * d;
    const int cpr = d / 8;                                      // 16-byte pieces of a row of the head
    // floor(2^32 / block_size): the high half of j * bs_magic is j / block_size or one less
    const uint32_t bs_magic = block_size == 1 ? 0xffffffffu : static_cast<uint32_t>(0x100000000ull / static_cast<uint32_t>(block_size));

    // A tile travels global memory -> registers -> LDS.  The loads of the next tile are issued before
    // the products of this one, so that their latency passes behind the matrix cores.
    constexpr int CP = DP / 8;                                  // 16-byte pieces of a padded row
    constexpr int KI = (AP_BN * CP + NT - 1) / NT;              // pieces of the key tile a thread carries
    ap_vec4 kreg[KI], vreg[KI];                                 // and the same pieces of the value tile

    // Loads are unconditional, from an address that is valid in any case, and what they bring is
    // masked afterwards where the key does not exist: a load inside a branch would be waited for
    // at the branch's end, one load after the other.  The page numbers of a tile are looked up one
    // tile before its keys and values are loaded, so that no load waits for another.
    // A lookup leaves the table's answer raw: what depends on it is computed by the fetch, one tile
    // later, so that the wait for the answer stands there and not in the middle of this tile.
    int kblk[KI], kwithin[KI];       // UP: the page of the wave's keys of piece i and their first row in it
    int kj0[KI];                     // UP: the key that this row is
    bool kin[KI];
    uint32_t keep[KI];
    const int log2_bs = 31 - __builtin_clz(static_cast<unsigned>(block_size));
    const uint32_t row_bytes = static_cast<uint32_t>(nkv) * d * 2;
    // UP: this lane's place beside the wave's base: its row among the wave's rows, its piece of the row
    const uint32_t lane_piece = static_cast<uint32_t>(head_off + min(lane % CP, cpr - 1) * 8) * 2;
    const uint32_t lane_place = (lane / CP) * row_bytes + lane_piece;
    // UP: the row of the last key that the tile's queries see, where the values of later rows are read from
    size_t last_base = 0;
    if constexpr (UP) {
        const int last_page = __builtin_amdgcn_readfirstlane(max(table[last_pos >> log2_bs], 0));
        last_base = (static_cast<size_t>(last_page) * block_size + (last_pos & (block_size - 1))) * row_bytes;
    }
    auto locate = [&](int j, int& blk, int& within, bool& in) {  // page and place in the page of key j
        in = j <= last_pos;
        const int jj = in ? j : last_pos;
        int bi = static_cast<int>(__umulhi(static_cast<uint32_t>(jj), bs_magic));
        within = jj - bi * block_size;
        const int low = within >= block_size ? 1 : 0;            // the estimate is the quotient or one less
        bi += low;
        within -= low * block_size;
        blk = table[bi];
    };
    // UP: the page of key j (of the last key, past it), through the scalar unit: the entry's place as a 32-bit
    // count of bytes behind the table's row, which one scalar load takes as it stands
    auto page_of = [&](int j) {
        const uint32_t at = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(min(j, last_pos) >> log2_bs)) << 2;
        return *reinterpret_cast<const int*>(reinterpret_cast<const char*>(table) + at);
    };
    auto lookup = [&](int k0) {
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            if constexpr (UP) {
                // the first key of the wave's rows; past the last key the page of the last key serves
                // (its rows exist, and what they hold is never seen)
                const int j0 = k0 + (64 * wave_id + i * NT) / CP;
                kj0[i] = j0;
                kwithin[i] = j0 & (block_size - 1);
                kblk[i] = page_of(j0);
            } else {
                locate(k0 + ((tid + i * NT) / CP) % AP_BN, kblk[i], kwithin[i], kin[i]);
            }
        }
    };
    // UP: the scalar unit answers slowly, so the pages of the tile after the next are asked for at the
    // start of the half round whose end needs them
    int ahead_blk[KI], ahead_within[KI], ahead_j0[KI];
    auto look_ahead = [&](int k0) {
        if constexpr (UP) {
#pragma unroll
            for (int i = 0; i < KI; ++i) {
                const int j0 = k0 + (64 * wave_id + i * NT) / CP;
                ahead_j0[i] = j0;
                ahead_within[i] = j0 & (block_size - 1);
                ahead_blk[i] = page_of(j0);
            }
        }
    };
    auto row_of = [&](int blk, int within) -> size_t {
        return (static_cast<size_t>(max(blk, 0)) * block_size + within) * row_stride;
    };
    // What a load brings is masked only when it goes into LDS, one tile later: a mask applied here
    // would make the wave wait for the load in the middle of the tile that should hide it.
    auto fetch = [&]() {
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            if constexpr (UP) {
                const int page = __builtin_amdgcn_readfirstlane(max(kblk[i], 0));
                const size_t base = (static_cast<size_t>(page) * block_size + kwithin[i]) * row_bytes;
                kreg[i] = *reinterpret_cast<const ap_vec4*>(reinterpret_cast<const char*>(k_pool) + base + lane_place);
                size_t vat = base + lane_place;
                if (kj0[i] + 64 / CP - 1 > last_pos || kj0[i] < first_pos) {   // (the same for the wave)
                    const int j = kj0[i] + lane / CP;
                    vat = (j > last_pos || j < first_pos) ? last_base + lane_piece : vat;
                }
                vreg[i] = *reinterpret_cast<const ap_vec4*>(reinterpret_cast<const char*>(v_pool) + vat);
            } else {
                const int c = (tid + i * NT) % CP;
                const size_t at = row_of(kblk[i], kwithin[i]) + head_off + min(c, cpr - 1) * 8;
                kreg[i] = *reinterpret_cast<const ap_vec4*>(k_pool + at);
                vreg[i] = *reinterpret_cast<const ap_vec4*>(v_pool + at);
                keep[i] = (kin[i] && kblk[i] >= 0 && c < cpr) ? 0xffffffffu : 0u;
            }
        }
    };
    auto stash = [&](int kbuf, int vbuf) {
        uint16_t* Ks = Kbase + kbuf * KTILE;
        uint16_t* Vs = Vbase + vbuf * VTILE;
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            const int idx = tid + i * NT;
            const int key = idx / CP, c = idx % CP;
            ap_vec4 kk = kreg[i], vv = vreg[i];
            if constexpr (!UP) {
                kk &= keep[i];
                vv &= keep[i];
            }
            if (idx < AP_BN * CP) {
                *reinterpret_cast<ap_vec4*>(Ks + key * KROW + c * 8) = kk;
                *reinterpret_cast<ap_vec4*>(Vs + key * VROW + c * 8) = vv;
            }
        }
    };

    // this workgroup's share of the key tiles
    const int k_lowest = (first_pos / AP_BN) * AP_BN;
    const int key_tiles = (last_pos - k_lowest) / AP_BN + 1;
    const int tiles_a_split = (key_tiles + splits - 1) / splits;
    const int k_first = k_lowest + split * tiles_a_split * AP_BN;
    const int k_end = min(k_lowest + key_tiles * AP_BN, k_first + tiles_a_split * AP_BN);
    if (k_first >= k_end) {          // more splits than key tiles: nothing to add
        if (kt0 == 0 && q_ok) {
            float* ml = part_ml + ((static_cast<size_t>(row0 + wq) * nq + q_head) * splits + split) * 2;
            if (h == 0) {
                ml[0] = -INFINITY;
                ml[1] = 0.f;
            }
        }
        return;
    }
    int staged = 1, staged_v = 1;    // the tile that the registers hold, and the buffer its values go to
    // The direct feed: the loads of tile j, this wave's share (KI instructions for the keys, KI for the
    // values), into the buffers j % NKB and j % NVB.  The lane's place in the cache row differs between
    // keys and values by the permutation of the pieces.
    int asked = 0, asked_k = 0, asked_v = 0;   // the next tile to ask for and its buffers
    // (A wave's loads of one tile are NT / CP rows apart: where that is no multiple of 16, the row number
    // mod 16, and with it the permutation, alternates between two values from one load to the next.)
    constexpr bool ROWS_ALTERNATE = DIRECT && (NT / CP) % 16 != 0;
    static_assert(!DIRECT || (2 * NT / CP) % 16 == 0, "the rows of a wave's loads repeat mod 16 after two loads at most");
    uint32_t place_k[2] = {0, 0}, place_v[2] = {0, 0}, piece_v[2] = {0, 0};
    if constexpr (DIRECT) {
#pragma unroll
        for (int odd = 0; odd < 2; ++odd) {
            const int r15 = ((64 * wave_id + odd * NT) / CP + lane / CP) & 15;
            const int ck = (lane % CP) ^ ap_key_shift(r15, CP), cv = (lane % CP) ^ ap_value_shift(r15, CP);
            place_k[odd] = (lane / CP) * row_bytes + static_cast<uint32_t>(head_off + min(ck, cpr - 1) * 8) * 2;
            piece_v[odd] = static_cast<uint32_t>(head_off + min(cv, cpr - 1) * 8) * 2;
            place_v[odd] = (lane / CP) * row_bytes + piece_v[odd];
        }
    }
    // (The scalar unit, which the waves of a compute unit share, does the addresses: a page's first byte as one
    // product of two 32-bit numbers, and one comparison a tile for whether any of its rows needs the redirection
    // below; with both done a load at a time the addresses took a sixth of the kernel's time.)
    const uint32_t page_bytes = static_cast<uint32_t>(block_size) * row_bytes;
    auto ask = [&]() {               // pages from kblk/kwithin, looked up before
        if constexpr (DIRECT) {
            const int tile_first = k_first + asked * AP_BN;
            const bool at_an_edge = tile_first + AP_BN - 1 > last_pos || tile_first < first_pos;
#pragma unroll
            for (int i = 0; i < KI; ++i) {
                const int first_row = (64 * wave_id + i * NT) / CP;
                const uint32_t page = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(max(kblk[i], 0)));
                const size_t base = static_cast<size_t>(page) * page_bytes + static_cast<uint32_t>(kwithin[i]) * row_bytes;
                const char* gk = reinterpret_cast<const char*>(k_pool) + base + place_k[ROWS_ALTERNATE ? i & 1 : 0];
                const char* gv = reinterpret_cast<const char*>(v_pool) + base + place_v[ROWS_ALTERNATE ? i & 1 : 0];
                if (at_an_edge && (kj0[i] + 64 / CP - 1 > last_pos || kj0[i] < first_pos)) {   // (the same for the wave)
                    const int j = kj0[i] + lane / CP;
                    if (j > last_pos || j < first_pos)
                        gv = reinterpret_cast<const char*>(v_pool) + last_base + piece_v[ROWS_ALTERNATE ? i & 1 : 0];
                }
                uint16_t* lk = Kbase + asked_k * KTILE + first_row * KROW;
                uint16_t* lv = Vbase + asked_v * VTILE + first_row * VROW;
                ap_load_to_lds(gk, lk);
                ap_load_to_lds(gv, lv);
            }
            ++asked;
            asked_k = asked_k + 1 == NKB ? 0 : asked_k + 1;
            asked_v = asked_v + 1 == NVB ? 0 : asked_v + 1;
        }
    };
    auto take_pages = [&]() {
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            kblk[i] = ahead_blk[i];
            kwithin[i] = ahead_within[i];
            kj0[i] = ahead_j0[i];
        }
    };
    if constexpr (DIRECT) {
        lookup(k_first);
        ask();
        if constexpr (AHEAD == 2) {
            lookup(k_first + AP_BN);
            ask();
        }
        lookup(k_first + AHEAD * AP_BN);         // for the first round's asking
        __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): the first tiles have landed
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    } else {
        lookup(k_first);
        fetch();
        lookup(k_first + AP_BN);
        stash(0, 0);
        fetch();                         // the second tile, all zeros past the last key
        lookup(k_first + 2 * AP_BN);
        __syncthreads();
    }
    // The registers hold tile `staged`: it goes into buffers that nobody reads now, the tile after it
    // is asked for and the one after that looked up.
    auto advance = [&]() {
        if constexpr (!DIRECT) {
            stash(staged & 1, staged_v);
            fetch();
            if constexpr (UP) {
                take_pages();
            } else {
                lookup(k_first + (staged + 2) * AP_BN);
            }
            ++staged;
            staged_v = staged_v + 1 == NVB ? 0 : staged_v + 1;
        }
    };

    // A round has two halves with a barrier after each.  In the first a wave multiplies: the scores of
    // tile t, and the values of tile t-1 into the output.  In the second it turns the scores of tile t
    // into probabilities and moves the next tile into LDS.  With KS == 2 the waves of the later keys
    // run half a round behind the others, so that on every SIMD one wave multiplies while the other
    // exponentiates.
    //
    // The running maximum is kept on the raw scores; the scale (with log2 e folded in) enters inside
    // the exponential's argument, one multiply-add an element.  The output is rescaled only when some
    // query's maximum has grown.
    f32x16 s[KT];
    ap_frag pb[KT][2];               // probabilities of the tile before, rounded: [kt][half] is 16 keys
    const int v_corner = (32 * kt0 + 4 * h + ((lane & 15) >> 2)) * VROW + (lane & 16) + 4 * (lane & 3);
    // The direct feed's permuted pieces: where piece 2*kk + h of this lane's key stands, and where the
    // block of head elements 32*dt .. of this lane's four keys begins.
    int k_piece[2 * DT], v_piece[DT];
    if constexpr (DIRECT) {
        const int fk = ap_key_shift(r32 & 15, CP);
#pragma unroll
        for (int kk = 0; kk < 2 * DT; ++kk) k_piece[kk] = ((2 * kk + h) ^ fk) * 8;
        const int i16 = lane & 15, g = lane >> 4;
        const int fv = ap_value_shift(i16 >> 2, CP);     // of the lane's key 4h + i16/4 (+ 8, + 16: the same)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v_piece[dt] = ((4 * dt + 2 * (g & 1) + ((i16 & 3) >> 1)) ^ fv) * 8 + 4 * (i16 & 1);
    }
    // The multiplying half of a round: O^T += V^T . P^T for the tile before (sixteen keys a product:
    // pb[kt][half] holds the keys 32*(kt0+kt) + 16*half + {4h..4h+3} and + 8 + {4h..4h+3}; 16 lanes read a
    // block of 4 keys x 16 head elements transposed), and the scores of this tile, transposed:
    // s[kt][4*j + i] is key k0 + 32*(kt0+kt) + 8*j + 4*h + i against query r32.  For heads up to 128 all
    // operands are asked for before the first product, values first, so that LDS is waited for once.
    auto multiply = [&](int kbuf, int vbuf, bool with_scores) {
        const uint16_t* Ks = Kbase + kbuf * KTILE;
        const uint16_t* Vs = Vbase + vbuf * VTILE + v_corner;
        if constexpr (DT <= 4 && KT == 1) {
            ap_frag va[2][DT], ka[2 * DT];
            const uint16_t* Vrows = Vbase + vbuf * VTILE + (32 * kt0 + 4 * h + ((lane & 15) >> 2)) * VROW;
            auto ask_values = [&](int half, int dt) {
                const uint16_t* block = DIRECT ? Vrows + 16 * half * VROW + v_piece[dt] : Vs + 16 * half * VROW + 32 * dt;
                va[half][dt].half[0] = ap_read_transposed(block);
                va[half][dt].half[1] = ap_read_transposed(block + 8 * VROW);
            };
            // The scores first (they are done when the softmax asks for them, while the last products
            // of the values still run), and the values asked for between their products: the reads
            // of LDS go on while the matrix cores work.
            if (with_scores) {
#pragma unroll
                for (int kk = 0; kk < 2 * DT; ++kk)
                    ka[kk].raw = *reinterpret_cast<const ap_u32x4*>(Ks + (32 * kt0 + r32) * KROW +
                                                                    (DIRECT ? k_piece[kk] : 16 * kk + 8 * h));
#pragma unroll
                for (int r = 0; r < 16; ++r) s[0][r] = 0.f;
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kk = 0; kk < 2 * DT; ++kk) {
                    s[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[kk].vec, qf[kk].vec, s[0], 0, 0, 0);
                    ask_values(kk / DT, kk % DT);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int kk = 0; kk < 2 * DT; ++kk) ask_values(kk / DT, kk % DT);
            }
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[half][dt].vec, pb[0][half].vec, o[dt], 0, 0, 0);
        } else {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    ap_frag a[DT];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        const uint16_t* block = Vs + (32 * kt + 16 * half) * VROW + 32 * dt;
                        a[dt].half[0] = ap_read_transposed(block);
                        a[dt].half[1] = ap_read_transposed(block + 8 * VROW);
                    }
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
                        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[dt].vec, pb[kt][half].vec, o[dt], 0, 0, 0);
                }
            if (with_scores) {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) s[kt][r] = 0.f;
                    ap_frag a[2 * DT];
#pragma unroll
                    for (int kk = 0; kk < 2 * DT; ++kk)
                        a[kk].raw = *reinterpret_cast<const ap_u32x4*>(Ks + (32 * (kt0 + kt) + r32) * KROW + 16 * kk + 8 * h);
#pragma unroll
                    for (int kk = 0; kk < 2 * DT; ++kk)
                        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kk].vec, qf[kk].vec, s[kt], 0, 0, 0);
                }
            }
        }
    };
    auto soften = [&](int k0, bool masked) {
        float mx = -INFINITY;
        if (masked) {
            // Key k0 + c + 4*h, c a constant of the register, is seen by this lane's query iff c <= reach
            // (and c > reach - window).
            const int reach = q_pos - k0 - 32 * kt0 - 4 * h;
            const int behind = window > 0 ? reach - window : -(1 << 30);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int c = 32 * kt + 8 * (r >> 2) + (r & 3);
                    s[kt][r] = (c <= reach && c > behind) ? s[kt][r] : -INFINITY;
                }
        }
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kt][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, PL_WAVE));
        const float m_new = fmaxf(m, mx);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {   // the same for the whole wave
            const float corr = __builtin_amdgcn_exp2f((m - m_use) * scale_log2e);
            lsum *= corr;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[dt][r] *= corr;
            m = m_new;
        }
        const float shift = -m_use * scale_log2e;
        float psum = 0.f;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                // v_exp_f32: arguments are <= 0, tiny results may flush
                const float p = __builtin_amdgcn_exp2f(fmaf(s[kt][r], scale_log2e, shift));
                s[kt][r] = p;
                psum += p;
            }
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int w = 0; w < 4; ++w)
                    pb[kt][half].w[w] = ap_pack2(s[kt][8 * half + 2 * w], s[kt][8 * half + 2 * w + 1]);
        }
        lsum += psum;
    };

    // The end of half a round: the products stay on their side of the barrier (the compiler would let
    // them drift behind it, into the half that should run beside another wave's products).
    // (The direct feed has no writes of its own to LDS to make visible, and the fence of __syncthreads
    // would wait for every load on its way: there the bare barrier stands, between compiler fences.)
    auto half_done = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (DIRECT) {
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else {
            __syncthreads();
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    const bool behind_group = KS == 2 && kt0 != 0;
    // One round ahead, both groups ask for a tile in the same half (the earlier group's multiplying half, the
    // later group's half before) and wait for it a round later, each before the barrier that ends the half
    // before the earlier group reads it.
    const bool ask_late = DIRECT && AHEAD == 1 && behind_group;
    auto feed_before = [&]() {
        if constexpr (DIRECT) {
            ask();
            look_ahead(k_first + asked * AP_BN);
        }
    };
    if (behind_group) {              // half a round in which the later group only moves a tile
        look_ahead(k_first + (staged + 2) * AP_BN);
        advance();
        if (ask_late) feed_before();
        half_done();
    }
    // The direct feed in the multiplying half of round t: ask for tile t + AHEAD (pages looked up a round
    // before), look up the pages of the tile after it, and wait until this wave's loads of tile t + 1 have
    // landed, after the barrier every wave's have: two rounds ahead at the end of the multiplying half (all
    // but the newest tile), one round ahead at the end of the round (everything), a whole round of flight.
    constexpr int LOADS_A_TILE = 2 * KI;
    auto feed_after = [&]() {
        if constexpr (DIRECT) {
            take_pages();
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (AHEAD == 2) {
                // vmcnt(LOADS_A_TILE): all but the newest tile (the count's bits 4 and 5 stand at bits 14 and 15)
                __builtin_amdgcn_s_waitcnt(0x0F70 | (LOADS_A_TILE & 15) | ((LOADS_A_TILE >> 4) << 14));
            } else if (ask_late) {
                __builtin_amdgcn_s_waitcnt(0x0F70);
            }
        }
    };
    auto feed_landed = [&]() {       // before the barrier that ends a round
        if constexpr (DIRECT && AHEAD == 1) {
            if (!ask_late) {
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_waitcnt(0x0F70);
            }
        }
    };
    // First the tiles that every query of the workgroup sees whole: no masks, no wave stands idle
    // (a wave past the request's last token works on zero queries and stores nothing).  Then the
    // few tiles around the diagonal, where keys are hidden and waves of early tokens are done.
    // A tile that left no probabilities (the one before the first, one a wave sat out) left zeros:
    // the values are multiplied in every round.
    int k0 = k_first, kbuf = 0, vbuf_before = 0;   // vbuf_before: where the values of the tile before lie
    auto no_weights = [&]() {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int w = 0; w < 4; ++w) pb[kt][half].w[w] = 0u;
    };
    no_weights();
    const int open_end = window > 0 ? k_first : ((start + q0 + 1) / AP_BN) * AP_BN;   // keys below it are seen by all
    auto next_tile = [&]() {
        if (k0 != k_first) vbuf_before = vbuf_before + 1 == NVB ? 0 : vbuf_before + 1;
        k0 += AP_BN;
        kbuf = kbuf + 1 == NKB ? 0 : kbuf + 1;
    };
    const int open_stop = min(open_end, k_end);
    for (; k0 < open_stop; next_tile()) {
        if (!ask_late) feed_before();
        multiply(kbuf, vbuf_before, true);
        feed_after();
        half_done();
        if constexpr (!DIRECT) look_ahead(k_first + (staged + 2) * AP_BN);
        if (ask_late) feed_before();
        soften(k0, false);
        advance();
        feed_landed();
        half_done();
    }
    for (; k0 < k_end; next_tile()) {
        // a wave whose queries all stand before this tile, or that has no queries, has nothing to add
        const bool idle = !wave_active || k0 + 32 * kt0 > wave_last ||
                          (window > 0 && k0 + 32 * (kt0 + KT) - 1 <= wave_first - window);
        if (!ask_late) feed_before();
        multiply(kbuf, vbuf_before, !idle);
        feed_after();
        half_done();
        if constexpr (!DIRECT) look_ahead(k_first + (staged + 2) * AP_BN);
        if (ask_late) feed_before();
        if (!idle) soften(k0, true);
        else no_weights();
        advance();
        feed_landed();
        half_done();
    }
    multiply(kbuf, vbuf_before, false);
    if (KS == 2 && !behind_group) half_done();   // the later group is half a round behind
    if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0x0F70);   // nothing may still be on its way into LDS
    lsum += __shfl_xor(lsum, 32, PL_WAVE);
    if (KS == 2) {
        // The wave of the later keys hands its state to the wave of the earlier ones through LDS
        // (the tiles are done with): out = (o0 2^(m0-M) + o1 2^(m1-M)) / (l0 2^(m0-M) + l1 2^(m1-M)).
        float* hand = reinterpret_cast<float*>(lds) + static_cast<size_t>(wave) * (16 * DT + 2) * PL_WAVE;
        __syncthreads();             // the tiles are done with in every wave
        if (kt0 != 0) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) hand[(dt * 16 + r) * PL_WAVE + lane] = o[dt][r];
            hand[(16 * DT) * PL_WAVE + lane] = m;
            hand[(16 * DT + 1) * PL_WAVE + lane] = lsum;
        }
        __syncthreads();
        if (kt0 != 0) return;
        const float m1 = hand[(16 * DT) * PL_WAVE + lane], l1 = hand[(16 * DT + 1) * PL_WAVE + lane];
        const float big = fmaxf(m, m1);
        const float use = big == -INFINITY ? 0.f : big;
        const float w0 = __builtin_amdgcn_exp2f((m - use) * scale_log2e), w1 = __builtin_amdgcn_exp2f((m1 - use) * scale_log2e);
        lsum = lsum * w0 + l1 * w1;
        m = big;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[dt][r] = o[dt][r] * w0 + hand[(dt * 16 + r) * PL_WAVE + lane] * w1;
    }
    if (!q_ok) return;
    // o[dt][4*j + i] is element 32*dt + 8*j + 4*h + i of query r32
    if (splits > 1) {
        const size_t at = (static_cast<size_t>(row0 + wq) * nq + q_head) * splits + split;
        if (h == 0) {
            part_ml[at * 2] = m * scale_log2e;     // in the exponent's own unit; -inf stays
            part_ml[at * 2 + 1] = lsum;
        }
        float* arow = part_acc + at * d;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int e0 = 32 * dt + 8 * j + 4 * h;
                if (e0 < d) *reinterpret_cast<f32x4*>(arow + e0) = f32x4{o[dt][4 * j], o[dt][4 * j + 1], o[dt][4 * j + 2], o[dt][4 * j + 3]};
            }
        return;
    }
    const float total = lsum;
    const float inv = total > 0.f ? 1.f / total : 0.f;
    bf16_t* orow = out + (static_cast<size_t>(row0 + wq) * nq + q_head) * d;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e0 = 32 * dt + 8 * j + 4 * h;
            if (e0 < d) {
                ap_u32x2 w;
                w.v[0] = ap_pack2(o[dt][4 * j] * inv, o[dt][4 * j + 1] * inv);
                w.v[1] = ap_pack2(o[dt][4 * j + 2] * inv, o[dt][4 * j + 3] * inv);
                *reinterpret_cast<ap_u32x2*>(orow + e0) = w;
            }
        }
}

// Puts the splits of a token tile together: out = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M).
// The step's rows are its grid: blockIdx.x names a stretch of rows of q, blockIdx.y a query head; a thread takes
// four head elements of one row, finds the request the row belongs to (the requests' rows follow each other in
// q) and asks for all it needs at once.  A step of one portion beside many single tokens so has no workgroups
// for token tiles that do not exist.
// SP: the splits the registers are laid out for (every one of them is asked for, used or not).
#define AP_MERGE_MAX 16
template <int SP>
__global__ void __launch_bounds__(256)
paged_attention_prefill_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                                          bf16_t* __restrict__ out, const int* __restrict__ q_start,
                                          const int* __restrict__ q_len, const int* __restrict__ ctx_len,
                                          int short_limit, int num_seqs, int nq, int d, int splits, int total_rows,
                                          int grouped) {
    const int quads = d / 4, rows = blockDim.x / quads;
    const int r = blockIdx.x * rows + threadIdx.x / quads;
    const int head = blockIdx.y;
    const int e0 = (threadIdx.x % quads) * 4;
    // The requests are read 64 at a time, one a lane; each lane says for each of the few rows of its wave
    // whether its request holds that row and is served here.
    const int lane = threadIdx.x & 63, wave_first = threadIdx.x - lane;
    const int row_first = blockIdx.x * rows + wave_first / quads, row_last = blockIdx.x * rows + (wave_first + 63) / quads;
    bool served = false;
    for (int base = 0; base < num_seqs; base += 64) {
        const int s = base + lane;
        int first = 0, count = 0;
        bool ok = false;
        if (s < num_seqs) {
            first = q_start[s];
            count = q_len[s];
            ok = ctx_len[s] > 0 && (grouped ? (short_limit <= 0 || count < short_limit) : count >= short_limit);
        }
        for (int row = row_first; row <= row_last; ++row) {
            const bool holds = __ballot(ok && row >= first && row < first + count) != 0;
            if (holds && row == r) served = true;
        }
    }
    if (static_cast<int>(threadIdx.x) >= rows * quads || r >= total_rows || !served) return;
    const size_t at = (static_cast<size_t>(r) * nq + head) * splits;
    float ms[SP], ls[SP];
    f32x4 os[SP];
#pragma unroll
    for (int sp = 0; sp < SP; ++sp) {
        const int sc = min(sp, splits - 1);
        const float2 ml = *reinterpret_cast<const float2*>(part_ml + (at + sc) * 2);
        ms[sp] = ml.x;
        ls[sp] = ml.y;
    }
    float big = -INFINITY;
#pragma unroll
    for (int sp = 0; sp < SP; ++sp) big = fmaxf(big, sp < splits ? ms[sp] : -INFINITY);
#pragma unroll
    for (int sp = 0; sp < SP; ++sp) {
        // a split that saw no key wrote no output: its place in the workspace holds anything
        const bool live = sp < splits && ms[sp] != -INFINITY;
        os[sp] = live ? *reinterpret_cast<const f32x4*>(part_acc + (at + sp) * d + e0) : f32x4{0.f, 0.f, 0.f, 0.f};
        ms[sp] = live ? exp2f(ms[sp] - big) : 0.f;
    }
    float sum = 0.f;
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sp = 0; sp < SP; ++sp) {
        sum = fmaf(ls[sp], ms[sp], sum);
        a += os[sp] * ms[sp];
    }
    const float inv = sum > 0.f ? 1.f / sum : 0.f;
    ap_u32x2 w;
    w.v[0] = ap_pack2(a[0] * inv, a[1] * inv);
    w.v[1] = ap_pack2(a[2] * inv, a[3] * inv);
    *reinterpret_cast<ap_u32x2*>(out + (static_cast<size_t>(r) * nq + head) * d + e0) = w;
}

template <int DT, int NW, int KS, int FEED, bool GR = false>
static int launch_prefill(const void* q, int q_stride, void* out, const int* q_start, const int* q_len,
                          const int* ctx_len, int short_limit, int num_seqs, int max_q_len, const int* block_table,
                          int max_blocks, int block_size, const void* k_pool, const void* v_pool, int nq, int nkv,
                          int d, float scale, int window, int splits, float* part_acc, float* part_ml,
                          int total_rows, int short_rows, hipStream_t stream) {
    constexpr int DP = 32 * DT;
    constexpr int BM = 32 * NW;
    const size_t tile_bytes = FEED == 2 ? (2 * ap_direct_ahead(GR) + 3) * static_cast<size_t>(AP_BN) * DP * 2
                                        : (2 * static_cast<size_t>(AP_BN) * (DP + AP_KPAD) +
                                           ap_value_buffers(KS) * static_cast<size_t>(AP_BN) * (DP + ap_vpad(DT))) * 2;
    const size_t hand_bytes = KS == 2 ? static_cast<size_t>(NW) * (16 * DT + 2) * PL_WAVE * sizeof(float) : 0;
    const size_t lds_bytes = tile_bytes > hand_bytes ? tile_bytes : hand_bytes;
    if (lds_bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&paged_attention_prefill_kernel<DT, NW, KS, FEED, GR>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
        PL_REQUIRE(e == hipSuccess, "prefill attention: %zu bytes of LDS refused: %s", lds_bytes, hipGetErrorString(e));
    }
    const int tiles = GR ? max_q_len : pl_ceil_div(max_q_len, BM);
    long long whole = static_cast<long long>(tiles) * (GR ? nkv : nq) * num_seqs;
    // The requests served bring total_rows tokens at most, and each of them short_limit at least: so many token
    // tiles there can be.  Where that is fewer than tiles of the longest times requests, workgroups are dealt
    // to the tiles that there are (ap_find_tile).
    // (Grouped, a tile is a token: there are total_rows of them at most, or short_rows where the caller knows
    // how many tokens the requests served here bring together.)
    int compact = 0;
    {
        const long long served = short_limit > 0 ? (total_rows / short_limit < num_seqs ? total_rows / short_limit : num_seqs) : num_seqs;
        const long long bound = GR ? (short_rows > 0 && short_rows < total_rows ? short_rows : total_rows)
                                   : (total_rows + served * (BM - 1)) / BM;
        if (bound < static_cast<long long>(tiles) * num_seqs) {
            compact = 1;
            whole = bound * (GR ? nkv : nq);
        }
    }
    const long long total = whole * splits;
    PL_REQUIRE(total > 0 && total < (1ll << 30), "prefill attention: %lld workgroups", total);
    paged_attention_prefill_kernel<DT, NW, KS, FEED, GR><<<static_cast<int>(total), 64 * NW * KS, lds_bytes, stream>>>(
        static_cast<const bf16_t*>(q), q_stride, static_cast<bf16_t*>(out), q_start, q_len, ctx_len, short_limit, tiles,
        num_seqs, block_table, max_blocks, block_size, static_cast<const bf16_t*>(k_pool),
        static_cast<const bf16_t*>(v_pool), nq, nkv, d, scale * 1.4426950408889634f, window, static_cast<int>(total),
        splits, part_acc, part_ml, compact);
    PL_CHECK_LAUNCH("paged_attention_prefill");
    if (splits > 1) {
        const int rows = 256 / (d / 4);
#define AP_MERGE(SP)                                                                                               \
    paged_attention_prefill_merge_kernel<SP><<<dim3(pl_ceil_div(total_rows, rows), nq), 256, 0, stream>>>(         \
        part_acc, part_ml, static_cast<bf16_t*>(out), q_start, q_len, ctx_len, short_limit, num_seqs, nq, d, splits, \
        total_rows, GR ? 1 : 0)
        if (splits <= 2) AP_MERGE(2);
        else if (splits <= 4) AP_MERGE(4);
        else if (splits <= 8) AP_MERGE(8);
        else AP_MERGE(AP_MERGE_MAX);
#undef AP_MERGE
        PL_CHECK_LAUNCH("paged_attention_prefill_merge");
    }
    return 0;
}

template <int D>
static int ap_dispatch(bool small, bool uniform_pages, const void* q, int q_stride, void* out, const int* q_start,
                       const int* q_len, const int* ctx_len, int short_limit, int num_seqs, int max_q_len,
                       const int* block_table, int max_blocks, int block_size, const void* k_pool, const void* v_pool,
                       int nq, int nkv, int d, float scale, int window, int splits, float* part_acc, float* part_ml,
                       int total_rows, hipStream_t stream) {
#define AP_LAUNCH(NW, KS, FEED)                                                                                    \
    launch_prefill<D, NW, KS, FEED>(q, q_stride, out, q_start, q_len, ctx_len, short_limit, num_seqs, max_q_len,    \
                                    block_table, max_blocks, block_size, k_pool, v_pool, nq, nkv, d, scale, window, \
                                    splits, part_acc, part_ml, total_rows, 0, stream)
    constexpr bool can_fit = 64 % (4 * D) == 0;
    constexpr int BEST = (D == 2 || D == 4) && AP_KS == 2 && AP_SMALL_KS == 2 ? AP_FEED : 1;   // the feed with uniform pages
    if constexpr (D <= 4) {
        if (small) {
            if constexpr (can_fit) {
                if (uniform_pages) return AP_LAUNCH(2, AP_SMALL_KS, BEST);
            }
            return AP_LAUNCH(2, AP_SMALL_KS, 0);
        }
        if constexpr (can_fit) {
            if (uniform_pages) return AP_LAUNCH(4, AP_KS, BEST);
        }
        return AP_LAUNCH(4, AP_KS, 0);
    } else {
        if constexpr (can_fit) {
            if (uniform_pages) return AP_LAUNCH(4, 1, 1);
        }
        return AP_LAUNCH(4, 1, 0);
    }
#undef AP_LAUNCH
}

// bfloat16 only.  q rows begin with the nq*d rotated query values; request s brings the rows
// q_start[s] .. q_start[s] + q_len[s] - 1, which stand at the positions ctx_len[s] - q_len[s] .. ctx_len[s] - 1.
// Requests with q_len < short_limit are skipped.  max_q_len bounds q_len over the requests.
// splits > 1 deals the keys of every token tile to that many workgroups; the workspace then needs
// rows*nq*splits*d floats (part_acc) and rows*nq*splits*2 (part_ml), rows being the step's rows of q.
// total_rows: the rows of q (the requests bring so many together at most); workgroups are dealt to the token
// tiles that can exist among them where that is fewer than tiles-of-the-longest for every request.
// pl_paged_attention_prefill_tile says how many tokens a token tile will have.
extern "C" int pl_paged_attention_prefill_tile(int max_q_len, int d) {
    return (max_q_len <= 64 && d <= 128) ? 64 : 128;
}

extern "C" int pl_paged_attention_prefill(const void* q, int q_stride, void* out, const int* q_start,
                                          const int* q_len, const int* ctx_len, int short_limit, int num_seqs,
                                          int max_q_len, const int* block_table, int max_blocks, int block_size,
                                          const void* k_pool, const void* v_pool, int nq, int nkv, int d,
                                          float scale, int window, int splits, float* part_acc, float* part_ml,
                                          int total_rows, hipStream_t stream) {
    PL_REQUIRE(splits >= 1 && splits <= AP_MERGE_MAX && (splits == 1 || (part_acc && part_ml)),
               "prefill attention: %d splits%s", splits, splits > 1 ? " without a workspace" : "");
    PL_REQUIRE(d > 0 && d <= 256 && d % 16 == 0, "prefill attention: head size %d, which has to be a multiple of 16 up to 256", d);
    PL_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "prefill attention: %d query heads over %d key heads", nq, nkv);
    PL_REQUIRE(block_size > 0 && max_blocks > 0 && q_stride >= nq * d && q_stride % 8 == 0 && window >= 0,
               "prefill attention: block size %d, %d blocks a row, query stride %d, window %d", block_size, max_blocks,
               q_stride, window);
    PL_REQUIRE((nkv * d) % 8 == 0, "prefill attention: a cache row of %d elements is not read 16 bytes at a time", nkv * d);
    if (num_seqs <= 0 || max_q_len <= 0) return 0;
    PL_REQUIRE(total_rows >= max_q_len, "prefill attention: %d rows for a portion of %d", total_rows, max_q_len);
    PL_REQUIRE(static_cast<unsigned long long>(block_size) * nkv * d * 2 < (1ull << 32),
               "prefill attention: a page of %d tokens of %d heads of %d takes more bytes than 32 bits count", block_size, nkv, d);
    const int dt = pl_ceil_div(d, 32);
    // few tokens a request: 64-token tiles give twice the workgroups
#ifdef AP_FORCE_SMALL
    const bool small = AP_FORCE_SMALL;
#else
    // half the threads have twice the pieces of a tile to carry each: large heads leave them no registers for that
    const bool small = max_q_len <= 64 && dt <= 4;
#endif
    // one instruction of a wave loads 64 / (4*D) keys: they share a page when pages are a power of two that large
    const bool pages_fit = (block_size & (block_size - 1)) == 0 && block_size * 4 * dt >= 64 && 64 % (4 * dt) == 0;
#define AP_CALL(D)                                                                                                 \
    return ap_dispatch<D>(small, pages_fit, q, q_stride, out, q_start, q_len, ctx_len, short_limit, num_seqs, max_q_len, \
                          block_table, max_blocks, block_size, k_pool, v_pool, nq, nkv, d, scale, window, splits,   \
                          part_acc, part_ml, total_rows, stream)
    switch (dt) {
        case 1: AP_CALL(1);
        case 2: AP_CALL(2);
        case 3: AP_CALL(3);
        case 4: AP_CALL(4);
        case 5: AP_CALL(5);
        case 6: AP_CALL(6);
        case 7: AP_CALL(7);
        default: AP_CALL(8);
    }
#undef AP_CALL
}

// One token's query heads of a key-head group as the rows of a tile (see GR above): for single tokens and the
// tokens of short portions where a group has four heads or more, so that the keys are read once a group and
// multiplied on the matrix cores.  Same arguments as pl_paged_attention_prefill, but requests with
// short_limit tokens or more are the ones left out (0: none is), and max_q_len bounds the tokens of those
// that are served.  Heads of 64 or 128, groups of up to 32, pages of a power of two of at least
// 64 / (head size / 8) tokens; pl_paged_attention_grouped_applies says whether a shape is served.
// short_rows: the most tokens that the requests served bring together (0: not known, the step's rows then).
extern "C" int pl_paged_attention_grouped_applies(int nq, int nkv, int d, int block_size) {
    if (nq <= 0 || nkv <= 0 || nq % nkv || nq / nkv > 32 || (d != 64 && d != 128)) return 0;
    const int rows_a_load = 64 / (d / 8);
    return block_size >= rows_a_load && (block_size & (block_size - 1)) == 0 ? 1 : 0;
}

extern "C" int pl_paged_attention_grouped(const void* q, int q_stride, void* out, const int* q_start,
                                          const int* q_len, const int* ctx_len, int short_limit, int num_seqs,
                                          int max_q_len, const int* block_table, int max_blocks, int block_size,
                                          const void* k_pool, const void* v_pool, int nq, int nkv, int d,
                                          float scale, int window, int splits, float* part_acc, float* part_ml,
                                          int total_rows, int short_rows, hipStream_t stream) {
    PL_REQUIRE(pl_paged_attention_grouped_applies(nq, nkv, d, block_size),
               "grouped attention: %d query heads over %d key heads of %d, pages of %d", nq, nkv, d, block_size);
    PL_REQUIRE(splits >= 1 && splits <= AP_MERGE_MAX && (splits == 1 || (part_acc && part_ml)),
               "grouped attention: %d splits%s", splits, splits > 1 ? " without a workspace" : "");
    PL_REQUIRE(max_blocks > 0 && q_stride >= nq * d && q_stride % 8 == 0 && window >= 0,
               "grouped attention: %d blocks a row, query stride %d, window %d", max_blocks, q_stride, window);
    if (num_seqs <= 0 || max_q_len <= 0) return 0;
    PL_REQUIRE(total_rows >= max_q_len, "grouped attention: %d rows for portions of %d", total_rows, max_q_len);
    PL_REQUIRE(static_cast<unsigned long long>(block_size) * nkv * d * 2 < (1ull << 32),
               "grouped attention: a page of %d tokens of %d heads of %d takes more bytes than 32 bits count", block_size, nkv, d);
    if (d == 64)
        return launch_prefill<2, 1, 2, 2, true>(q, q_stride, out, q_start, q_len, ctx_len, short_limit, num_seqs, max_q_len,
                                                block_table, max_blocks, block_size, k_pool, v_pool, nq, nkv, d, scale,
                                                window, splits, part_acc, part_ml, total_rows, short_rows, stream);
    return launch_prefill<4, 1, 2, 2, true>(q, q_stride, out, q_start, q_len, ctx_len, short_limit, num_seqs, max_q_len,
                                            block_table, max_blocks, block_size, k_pool, v_pool, nq, nkv, d, scale,
                                            window, splits, part_acc, part_ml, total_rows, short_rows, stream);
}

// Choosing the next token on the device.
#include "common.hpp"
#include "no_alloc.h"

#include <mutex>

// ---------------------------------------------------------------------------
// Greedy: the index of the largest logit of each row; the first maximum wins
// (ties go to the lower index), NaNs never win.  Two stages, so that a few rows
// over a vocabulary of a hundred and fifty thousand still fill the chip: every
// row is cut into ARGMAX_CHUNKS stretches whose winners a second kernel compares.
// ---------------------------------------------------------------------------
#define ARGMAX_CHUNKS 64

__device__ __forceinline__ void better(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) {
        bv = v;
        bi = i;
    }
}

__device__ __forceinline__ void block_best(float& bv, int& bi) {
    __shared__ float best_v[4];
    __shared__ int best_i[4];
#pragma unroll
    for (int off = PL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, PL_WAVE);
        const int oi = __shfl_xor(bi, off, PL_WAVE);
        better(bv, bi, ov, oi);
    }
    const int wave = threadIdx.x / PL_WAVE;
    if (threadIdx.x % PL_WAVE == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int w = 1; w < static_cast<int>(blockDim.x) / PL_WAVE; ++w) better(bv, bi, best_v[w], best_i[w]);
}

__global__ void __launch_bounds__(256)
argmax_stage1_kernel(const float* __restrict__ logits, float* __restrict__ part_v, int* __restrict__ part_i, int V) {
    const int row = blockIdx.y, chunk = blockIdx.x;
    const int per = (V + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
    const int begin = chunk * per, end = min(V, begin + per);
    const float* x = logits + static_cast<size_t>(row) * V;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) better(bv, bi, x[i], i);
    block_best(bv, bi);
    if (threadIdx.x == 0) {
        part_v[row * ARGMAX_CHUNKS + chunk] = bv;
        part_i[row * ARGMAX_CHUNKS + chunk] = bi;
    }
}

__global__ void __launch_bounds__(64)
argmax_stage2_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i, int* __restrict__ out) {
    const int row = blockIdx.x;
    float bv = part_v[row * ARGMAX_CHUNKS + threadIdx.x];
    int bi = part_i[row * ARGMAX_CHUNKS + threadIdx.x];
#pragma unroll
    for (int off = PL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, PL_WAVE);
        const int oi = __shfl_xor(bi, off, PL_WAVE);
        better(bv, bi, ov, oi);
    }
    if (threadIdx.x == 0) out[row] = bi == 0x7fffffff ? 0 : bi;
}

// scratch: m * 64 floats and m * 64 ints.
extern "C" int pl_argmax(const float* logits, int* out, float* scratch_v, int* scratch_i, int m, int V,
                         hipStream_t stream) {
    PL_REQUIRE(m >= 0 && V > 0 && m <= 65535, "argmax: rows %d, vocabulary %d", m, V);
    if (m == 0) return 0;
    static_assert(ARGMAX_CHUNKS == PL_WAVE, "the second stage is one wave a row");
    argmax_stage1_kernel<<<dim3(ARGMAX_CHUNKS, m), 256, 0, stream>>>(logits, scratch_v, scratch_i, V);
    PL_CHECK_LAUNCH("argmax");
    argmax_stage2_kernel<<<m, 64, 0, stream>>>(scratch_v, scratch_i, out);
    PL_CHECK_LAUNCH("argmax");
    return 0;
}

// The same two kernels over scratch memory that the library owns, for callers that cannot allocate.
// The array's name is only a handle on the host: what kernels are given is its address on the current
// device, asked for once a device (every GPU holds its own copy at its own address).
static __device__ __align__(256) unsigned char scratch[PL_ARGMAX_STATIC_MAX_ROWS * ARGMAX_CHUNKS * (sizeof(float) + sizeof(int))];

#define PL_MAX_DEVICES 64
static std::mutex scratch_lock;
static void* scratch_on_device[PL_MAX_DEVICES];

static int scratch_address(void** at) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    PL_REQUIRE(e == hipSuccess, "argmax: no current device: %s", hipGetErrorString(e));
    PL_REQUIRE(device >= 0 && device < PL_MAX_DEVICES, "argmax: device %d is beyond the %d this library counts", device, PL_MAX_DEVICES);
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (!scratch_on_device[device]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        PL_REQUIRE(e == hipSuccess && ptr, "argmax: the scratch array has no address on device %d: %s", device, hipGetErrorString(e));
        scratch_on_device[device] = ptr;
    }
    *at = scratch_on_device[device];
    return 0;
}

extern "C" int pl_argmax_static(const float* logits, int* out, int m, int V, hipStream_t stream) {
    PL_REQUIRE(m >= 0 && V > 0, "argmax: rows %d, vocabulary %d", m, V);
    PL_REQUIRE(m <= PL_ARGMAX_STATIC_MAX_ROWS, "argmax: %d rows, the scratch array of this entry point holds %d", m,
               PL_ARGMAX_STATIC_MAX_ROWS);
    if (m == 0) return 0;
    void* base = nullptr;
    if (int code = scratch_address(&base)) return code;
    float* part_v = static_cast<float*>(base);
    int* part_i = reinterpret_cast<int*>(part_v + PL_ARGMAX_STATIC_MAX_ROWS * ARGMAX_CHUNKS);
    argmax_stage1_kernel<<<dim3(ARGMAX_CHUNKS, m), 256, 0, stream>>>(logits, part_v, part_i, V);
    PL_CHECK_LAUNCH("argmax");
    argmax_stage2_kernel<<<m, 64, 0, stream>>>(part_v, part_i, out);
    PL_CHECK_LAUNCH("argmax");
    return 0;
}

// ---------------------------------------------------------------------------
// Temperature, top-k, top-p and the draw, one workgroup a row (reference:
// crates/pagedllm/src/sampler.rs: scale, sort downwards, keep k, softmax, keep
// the shortest head of mass top_p, walk it with one uniform number).
//
// Nothing is sorted here.  Every step of that recipe asks for a place in the
// downward order at which a running sum crosses a mark: the k-th candidate (a
// sum of ones), the candidate at which the mass reaches top_p of the total,
// the candidate at which it reaches the drawn point.  Such a place is found by
// histogram passes over a 24-bit key that falls as the logit rises:
//     key = min(2^26 - 1, (max - y) * 2^20) >> 2,   y = logit / temperature,
// 12 bits a pass; the second pass is left out when the bin that the first one
// finds holds a single candidate, which is the usual case near the top of a
// row.  Logits closer than 4e-6 share a key and count as equal: they
// are ordered by index, as equal logits are in the recipe.  Logits more than 64
// below the maximum share the last key; their mass is zero.
//
// Masses are exp(y - max) in fixed point (2^40), added as integers: a sum does
// not depend on the order of its terms, so a row and a uniform number give the
// same token on every run.
// ---------------------------------------------------------------------------
#define SM_THREADS 1024
#define SM_BINS 4096
#define SM_NO_LIMIT 0x7fffffff
#define SM_LIST 256                    // the most candidates that top-k may keep for the short way (see sm_few)

struct sm_shared {
    unsigned long long sum[SM_BINS];   // mass, or count, a bin
    unsigned int count[SM_BINS];       // candidates a bin (second pass)
    int first[SM_BINS];                // lowest index a bin (second pass)
    unsigned long long wave_sum[SM_THREADS / PL_WAVE];
    float red_v[SM_THREADS / PL_WAVE];
    int red_i[SM_THREADS / PL_WAVE];
    unsigned long long found_before;   // sum over the bins before the one found
    unsigned long long found_in;       // sum of the bin found
    int found_bin;
    int nth_index;
    // the short way after top-k: the candidates kept, as they are found and in order
    uint32_t list_key[SM_LIST];
    int list_idx[SM_LIST];
    unsigned long long list_mass[SM_LIST];
    int list_order[SM_LIST];           // list_order[r]: which entry stands at place r of the order (key, then index)
    uint32_t maybe_key[SM_LIST];       // the candidates of the bin in which the k-th stands
    int maybe_idx[SM_LIST];
    int list_n, maybe_n;
};

__device__ __forceinline__ uint32_t sm_key(float y, float top) {
    if (!(y == y)) return (1u << 24) - 1;                      // a NaN is the last candidate
    const float t = (top - y) * 1048576.f;                      // >= 0, +inf for -inf
    const uint32_t q = t >= 67108863.f ? 67108863u : static_cast<uint32_t>(t);
    return q >> 2;
}

__device__ __forceinline__ unsigned long long sm_mass(float y, float top) {
    // 2^40 * exp(y - top): zero from about 28 below the maximum on
    const float p = __builtin_amdgcn_exp2f((y - top) * 1.4426950408889634f + 40.f);
    return (y == y) ? static_cast<unsigned long long>(p) : 0ull;
}

// f(value, index) for every element of a row that falls to this thread, in rising order.  Eight loads are asked
// for before the first is used: a pass over a row is one workgroup's and lives on what it has in flight.
template <class F>
__device__ __forceinline__ void sm_each(const float* __restrict__ x, int V, F&& f) {
    constexpr int AHEAD = 8;
    int i = threadIdx.x;
    for (; i + (AHEAD - 1) * SM_THREADS < V; i += AHEAD * SM_THREADS) {
        float v[AHEAD];
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) v[j] = x[i + j * SM_THREADS];
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) f(v[j], i + j * SM_THREADS);
    }
    for (; i < V; i += SM_THREADS) f(x[i], i);
}

// The mark that is `fraction` of `total`, at least one and at most all of it.
__device__ __forceinline__ unsigned long long sm_mark_of(double fraction, unsigned long long total) {
    const unsigned long long mark = static_cast<unsigned long long>(fraction * static_cast<double>(total));
    return mark < 1 ? 1 : (mark > total ? total : mark);
}

// The first bin, going up, at which the running sum of sm.sum reaches the mark (the last bin that holds
// anything if the sum never gets there).  The mark is `mark` (>= 1), or, with fraction >= 0, that fraction
// of the sum over all bins.  Leaves found_bin, found_before, found_in and returns the mark it used.
__device__ unsigned long long sm_find(sm_shared& sm, unsigned long long before, unsigned long long mark, double fraction) {
    constexpr int PER = SM_BINS / SM_THREADS;                  // bins a thread
    const int tid = threadIdx.x, lane = tid % PL_WAVE, wave = tid / PL_WAVE;
    unsigned long long mine = 0;
#pragma unroll
    for (int b = 0; b < PER; ++b) mine += sm.sum[tid * PER + b];
    // running sum over the threads of the wave, then over the waves
    unsigned long long run = mine;
#pragma unroll
    for (int off = 1; off < PL_WAVE; off <<= 1) {
        const unsigned long long other = __shfl_up(run, off, PL_WAVE);
        if (lane >= off) run += other;
    }
    if (lane == PL_WAVE - 1) sm.wave_sum[wave] = run;
    if (tid == 0) sm.found_bin = -1;
    __syncthreads();
    unsigned long long ahead = before, total = before;
    for (int w = 0; w < SM_THREADS / PL_WAVE; ++w) {
        const unsigned long long v = sm.wave_sum[w];
        if (w < wave) ahead += v;
        total += v;
    }
    if (fraction >= 0.0) mark = sm_mark_of(fraction, total);
    const unsigned long long through = ahead + run, upto = through - mine;   // sums through / before this thread's bins
    if (upto < mark && mark <= through) {
        unsigned long long at = upto;
        for (int b = 0; b < PER; ++b) {
            const unsigned long long v = sm.sum[tid * PER + b];
            if (at + v >= mark) {
                sm.found_bin = tid * PER + b;
                sm.found_before = at;
                sm.found_in = v;
                break;
            }
            at += v;
        }
    }
    __syncthreads();
    if (sm.found_bin < 0) {                                     // the mark lies past the total: the last bin in use
        if (tid == SM_THREADS - 1) {
            int b = SM_BINS - 1;
            while (b > 0 && sm.sum[b] == 0) --b;
            sm.found_bin = b;
            sm.found_in = sm.sum[b];
            unsigned long long tail = 0;
            for (int c = b; c < SM_BINS; ++c) tail += sm.sum[c];
            sm.found_before = total - tail;
        }
        __syncthreads();
    }
    return mark;
}

// Which candidates are still in: keys below `key`, and of that key the indices below `limit`.
struct sm_kept {
    uint32_t key;
    int limit;
    __device__ __forceinline__ bool has(uint32_t k, int i) const { return k < key || (k == key && i < limit); }
};

// The place, in the order of key then index, at which the running sum of `weight` over the kept
// candidates reaches the mark: `mark`, or with fraction >= 0 that fraction of the sum over all of them.
// Returns the key found; `limit` becomes the index after the candidate at which the mark is reached,
// `through` the sum up to and with that candidate, and `token` that candidate.  WEIGHTED: masses, else
// ones.  A first pass over the upper 12 bits of the keys; a second over the lower 12 only if the bin
// found holds more than one candidate.
template <bool WEIGHTED>
__device__ uint32_t sm_select(sm_shared& sm, const float* __restrict__ x, int V, float inverse, float top, sm_kept kept,
                              unsigned long long mark, double fraction, int& limit, unsigned long long& through, int& token) {
    const int tid = threadIdx.x;
    auto clear = [&]() {
        for (int b = tid; b < SM_BINS; b += SM_THREADS) {
            sm.sum[b] = 0;
            sm.count[b] = 0;
            sm.first[b] = SM_NO_LIMIT;
        }
        __syncthreads();
    };
    clear();
    sm_each(x, V, [&](float v, int i) {
        const float y = v * inverse;
        const uint32_t k = sm_key(y, top);
        if (!kept.has(k, i)) return;
        const unsigned long long w = WEIGHTED ? sm_mass(y, top) : 1ull;
        if (w) {
            atomicAdd(&sm.sum[k >> 12], w);
            atomicAdd(&sm.count[k >> 12], 1u);
            atomicMin(&sm.first[k >> 12], i);
        }
    });
    __syncthreads();
    mark = sm_find(sm, 0, mark, fraction);
    const uint32_t upper = sm.found_bin;
    uint32_t key;
    unsigned long long before = sm.found_before, in_bin = sm.found_in;
    unsigned int many = sm.count[upper];
    int lowest = sm.first[upper];
    __syncthreads();
    if (many == 1) {
        key = sm_key(x[lowest] * inverse, top);
    } else {
        const unsigned long long before_upper = before;
        clear();
        sm_each(x, V, [&](float v, int i) {
            const float y = v * inverse;
            const uint32_t k = sm_key(y, top);
            if ((k >> 12) != upper || !kept.has(k, i)) return;
            const unsigned long long w = WEIGHTED ? sm_mass(y, top) : 1ull;
            if (w) {
                atomicAdd(&sm.sum[k & 0xfff], w);
                atomicAdd(&sm.count[k & 0xfff], 1u);
                atomicMin(&sm.first[k & 0xfff], i);
            }
        });
        __syncthreads();
        sm_find(sm, before_upper, mark, -1.0);
        key = (upper << 12) | static_cast<uint32_t>(sm.found_bin);
        before = sm.found_before;
        in_bin = sm.found_in;
        many = sm.count[sm.found_bin];
        lowest = sm.first[sm.found_bin];
        __syncthreads();
    }
    if (many <= 1) {                                            // the usual case: one candidate has this key
        limit = many == 1 ? lowest + 1 : SM_NO_LIMIT;
        through = before + in_bin;
        token = many == 1 ? lowest : 0;
        return key;
    }
    // Several candidates share the key.  A few of them are gathered in one pass and one thread walks them
    // in the order of their indices; more than SM_LIST are walked where they lie, a stretch of SM_THREADS
    // indices at a time, until the running sum reaches the mark.
    unsigned long long run = before;
    if (tid == 0) {
        sm.nth_index = -1;
        sm.maybe_n = 0;
    }
    __syncthreads();
    const int lane = tid % PL_WAVE, wave = tid / PL_WAVE;
    if (many <= SM_LIST) {
        sm_each(x, V, [&](float v, int i) {
            const float y = v * inverse;
            const uint32_t k = sm_key(y, top);
            if (k != key || !kept.has(k, i)) return;
            const unsigned long long w = WEIGHTED ? sm_mass(y, top) : 1ull;
            if (w) {
                const int at = atomicAdd(&sm.maybe_n, 1);
                sm.maybe_idx[at] = i;
                sm.list_mass[at] = w;
            }
        });
        __syncthreads();
        const int n = sm.maybe_n;                               // == many: the same candidates were counted
        if (tid < n) {
            int place = 0;
            for (int j = 0; j < n; ++j) place += sm.maybe_idx[j] < sm.maybe_idx[tid] ? 1 : 0;
            sm.list_order[place] = tid;
        }
        __syncthreads();
        if (tid == 0) {
            for (int r = 0; r < n; ++r) {
                const int e = sm.list_order[r];
                run += sm.list_mass[e];
                if (run >= mark) {
                    sm.nth_index = sm.maybe_idx[e];
                    sm.found_before = run;
                    break;
                }
            }
        }
        __syncthreads();
    } else
    for (int base = 0; base < V; base += SM_THREADS) {
        const int i = base + tid;
        unsigned long long w = 0;
        if (i < V) {
            const float y = x[i] * inverse;
            const uint32_t k = sm_key(y, top);
            if (k == key && kept.has(k, i)) w = WEIGHTED ? sm_mass(y, top) : 1ull;
        }
        unsigned long long scan = w;
#pragma unroll
        for (int off = 1; off < PL_WAVE; off <<= 1) {
            const unsigned long long other = __shfl_up(scan, off, PL_WAVE);
            if (lane >= off) scan += other;
        }
        if (lane == PL_WAVE - 1) sm.wave_sum[wave] = scan;
        __syncthreads();
        unsigned long long ahead = run, all = 0;
        for (int v = 0; v < SM_THREADS / PL_WAVE; ++v) {
            if (v < wave) ahead += sm.wave_sum[v];
            all += sm.wave_sum[v];
        }
        const unsigned long long mine_through = ahead + scan;
        if (w && mine_through - w < mark && mark <= mine_through) {
            sm.nth_index = i;
            sm.found_before = mine_through;
        }
        __syncthreads();
        if (sm.nth_index >= 0) break;
        run += all;
        __syncthreads();
    }
    if (sm.nth_index >= 0) {
        limit = sm.nth_index + 1;
        through = sm.found_before;
        token = sm.nth_index;
    } else {                                                    // the mark lies past them all: all are kept, the last is drawn
        limit = SM_NO_LIMIT;
        through = before + in_bin;
        token = lowest;
    }
    __syncthreads();
    return key;
}

// Top-k with few candidates kept (k <= SM_LIST), and everything after it: one pass finds the bin of the upper
// 12 key bits in which the k-th candidate stands, a second gathers the candidates of the bins before it (kept for
// certain) and those of that bin, of which the first k - (kept so far) in the order (key, index) are kept too.
// The k candidates are then ordered and one thread walks them: the mass up to top_p of the total, and in what
// is left the drawn point.  Three passes over the row with the one for the maximum, where the general way
// takes five to seven.  Returns false (the same in every thread, nothing decided) when the k-th candidate's
// bin holds more than SM_LIST candidates: the general way then serves the row.
__device__ bool sm_few(sm_shared& sm, const float* __restrict__ x, int V, float inverse, float top, int k, float p,
                       float u, int& token) {
    const int tid = threadIdx.x;
    for (int b = tid; b < SM_BINS; b += SM_THREADS) sm.sum[b] = 0;
    if (tid == 0) sm.list_n = sm.maybe_n = 0;
    __syncthreads();
    sm_each(x, V, [&](float v, int) { atomicAdd(&sm.sum[sm_key(v * inverse, top) >> 12], 1ull); });
    __syncthreads();
    sm_find(sm, 0, static_cast<unsigned long long>(k), -1.0);
    const uint32_t upper = sm.found_bin;
    const int sure = static_cast<int>(sm.found_before), in_bin = static_cast<int>(sm.found_in);
    __syncthreads();
    if (in_bin > SM_LIST) return false;
    sm_each(x, V, [&](float v, int i) {
        const uint32_t key = sm_key(v * inverse, top);
        if ((key >> 12) < upper) {
            const int at = atomicAdd(&sm.list_n, 1);
            sm.list_key[at] = key;
            sm.list_idx[at] = i;
        } else if ((key >> 12) == upper) {
            const int at = atomicAdd(&sm.maybe_n, 1);
            sm.maybe_key[at] = key;
            sm.maybe_idx[at] = i;
        }
    });
    __syncthreads();
    // of the k-th candidate's bin, the first k - sure in the order
    if (tid < in_bin) {
        const uint32_t key = sm.maybe_key[tid];
        const int idx = sm.maybe_idx[tid];
        int before = 0;
        for (int j = 0; j < in_bin; ++j)
            before += (sm.maybe_key[j] < key || (sm.maybe_key[j] == key && sm.maybe_idx[j] < idx)) ? 1 : 0;
        if (before < k - sure) {
            sm.list_key[sure + before] = key;
            sm.list_idx[sure + before] = idx;
        }
    }
    __syncthreads();
    // masses, and the place of every kept candidate in the order
    if (tid < k) {
        const uint32_t key = sm.list_key[tid];
        const int idx = sm.list_idx[tid];
        sm.list_mass[tid] = sm_mass(x[idx] * inverse, top);
        int before = 0;
        for (int j = 0; j < k; ++j)
            before += (sm.list_key[j] < key || (sm.list_key[j] == key && sm.list_idx[j] < idx)) ? 1 : 0;
        sm.list_order[before] = tid;
    }
    __syncthreads();
    if (tid == 0) {
        unsigned long long total = 0;
        for (int r = 0; r < k; ++r) total += sm.list_mass[sm.list_order[r]];
        int last = k - 1;                                       // the last candidate that top_p keeps
        if (p < 1.f) {
            const unsigned long long mark = sm_mark_of(static_cast<double>(p), total);
            unsigned long long run = 0;
            for (int r = 0; r < k; ++r) {
                run += sm.list_mass[sm.list_order[r]];
                if (run >= mark) {
                    last = r;
                    break;
                }
            }
            total = run;
        }
        const unsigned long long mark = sm_mark_of(static_cast<double>(u), total);
        unsigned long long run = 0;
        int chosen = sm.list_order[0];
        for (int r = 0; r <= last; ++r) {
            const int e = sm.list_order[r];
            run += sm.list_mass[e];
            if (sm.list_mass[e] && run >= mark) {
                chosen = e;
                break;
            }
        }
        sm.nth_index = sm.list_idx[chosen];
    }
    __syncthreads();
    token = sm.nth_index;
    __syncthreads();
    return true;
}

__global__ void __launch_bounds__(SM_THREADS)
sample_rows_kernel(const float* __restrict__ logits, const float* __restrict__ temperature, const int* __restrict__ top_k,
                   const float* __restrict__ top_p, const float* __restrict__ uniform, int* __restrict__ out, int V,
                   int out_holds_largest) {
    __shared__ sm_shared sm;
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* x = logits + static_cast<size_t>(row) * V;
    const float temp = temperature[row];
    // the largest logit and its first index: already in out[row] where the caller says so (an argmax by the same
    // rule ran before), unless what stands there is no finite number's place (a row of NaNs has none)
    float bv = -INFINITY;
    int bi = SM_NO_LIMIT;
    bool known = false;
    if (out_holds_largest) {
        const int hint = out[row];
        if (hint >= 0 && hint < V) {
            const float v = x[hint];
            if (v > -INFINITY) {                                // (false for a NaN)
                bv = v;
                bi = hint;
                known = true;
            }
        }
    }
    if (!known) {                                               // (the same in every thread)
        sm_each(x, V, [&](float v, int i) { better(bv, bi, v, i); });
#pragma unroll
        for (int off = PL_WAVE / 2; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, PL_WAVE);
            const int oi = __shfl_xor(bi, off, PL_WAVE);
            better(bv, bi, ov, oi);
        }
        if (tid % PL_WAVE == 0) {
            sm.red_v[tid / PL_WAVE] = bv;
            sm.red_i[tid / PL_WAVE] = bi;
        }
        __syncthreads();
        bv = sm.red_v[0];
        bi = sm.red_i[0];
        for (int w = 1; w < SM_THREADS / PL_WAVE; ++w) better(bv, bi, sm.red_v[w], sm.red_i[w]);
        __syncthreads();
    }
    if (!(temp > 0.f) || bi == SM_NO_LIMIT) {                   // greedy, or a row of NaNs
        if (tid == 0) out[row] = bi == SM_NO_LIMIT ? 0 : bi;
        return;
    }
    const float inverse = 1.0f / temp;
    const float top = bv * inverse;

    sm_kept kept{(1u << 24), SM_NO_LIMIT};                      // everything
    int limit, token;
    unsigned long long through;
    const int k = top_k[row];
    if (k > 0 && k < V && k <= SM_LIST && sm_few(sm, x, V, inverse, top, k, top_p[row], uniform[row], token)) {
        if (tid == 0) out[row] = token;
        return;
    }
    if (k > 0 && k < V) {
        const uint32_t key = sm_select<false>(sm, x, V, inverse, top, kept, static_cast<unsigned long long>(k), -1.0, limit, through, token);
        kept = sm_kept{key, limit};
    }
    const float p = top_p[row];
    double fraction = static_cast<double>(uniform[row]);       // of everything kept
    unsigned long long mark = 0;
    if (p < 1.f) {
        const uint32_t key = sm_select<true>(sm, x, V, inverse, top, kept, 0, static_cast<double>(p), limit, through, token);
        kept = sm_kept{key, limit};
        mark = sm_mark_of(fraction, through);                   // the candidate that crosses the mark is kept
        fraction = -1.0;
    }
    sm_select<true>(sm, x, V, inverse, top, kept, mark, fraction, limit, through, token);
    if (tid == 0) out[row] = token;
}

// One token a row.  temperature <= 0: the largest logit (the first of equals).  top_k <= 0 or >= V and
// top_p >= 1 switch the cuts off.  uniform: a number in [0, 1) a row, the request's own draw.
// out_holds_largest: out[row] already is the place of the row's largest logit, as pl_argmax leaves it (the first
// of equals, NaNs never); the pass over the row that would find it is then left out.
extern "C" int pl_sample(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                         const float* uniform, int* out, int m, int V, int out_holds_largest, hipStream_t stream) {
    PL_REQUIRE(m >= 0 && V > 0, "sampling: rows %d, vocabulary %d", m, V);
    if (m == 0) return 0;
    sample_rows_kernel<<<m, SM_THREADS, 0, stream>>>(logits, temperature, top_k, top_p, uniform, out, V,
                                                     out_holds_largest ? 1 : 0);
    PL_CHECK_LAUNCH("sample");
    return 0;
}

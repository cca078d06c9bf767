// Next-token choice on the device: argmax, and the reference's sampler
// (src/utils.cpp:31-115): logits times 1/temp, repeat penalty on the ids of the
// last-n window (negative logits multiplied, others divided, :46-56), the top_k
// largest kept (:21-29), softmax with the max subtracted (:65-84), the shortest
// prefix in descending order whose probability reaches top_p kept and renormalised
// (:86-101), one draw from what is left (:111-114).
//
// The reference sorts on the CPU; here nothing is sorted.  The k-th largest value
// and the top_p cut are found by bisection over the order-preserving integer image
// of the floats (ties go to the lower id, as a stable descending sort would put
// them), and the draw is the inverse CDF over the kept ids in ascending id order
// at a uniform number that is a hash of (seed, counter): the same request gives the
// same tokens whatever else is in the batch.
#include <math.h>

#include "api.h"
#include "common.h"

#define SB 1024  // threads of a sampling block

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// splitmix64 of seed + (counter + 1) * golden ratio; 24 bits -> [0, 1)
__device__ __forceinline__ float uniform_from(uint64_t seed, int32_t counter) {
    uint64_t z = seed + 0x9E3779B97F4A7C15ull * (uint64_t)((int64_t)counter + 1);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

template <typename T>
__device__ __forceinline__ T block_sum_t(T v, T* red) {
    const int lane = threadIdx.x & (ILLM_WAVE - 1), w = threadIdx.x / ILLM_WAVE;
#pragma unroll
    for (int o = ILLM_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, ILLM_WAVE);
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    T t = 0;
    for (int i = 0; i < SB / ILLM_WAVE; ++i) t += red[i];
    return t;
}

// exclusive prefix over the block's threads in thread order; `total` = sum of all
template <typename T>
__device__ __forceinline__ T block_exclusive_scan(T v, T* red, T* total) {
    const int lane = threadIdx.x & (ILLM_WAVE - 1), w = threadIdx.x / ILLM_WAVE;
    T inc = v;
#pragma unroll
    for (int o = 1; o < ILLM_WAVE; o <<= 1) {
        const T n = __shfl_up(inc, o, ILLM_WAVE);
        if (lane >= o) inc += n;
    }
    __syncthreads();
    if (lane == ILLM_WAVE - 1) red[w] = inc;
    __syncthreads();
    T before = 0, all = 0;
    for (int i = 0; i < SB / ILLM_WAVE; ++i) {
        if (i < w) before += red[i];
        all += red[i];
    }
    *total = all;
    return before + inc - v;
}

// Walks of a row by one block wait for each load in turn unless several are asked for at once:
// these bring eight values at a time, all loads issued before the first is used.
typedef float sample_f32x4_t __attribute__((ext_vector_type(4)));

template <typename F>
__device__ __forceinline__ void each_strided8(const float* a, int n, int tid, F f) {
    if ((((size_t)a) & 15) == 0) {
        // 16 bytes a load where the row starts at a multiple of 16 bytes (the same for the whole
        // block): four loads of four values in flight a thread, a quarter of the trips
        const int n4 = n >> 2;
        const sample_f32x4_t* a4 = (const sample_f32x4_t*)a;
        for (int base = tid; base < n4; base += SB * 4) {
            sample_f32x4_t v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i4 = base + u * SB;
                v[u] = i4 < n4 ? a4[i4] : (sample_f32x4_t){0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i4 = base + u * SB;
                if (i4 < n4) {
                    f(4 * i4, v[u][0]);
                    f(4 * i4 + 1, v[u][1]);
                    f(4 * i4 + 2, v[u][2]);
                    f(4 * i4 + 3, v[u][3]);
                }
            }
        }
        for (int i = 4 * n4 + tid; i < n; i += SB) f(i, a[i]);
        return;
    }
    for (int base = tid; base < n; base += SB * 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = base + u * SB;
            v[u] = i < n ? a[i] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = base + u * SB;
            if (i < n) f(i, v[u]);
        }
    }
}

template <typename F>
__device__ __forceinline__ void each_in_order8(const float* a, int lo, int hi, F f) {
    for (int base = lo; base < hi; base += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = base + u < hi ? a[base + u] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (base + u < hi) f(base + u, v[u]);
    }
}

// ---------------------------------------------------------------- argmax
// The lowest id among the largest values of a row; NaN never wins, a row of nothing else gives 0.
// A row is cut into gridDim.x parts (a block each, eight loads in flight a thread) that leave
// (value, id) pairs; the second kernel takes the best of a row's parts.  With one part the
// first kernel writes the id itself.
__device__ __forceinline__ void argmax_take(float& best, int& idx, float v, int i) {
    if (v > best || (v == best && i < idx) || idx == 0x7fffffff) {
        if (!(v != v)) { best = v; idx = i; }
    }
}

__global__ void __launch_bounds__(SB)
argmax_kernel(const float* __restrict__ logits, int32_t* __restrict__ out, float* __restrict__ part_v,
              int32_t* __restrict__ part_i, int V, int chunk) {
    __shared__ float bv[SB / ILLM_WAVE];
    __shared__ int bi[SB / ILLM_WAVE];
    const int lo = blockIdx.x * chunk, n = min(chunk, V - lo);
    const float* row = logits + (size_t)blockIdx.y * V + lo;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    each_strided8(row, n, threadIdx.x, [&](int i, float v) { argmax_take(best, idx, v, lo + i); });
#pragma unroll
    for (int o = ILLM_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, ILLM_WAVE);
        const int oi = __shfl_xor(idx, o, ILLM_WAVE);
        if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
    }
    const int lane = threadIdx.x & (ILLM_WAVE - 1), w = threadIdx.x / ILLM_WAVE;
    if (lane == 0) { bv[w] = best; bi[w] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < SB / ILLM_WAVE; ++i)
            if (bv[i] > best || (bv[i] == best && bi[i] < idx)) { best = bv[i]; idx = bi[i]; }
        if (gridDim.x == 1) {
            out[blockIdx.y] = idx == 0x7fffffff ? 0 : idx;
        } else {
            part_v[blockIdx.y * gridDim.x + blockIdx.x] = best;
            part_i[blockIdx.y * gridDim.x + blockIdx.x] = idx;
        }
    }
}

// one wave a row over its parts (at most 64)
__global__ void __launch_bounds__(ILLM_WAVE)
argmax_parts_kernel(const float* __restrict__ part_v, const int32_t* __restrict__ part_i,
                    int32_t* __restrict__ out, int parts) {
    const int lane = threadIdx.x;
    float best = lane < parts ? part_v[blockIdx.x * parts + lane] : -INFINITY;
    int idx = lane < parts ? part_i[blockIdx.x * parts + lane] : 0x7fffffff;
#pragma unroll
    for (int o = ILLM_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, ILLM_WAVE);
        const int oi = __shfl_xor(idx, o, ILLM_WAVE);
        if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
    }
    if (lane == 0) out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
}

// scratch: parts x B floats and as many int32 behind them (parts > 1), parts <= 64.
extern "C" int illm_argmax(const float* logits, int32_t* out, void* scratch, int B, int V, int parts,
                           void* stream) {
    if (B < 0 || V <= 0 || parts < 1 || parts > ILLM_WAVE || (parts > 1 && !scratch) || B > 65535)
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    const int chunk = (V + parts - 1) / parts;
    parts = (V + chunk - 1) / chunk;                       // (no part without values)
    float* pv = (float*)scratch;
    int32_t* pi = (int32_t*)scratch + (size_t)B * parts;
    hipLaunchKernelGGL(argmax_kernel, dim3(parts, B), dim3(SB), 0, (hipStream_t)stream, logits, out, pv, pi,
                       V, chunk);
    if (parts > 1)
        hipLaunchKernelGGL(argmax_parts_kernel, dim3(B), dim3(ILLM_WAVE), 0, (hipStream_t)stream, pv, pi,
                           out, parts);
    return illm_launch_status();
}

// ---------------------------------------------------------------- sampler
struct Keep {  // an id is kept iff key > t, or key == t and id <= cut
    uint32_t t;
    int cut;
};

__device__ __forceinline__ bool kept(const Keep& k, uint32_t key, int id) {
    return key > k.t || (key == k.t && id <= k.cut);
}

// id of the r-th (1-based) kept id whose key equals k.t, in ascending id order
__device__ int nth_equal_id(const float* s, int lo, int hi, const Keep& k, int r, int* red_i,
                            int* shared_out) {
    int mine = 0;
    for (int i = lo; i < hi; ++i) mine += (order_key(s[i]) == k.t && i <= k.cut) ? 1 : 0;
    int total;
    const int before = block_exclusive_scan<int>(mine, red_i, &total);
    __syncthreads();
    if (threadIdx.x == 0) *shared_out = k.cut;
    __syncthreads();
    if (r > before && r <= before + mine) {
        int c = before;
        for (int i = lo; i < hi; ++i)
            if (order_key(s[i]) == k.t && i <= k.cut && ++c == r) { *shared_out = i; break; }
    }
    __syncthreads();
    return *shared_out;
}

// Every pass over the row is coalesced (thread t takes ids t, t + SB, ...; eight loads asked for
// before the first is used), the probabilities exp(s - max) are computed once into the second
// half of the scratch, and only the steps that need the ids in order (the tie at a cut, the
// inverse CDF) walk a thread's own contiguous chunk.  A row of up to 32 ids a thread stays in
// registers for the two bisections (IN_REGS); a longer one finds the top_p threshold 8 bits a
// pass from the mass per digit instead of 32 walks.  Measured with top_p alone: 32,000 ids
// 557 -> 104 us (every pass in chunks and the exponentials recomputed in each, before), 128,256
// ids and 16 rows 2,190 -> 400 us.
constexpr int SAMPLE_REG_IDS = 32;      // ids a thread keeps in registers (IN_REGS: V <= 32 * SB)

template <bool IN_REGS>
__global__ void __launch_bounds__(SB)
sample_kernel(const float* __restrict__ logits, float* __restrict__ scratch,
              int32_t* __restrict__ out, int V, float temp, int top_k, float top_p,
              float repeat_penalty, const int32_t* __restrict__ last_tokens, int n_last,
              const uint64_t* __restrict__ seeds, const int32_t* __restrict__ counters) {
    __shared__ float red_f[SB / ILLM_WAVE];
    __shared__ int red_i[SB / ILLM_WAVE];
    __shared__ int last[256];
    __shared__ int sh_i;
    const int b = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)b * V;
    float* s = scratch + (size_t)b * V;                       // scaled, penalised scores
    float* pr = scratch + ((size_t)gridDim.x + b) * V;        // exp(s - max)
    const int chunk = (V + SB - 1) / SB;
    const int lo = min(V, tid * chunk), hi = min(V, lo + chunk);
    const int nl = last_tokens ? min(n_last, 256) : 0;
    if (tid < nl) last[tid] = last_tokens[(size_t)b * n_last + tid];
    __syncthreads();

    // 1. scaled and penalised scores; their max; the probabilities up to their sum
    const float inv_temp = 1.0f / temp;
    float mx = -INFINITY;
    each_strided8(row, V, tid, [&](int i, float l) {
        bool rep = false;
        for (int j = 0; j < nl; ++j) rep |= (last[j] == i);
        float v = l * inv_temp;
        if (rep) v = l < 0.f ? v * repeat_penalty : v / repeat_penalty;
        s[i] = v;
        mx = fmaxf(mx, v);
    });
    mx = block_max(mx, red_f);
    // (a thread reads back what it wrote itself: the same ids)
    each_strided8(s, V, tid, [&](int i, float v) { pr[i] = expf(v - mx); });
    __syncthreads();                                          // the chunked walks read others' values

    // The passes below walk the row's (id, key, probability): from registers, or from the
    // scratch again (a pass of 32,000 ids then waits for the cache four times over, 8 us).
    constexpr int RV = SAMPLE_REG_IDS;
    constexpr bool in_regs = IN_REGS;
    uint32_t rkey[RV];
    float rp[RV];
    if constexpr (in_regs) {
#pragma unroll
        for (int u = 0; u < RV; ++u) {
            const int i = tid + u * SB;
            rkey[u] = i < V ? order_key(s[i]) : 0u;
            rp[u] = i < V ? pr[i] : 0.f;
        }
    }
    auto walk = [&](auto f) __attribute__((always_inline)) {
        if constexpr (in_regs) {
#pragma unroll
            for (int u = 0; u < RV; ++u)
                if (tid + u * SB < V) f(tid + u * SB, rkey[u], rp[u]);
        } else {
            each_strided8(s, V, tid, [&](int i, float v) { f(i, order_key(v), pr[i]); });
        }
    };

    // 2. top_k: largest t with count(key >= t) >= k
    Keep keep = {0u, V};
    if (top_k > 0 && top_k < V) {
        uint32_t t = 0;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = t | (1u << bit);
            int c = 0;
            walk([&](int, uint32_t key, float) { c += key >= cand ? 1 : 0; });
            if (block_sum_t<int>(c, red_i) >= top_k) t = cand;
        }
        int c = 0;
        walk([&](int, uint32_t key, float) { c += key > t ? 1 : 0; });
        const int above = block_sum_t<int>(c, red_i);
        keep.t = t;
        keep.cut = nth_equal_id(s, lo, hi, keep, top_k - above, red_i, &sh_i);
    }

    // 3. top_p over the kept ids, in descending order of score
    if (top_p < 1.0f) {
        float z = 0.f;
        walk([&](int i, uint32_t key, float p) {
            if (kept(keep, key, i)) z += p;
        });
        z = block_sum_t<float>(z, red_f);
        const float need = top_p * z;
        uint32_t t = 0;  // every threshold up to keep.t holds the whole kept mass
        if constexpr (in_regs) {
            for (int bit = 31; bit >= 0; --bit) {
                const uint32_t cand = t | (1u << bit);
                float mass = 0.f;
                walk([&](int i, uint32_t key, float p) {
                    if (key >= cand && kept(keep, key, i)) mass += p;
                });
                if (block_sum_t<float>(mass, red_f) >= need) t = cand;
            }
        } else {
            // A longer row is not walked 32 times: the threshold's key comes 8 bits a pass from
            // the mass per digit, held as integers (p * 2^40, so that the order in which the
            // waves add them does not matter; 2^17 ids of at most 2^40 stay below 2^63).
            constexpr int NW = SB / ILLM_WAVE;
            __shared__ unsigned long long mhist[NW][256];
            __shared__ unsigned long long sh_total, sh_above;
            __shared__ int sh_digit;
            const int wave = tid / ILLM_WAVE;
            auto fixed = [](float p) { return (unsigned long long)(p * 1099511627776.0f); };
            unsigned long long mine_fx = 0;
            walk([&](int i, uint32_t key, float p) {
                if (kept(keep, key, i)) mine_fx += fixed(p);
            });
            if (tid == 0) sh_total = 0;
            __syncthreads();
            atomicAdd(&sh_total, mine_fx);
            __syncthreads();
            unsigned long long need_fx = (unsigned long long)((double)top_p * (double)sh_total);
            need_fx = need_fx > 0 ? need_fx : 1;
            unsigned long long above_fx = 0;         // mass of the keys above the prefix so far
            for (int pass = 0; pass < 4; ++pass) {
                const int shift = 24 - 8 * pass;
                const uint32_t hi_mask = pass ? (0xffffffffu << (shift + 8)) : 0u;
                for (int i = tid; i < NW * 256; i += SB) (&mhist[0][0])[i] = 0;
                __syncthreads();
                walk([&](int i, uint32_t key, float p) {
                    if ((key & hi_mask) == t && kept(keep, key, i))
                        atomicAdd(&mhist[wave][(key >> shift) & 255u], fixed(p));
                });
                __syncthreads();
                if (tid < 256) {
                    unsigned long long m = 0;
                    for (int w = 0; w < NW; ++w) m += mhist[w][tid];
                    mhist[0][tid] = m;
                }
                if (tid == 0) sh_digit = 0;
                __syncthreads();
                if (tid < 256) {
                    // the largest digit at which the mass from the top reaches what is needed
                    unsigned long long over = above_fx;
                    for (int d = tid + 1; d < 256; ++d) over += mhist[0][d];
                    if (over < need_fx && over + mhist[0][tid] >= need_fx) {
                        sh_digit = tid;
                        sh_above = over;
                    }
                }
                __syncthreads();
                t |= (uint32_t)sh_digit << shift;
                above_fx = sh_above;
                __syncthreads();
            }
        }
        // t is now the largest threshold whose kept mass still reaches top_p
        float mass = 0.f, eq_p = 0.f;
        int eq = 0;
        walk([&](int i, uint32_t key, float p) {
            if (!kept(keep, key, i)) return;
            if (key > t) mass += p;
            else if (key == t) { eq += 1; eq_p = p; }
        });
        const float above = block_sum_t<float>(mass, red_f);
        const int n_eq = block_sum_t<int>(eq, red_i);
        const float one = block_max(eq_p, red_f);
        int m = one > 0.f ? (int)ceilf((need - above) / one) : n_eq;
        m = max(1, min(m, n_eq));
        Keep k2 = {t, keep.t == t ? keep.cut : V};
        k2.cut = nth_equal_id(s, lo, hi, k2, m, red_i, &sh_i);
        keep = k2;
    }

    // 4. inverse CDF over the kept ids in ascending id order
    float mine = 0.f;
    each_in_order8(s, lo, hi, [&](int i, float v) {
        if (kept(keep, order_key(v), i)) mine += pr[i];
    });
    float total;
    const float before = block_exclusive_scan<float>(mine, red_f, &total);
    const float u = uniform_from(seeds[b], counters[b]);
    const float target = u * total;
    __syncthreads();
    if (tid == 0) sh_i = -1;
    __syncthreads();
    if (mine > 0.f && target >= before && target < before + mine) {
        float c = before;
        int pick = -1;
        for (int i = lo; i < hi; ++i) {
            if (!kept(keep, order_key(s[i]), i)) continue;
            pick = i;
            c += pr[i];
            if (target < c) break;
        }
        atomicMax(&sh_i, pick);
    }
    __syncthreads();
    if (sh_i < 0) {
        // rounding put the target past the last kept id: take that id
        int lastk = -1;
        for (int i = lo; i < hi; ++i)
            if (kept(keep, order_key(s[i]), i)) lastk = i;
        atomicMax(&sh_i, lastk);
        __syncthreads();
    }
    if (tid == 0) out[b] = sh_i < 0 ? 0 : sh_i;
}

// ---------------------------------------------------------------- sampler, small top_k
// The same choice for 0 < top_k <= SB (the reference's default is 40) in a few passes over the
// row instead of two bisections of 32 passes each: the top_k-th largest key by radix selection
// (4 passes of 8 bits, histograms per wave in LDS), the kept ids gathered in id order into LDS,
// top_p decided per kept id from the mass that lies before it in descending order, the draw by
// inverse CDF over what is left.  Ties at the k-th value and at the top_p cut go to the lower ids.
// PART: the block takes one of gridDim.x stretches of the row (grid (parts, B)) and leaves its
// top_k ids (global numbers, ascending) and their scores behind the rows' scores in `scratch`
// for `sample_topk_merge_kernel`: a row is then the work of several compute units instead of
// one, whose instruction issue bounds a block (top_k <= TOPK_PARTS_MAX_K, long rows).
#define TOPK_PARTS_MAX_K 64
#define TOPK_MAX_PARTS (SB / TOPK_PARTS_MAX_K)

// What a row's parts leave for the merge, in the second plane of `scratch` (floats; B rows of V
// before it): per part its count, then TOPK_PARTS_MAX_K scores, then as many ids.
__device__ __forceinline__ float* topk_part_slot(float* scratch, int B, int V, int b, int part) {
    return scratch + ((size_t)B + b) * V + (size_t)part * (1 + 2 * TOPK_PARTS_MAX_K);
}

// top_p over the n_kept candidates in cand_id / cand_s (ascending ids, one a thread), then the
// draw: steps 4 and 5 of the kernel below.
__device__ __forceinline__ void topk_finish(const int* cand_id, const float* cand_s, int n_kept,
                                            float top_p, uint64_t seed, int counter, float* red_f,
                                            int* sh_i, int32_t* out_b) {
    __shared__ float cand_p[SB];                        // exp(score - max), computed once
    const int tid = threadIdx.x;
    const bool have = tid < n_kept;
    const float my_s = have ? cand_s[tid] : -INFINITY;
    const float mx = block_max(my_s, red_f);            // the largest score is among the kept
    // 4. top_p: an id stays if the mass before it in descending order (ties: lower id first)
    // does not yet reach top_p of the whole kept mass
    const float my_p = have ? expf(my_s - mx) : 0.f;
    bool stay = have;
    if (top_p < 1.0f) {
        cand_p[tid] = my_p;
        const float z = block_sum_t<float>(my_p, red_f);        // (its barriers publish cand_p)
        const float need = top_p * z;
        if (have) {
            float before = 0.f;
            const uint32_t my_key = order_key(my_s);
            for (int j = 0; j < n_kept; ++j) {
                const uint32_t kj = order_key(cand_s[j]);
                if (kj > my_key || (kj == my_key && j < tid)) before += cand_p[j];
            }
            stay = before < need;
        }
    }
    // 5. inverse CDF over what stays, in ascending id order (the order of the list)
    const float mine = stay ? my_p : 0.f;
    float total;
    const float before = block_exclusive_scan<float>(mine, red_f, &total);
    const float target = uniform_from(seed, counter) * total;
    __syncthreads();
    if (tid == 0) *sh_i = -1;
    __syncthreads();
    if (mine > 0.f && target >= before && target < before + mine) atomicMax(sh_i, cand_id[tid]);
    __syncthreads();
    if (*sh_i < 0) {
        // rounding put the target past the last id that stays: take that id
        if (stay) atomicMax(sh_i, cand_id[tid]);
        __syncthreads();
    }
    if (tid == 0) *out_b = *sh_i < 0 ? 0 : *sh_i;
}

// NR > 0: the block's ids fit NR registers a thread (a wave's stretch of the row in 64 * NR ids) and
// every pass after the first reads them from there instead of from the scratch.
template <bool PART, int NR>
__global__ void __launch_bounds__(SB)
sample_topk_kernel(const float* __restrict__ logits, float* __restrict__ scratch,
                   int32_t* __restrict__ out, int Vrow, float temp, int top_k, float top_p,
                   float repeat_penalty, const int32_t* __restrict__ last_tokens, int n_last,
                   const uint64_t* __restrict__ seeds, const int32_t* __restrict__ counters) {
    constexpr int NW = SB / ILLM_WAVE;
    __shared__ float red_f[NW];
    __shared__ int red_i[NW];
    __shared__ int last[256];
    __shared__ int hist[NW][256];
    __shared__ int sh_d, sh_above, sh_i;
    __shared__ int cand_id[SB];
    __shared__ float cand_s[SB];
    const int b = PART ? blockIdx.y : blockIdx.x, tid = threadIdx.x, wave = tid / ILLM_WAVE;
    // the ids this block looks at: [first, first + V) of the row's Vrow
    const int stretch_ids = PART ? ((Vrow + (int)gridDim.x - 1) / (int)gridDim.x + 3) / 4 * 4 : Vrow;
    const int first = PART ? min(Vrow, (int)blockIdx.x * stretch_ids) : 0;
    const int V = PART ? min(stretch_ids, Vrow - first) : Vrow;
    const float* row = logits + (size_t)b * Vrow + first;
    float* s = scratch + (size_t)b * Vrow + first;
    const int nl = last_tokens ? min(n_last, 256) : 0;
    if (tid < nl) last[tid] = last_tokens[(size_t)b * n_last + tid];
    if (PART && V <= 0) {                               // (no ids left for this part)
        if (tid == 0) *(int*)topk_part_slot(scratch, gridDim.y, Vrow, b, blockIdx.x) = 0;
        return;
    }
    top_k = min(top_k, V);

    // 1. scaled scores; then the penalty, once for every id of the window
    const float inv_temp = 1.0f / temp;
    each_strided8(row, V, tid, [&](int i, float v) { s[i] = v * inv_temp; });
    __syncthreads();
    if (tid < nl) {
        const int id = last[tid] - first;
        bool once = last[tid] >= 0 && id >= 0 && id < V;     // in this block's ids, and not named before
        for (int j = 0; j < tid; ++j) once = once && last[j] != last[tid];
        if (once) {
            const float l = row[id], v = l * inv_temp;
            s[id] = l < 0.f ? v * repeat_penalty : v / repeat_penalty;
        }
    }
    __syncthreads();

    // A wave walks its own stretch of the row, 64 consecutive ids an instruction (a thread walking
    // a stretch of its own would touch 64 cache lines an instruction); within an instruction the
    // lanes are in id order, so the gather below gets counts and places from ballots.
    const int lane = tid & (ILLM_WAVE - 1);
    const int stretch = ((V + NW - 1) / NW + ILLM_WAVE - 1) / ILLM_WAVE * ILLM_WAVE;
    const int lo = min(V, wave * stretch), hi = min(V, lo + stretch);
    float rv[NR > 0 ? NR : 1];
    if constexpr (NR > 0) {
#pragma unroll
        for (int u = 0; u < NR; ++u) {
            const int i = lo + u * ILLM_WAVE + lane;
            rv[u] = i < hi ? s[i] : 0.f;
        }
    }
    auto walk = [&](auto f) __attribute__((always_inline)) {
        if constexpr (NR > 0) {
#pragma unroll
            for (int u = 0; u < NR; ++u) {
                const int i = lo + u * ILLM_WAVE + lane;
                f(i, rv[u], i < hi);
            }
        } else {
            for (int base = lo; base < hi; base += 8 * ILLM_WAVE) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int i = base + u * ILLM_WAVE + lane;
                    v[u] = i < hi ? s[i] : 0.f;
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int i = base + u * ILLM_WAVE + lane;
                    f(i, v[u], i < hi);
                }
            }
        }
    };

    // 2. the key of the top_k-th largest score, 8 bits a pass
    uint32_t prefix = 0;
    int krem = top_k;
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        const uint32_t hi_mask = pass ? (0xffffffffu << (shift + 8)) : 0u;
        for (int i = tid; i < NW * 256; i += SB) (&hist[0][0])[i] = 0;
        __syncthreads();
        walk([&](int, float v, bool in) {
            const uint32_t key = order_key(v);
            if (in && (key & hi_mask) == prefix) atomicAdd(&hist[wave][(key >> shift) & 255u], 1);
        });
        __syncthreads();
        // how many keys have a larger digit: a suffix sum over the 256 digits, within each of
        // the first four waves by shuffles, across them through LDS
        int cnt = 0, suffix = 0;
        if (tid < 256) {
            for (int w = 0; w < NW; ++w) cnt += hist[w][tid];
            suffix = cnt;
            const int ln = tid & (ILLM_WAVE - 1);
#pragma unroll
            for (int o = 1; o < ILLM_WAVE; o <<= 1) {
                const int t = __shfl_down(suffix, o, ILLM_WAVE);
                if (ln + o < ILLM_WAVE) suffix += t;
            }
            if (ln == 0) red_i[wave] = suffix;
        }
        __syncthreads();
        if (tid < 256) {
            int above = suffix - cnt;
            for (int w = wave + 1; w < 4; ++w) above += red_i[w];
            if (above < krem && above + cnt >= krem) { sh_d = tid; sh_above = above; }
        }
        __syncthreads();
        // (sh_d and sh_above are written again only after the next pass's barriers)
        prefix |= (uint32_t)sh_d << shift;
        krem -= sh_above;
    }
    // kept: key > prefix, and the first krem ids (ascending) with key == prefix

    // 3. the kept ids and scores in id order into LDS: counts and places from ballots
    const unsigned long long below = (1ull << lane) - 1ull;
    int n_eq = 0, n_gt = 0;                             // of the wave's stretch (the same in all its lanes)
    walk([&](int, float v, bool in) {
        const uint32_t key = order_key(v);
        n_gt += __popcll(__ballot(in && key > prefix));
        n_eq += __popcll(__ballot(in && key == prefix));
    });
    __syncthreads();
    if (lane == 0) { red_i[wave] = n_eq; hist[0][wave] = n_gt; }
    __syncthreads();
    int eq_before = 0;
    for (int w = 0; w < wave; ++w) eq_before += red_i[w];
    int eq_left = max(0, min(n_eq, krem - eq_before));  // ids with the k-th key this wave still takes
    int at = 0, n_kept = 0;                             // where the wave's first kept id goes; all kept (== top_k)
    for (int w = 0, eb = 0; w < NW; ++w) {
        const int took = hist[0][w] + max(0, min(red_i[w], krem - eb));
        if (w < wave) at += took;
        n_kept += took;
        eb += red_i[w];
    }
    __syncthreads();
    walk([&](int i, float v, bool in) {
        const uint32_t key = order_key(v);
        const bool eq = in && key == prefix;
        const unsigned long long eq_mask = __ballot(eq);
        const bool take = (in && key > prefix) || (eq && __popcll(eq_mask & below) < eq_left);
        const unsigned long long take_mask = __ballot(take);
        const int to = at + __popcll(take_mask & below);
        if (take && to < SB) { cand_id[to] = i; cand_s[to] = v; }
        at += __popcll(take_mask);
        eq_left -= min(eq_left, __popcll(eq_mask));
    });
    __syncthreads();

    if (PART) {
        // the part's kept ids (global numbers) and scores for the merge
        float* slot = topk_part_slot(scratch, gridDim.y, Vrow, b, blockIdx.x);
        if (tid == 0) *(int*)slot = n_kept;
        if (tid < n_kept) {
            slot[1 + tid] = cand_s[tid];
            ((int*)slot)[1 + TOPK_PARTS_MAX_K + tid] = first + cand_id[tid];
        }
        return;
    }
    topk_finish(cand_id, cand_s, n_kept, top_p, seeds[b], counters[b], red_f, &sh_i, out + b);
}

// The parts' kept ids of a row (at most SB together, in ascending id order part after part):
// the top_k of them by score (ties: the lower id), then top_p and the draw as above.
__global__ void __launch_bounds__(SB)
sample_topk_merge_kernel(float* __restrict__ scratch, int32_t* __restrict__ out, int V, int parts,
                         int top_k, float top_p, const uint64_t* __restrict__ seeds,
                         const int32_t* __restrict__ counters) {
    constexpr int NW = SB / ILLM_WAVE;
    __shared__ float red_f[NW];
    __shared__ int red_i[NW];
    __shared__ int sh_i;
    __shared__ int cand_id[SB];
    __shared__ float cand_s[SB];
    __shared__ int part_at[TOPK_MAX_PARTS + 1];
    const int b = blockIdx.x, tid = threadIdx.x;
    if (tid == 0) {
        int at = 0;
        for (int p = 0; p < parts; ++p) {
            part_at[p] = at;
            at += *(const int*)topk_part_slot(scratch, gridDim.x, V, b, p);
        }
        part_at[parts] = at;
    }
    __syncthreads();
    const int n_all = part_at[parts];
    {
        const int p = tid / TOPK_PARTS_MAX_K, j = tid % TOPK_PARTS_MAX_K;
        if (p < parts && j < part_at[p + 1] - part_at[p]) {
            const float* slot = topk_part_slot(scratch, gridDim.x, V, b, p);
            cand_s[part_at[p] + j] = slot[1 + j];
            cand_id[part_at[p] + j] = ((const int*)slot)[1 + TOPK_PARTS_MAX_K + j];
        }
    }
    __syncthreads();
    // a candidate's place in descending order of score, the lower id first among equals
    const bool have = tid < n_all;
    const float my_s = have ? cand_s[tid] : 0.f;
    const int my_id = have ? cand_id[tid] : 0;
    int rank = 0;
    if (have) {
        const uint32_t my_key = order_key(my_s);
        for (int j = 0; j < n_all; ++j) {
            const uint32_t kj = order_key(cand_s[j]);
            rank += (kj > my_key || (kj == my_key && j < tid)) ? 1 : 0;
        }
    }
    const bool keep = have && rank < top_k;
    int n_kept;
    const int to = block_exclusive_scan<int>(keep ? 1 : 0, red_i, &n_kept);
    __syncthreads();
    if (keep) { cand_id[to] = my_id; cand_s[to] = my_s; }
    __syncthreads();
    topk_finish(cand_id, cand_s, n_kept, top_p, seeds[b], counters[b], red_f, &sh_i, out + b);
}

// ---------------------------------------------------------------- sampler, long rows without top_k
// The same choice as `sample_kernel` makes for top_k == 0 (temperature, repeat penalty, top_p),
// for rows of 16,384 ids and more, by several blocks a row: one block walks 128,256 ids in 30 to
// 50 us a pass and needs three passes for temperature alone and nine with top_p, bound by one
// compute unit's instruction issue.  Here a row is cut into up to 16 parts with blocks of their
// own and every pass is a kernel; what a pass hands to the next lies in the row's `SpRow`.
// Masses are integers (p * 2^40), so no sum depends on the order of its terms:
//   scale   scaled and penalised scores; the parts' largest
//   mass    p = exp(s - max); the parts' masses; (top_p) the mass per top digit of the key
//   digit   x3 (top_p) every block finds the threshold's next digit from the last pass's masses
//           per digit, then adds up the masses per next digit among the keys with that prefix
//   edge    (top_p) the last digit; per part the mass above the threshold key and the ids at it
//   draw    one block a row: how many ids at the threshold key stay (the lowest ids), the part
//           that holds the target of the draw, and the id in it
#define SP_MAX_PARTS 16
typedef unsigned long long sp_u64;

struct SpRow {
    float pmax[SP_MAX_PARTS];
    sp_u64 ptotal[SP_MAX_PARTS];
    sp_u64 mass_gt[SP_MAX_PARTS];
    sp_u64 one_fx[SP_MAX_PARTS];              // the mass of an id at the threshold key (0: none in the part)
    int n_eq[SP_MAX_PARTS];
    uint32_t t[5];                            // the threshold's key after 0 .. 4 digits
    uint32_t pad;
    sp_u64 above[5];                          // mass of the keys above that prefix
    sp_u64 hist[2][SP_MAX_PARTS][256];        // mass per digit, two passes alternating
};
static_assert(sizeof(SpRow) <= ILLM_SAMPLE_LONG_ROW_BYTES, "SpRow must fit what callers allocate");

__device__ __forceinline__ sp_u64 sp_fixed(float p) { return (sp_u64)(p * 1099511627776.0f); }

struct SpPart {
    int first, n;                             // the ids [first, first + n) of the row
};
__device__ __forceinline__ SpPart sp_part(int V, int parts, int p) {
    const int stretch = ((V + parts - 1) / parts + 3) / 4 * 4;
    const int first = min(V, p * stretch);
    return {first, min(stretch, V - first)};
}

__global__ void __launch_bounds__(SB)
sp_scale_kernel(const float* __restrict__ logits, float* __restrict__ scratch, SpRow* __restrict__ rows,
                int V, float temp, float repeat_penalty, const int32_t* __restrict__ last_tokens,
                int n_last) {
    __shared__ float red_f[SB / ILLM_WAVE];
    __shared__ int last[256];
    const int p = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const SpPart part = sp_part(V, gridDim.x, p);
    const float* row = logits + (size_t)b * V + part.first;
    float* s = scratch + (size_t)b * V + part.first;
    const int nl = last_tokens ? min(n_last, 256) : 0;
    if (tid < nl) last[tid] = last_tokens[(size_t)b * n_last + tid];
    const float inv_temp = 1.0f / temp;
    each_strided8(row, part.n, tid, [&](int i, float v) { s[i] = v * inv_temp; });
    __syncthreads();
    // the penalty, once for every id of the window that lies in this part
    if (tid < nl) {
        const int id = last[tid] - part.first;
        bool once = last[tid] >= 0 && id >= 0 && id < part.n;
        for (int j = 0; j < tid; ++j) once = once && last[j] != last[tid];
        if (once) {
            const float l = row[id], v = l * inv_temp;
            s[id] = l < 0.f ? v * repeat_penalty : v / repeat_penalty;
        }
    }
    __syncthreads();
    float mx = -INFINITY;
    each_strided8(s, part.n, tid, [&](int, float v) { mx = fmaxf(mx, v); });
    mx = block_max(mx, red_f);
    if (tid == 0) rows[b].pmax[p] = mx;
}

// The mass per digit `(key >> shift) & 255` of the part's ids whose key has the prefix `t` above
// those bits (hi_mask == 0: all ids), into out[256]; by the waves into LDS, then added up.
template <typename F>
__device__ __forceinline__ void sp_histogram(sp_u64 (*mhist)[256], sp_u64* out, F walk, uint32_t t,
                                             uint32_t hi_mask, int shift) {
    const int tid = threadIdx.x, wave = tid / ILLM_WAVE;
    for (int i = tid; i < (SB / ILLM_WAVE) * 256; i += SB) (&mhist[0][0])[i] = 0;
    __syncthreads();
    walk([&](uint32_t key, sp_u64 fx) {
        if ((key & hi_mask) == t) atomicAdd(&mhist[wave][(key >> shift) & 255u], fx);
    });
    __syncthreads();
    if (tid < 256) {
        sp_u64 m = 0;
        for (int w = 0; w < SB / ILLM_WAVE; ++w) m += mhist[w][tid];
        out[tid] = m;
    }
}

__global__ void __launch_bounds__(SB)
sp_mass_kernel(float* __restrict__ scratch, SpRow* __restrict__ rows, int V, int n_rows, float top_p) {
    __shared__ sp_u64 mhist[SB / ILLM_WAVE][256];
    __shared__ sp_u64 sh_total;
    const int p = blockIdx.x, b = blockIdx.y, tid = threadIdx.x, parts = gridDim.x;
    const SpPart part = sp_part(V, parts, p);
    SpRow& R = rows[b];
    float mx = R.pmax[0];
    for (int q = 1; q < parts; ++q) mx = fmaxf(mx, R.pmax[q]);
    const float* s = scratch + (size_t)b * V + part.first;
    float* pr = scratch + ((size_t)n_rows + b) * V + part.first;
    sp_u64 mine = 0;
    each_strided8(s, part.n, tid, [&](int i, float v) {
        const float e = expf(v - mx);
        pr[i] = e;
        mine += sp_fixed(e);
    });
    if (tid == 0) sh_total = 0;
    __syncthreads();
    atomicAdd(&sh_total, mine);
    __syncthreads();
    if (tid == 0) {
        R.ptotal[p] = sh_total;
        if (p == 0) { R.t[0] = 0u; R.above[0] = 0; }
    }
    if (top_p < 1.0f) {
        // (a thread reads back the probabilities that it wrote itself)
        auto walk = [&](auto f) __attribute__((always_inline)) {
            each_strided8(s, part.n, tid, [&](int i, float v) { f(order_key(v), sp_fixed(pr[i])); });
        };
        sp_histogram(mhist, R.hist[0][p], walk, 0u, 0u, 24);
    }
}

// The threshold after `level` + 1 digits, from the masses per digit that pass `level` left: the
// largest digit at which the mass from the top reaches what top_p needs.  Every block of the next
// pass finds it for itself; the first of a row writes it down for the passes after.
__device__ __forceinline__ void sp_decide(SpRow& R, int parts, int level, float top_p, sp_u64* digit_mass,
                                          uint32_t* t_out, sp_u64* above_out, bool write) {
    __shared__ int sh_digit;
    __shared__ sp_u64 sh_above;
    const int tid = threadIdx.x, shift = 24 - 8 * level;
    sp_u64 total = 0;
    for (int q = 0; q < parts; ++q) total += R.ptotal[q];
    sp_u64 need = (sp_u64)((double)top_p * (double)total);
    need = need > 0 ? need : 1;
    if (tid < 256) {
        sp_u64 m = 0;
        for (int q = 0; q < parts; ++q) m += R.hist[level & 1][q][tid];
        digit_mass[tid] = m;
    }
    if (tid == 0) { sh_digit = 0; sh_above = R.above[level]; }
    __syncthreads();
    if (tid < 256) {
        sp_u64 over = R.above[level];
        for (int d = tid + 1; d < 256; ++d) over += digit_mass[d];
        if (over < need && over + digit_mass[tid] >= need) { sh_digit = tid; sh_above = over; }
    }
    __syncthreads();
    *t_out = R.t[level] | ((uint32_t)sh_digit << shift);
    *above_out = sh_above;
    if (write && tid == 0) { R.t[level + 1] = *t_out; R.above[level + 1] = sh_above; }
    __syncthreads();
}

// level 1 .. 3: decide digit `level - 1`, then the masses per digit `level` under the new prefix
__global__ void __launch_bounds__(SB)
sp_digit_kernel(const float* __restrict__ scratch, SpRow* __restrict__ rows, int V, int n_rows,
                float top_p, int level) {
    __shared__ sp_u64 mhist[SB / ILLM_WAVE][256];
    __shared__ sp_u64 digit_mass[256];
    const int p = blockIdx.x, b = blockIdx.y, tid = threadIdx.x, parts = gridDim.x;
    const SpPart part = sp_part(V, parts, p);
    SpRow& R = rows[b];
    uint32_t t;
    sp_u64 above;
    sp_decide(R, parts, level - 1, top_p, digit_mass, &t, &above, p == 0);
    const float* s = scratch + (size_t)b * V + part.first;
    const float* pr = scratch + ((size_t)n_rows + b) * V + part.first;
    auto walk = [&](auto f) __attribute__((always_inline)) {
        each_strided8(s, part.n, tid, [&](int i, float v) { f(order_key(v), sp_fixed(pr[i])); });
    };
    const int shift = 24 - 8 * level;
    sp_histogram(mhist, R.hist[level & 1][p], walk, t, 0xffffffffu << (shift + 8), shift);
}

// the last digit; the part's mass above the threshold key, its ids at that key and their mass
__global__ void __launch_bounds__(SB)
sp_edge_kernel(const float* __restrict__ scratch, SpRow* __restrict__ rows, int V, int n_rows,
               float top_p) {
    __shared__ sp_u64 digit_mass[256];
    __shared__ sp_u64 sh_gt, sh_one;
    __shared__ int sh_eq;
    const int p = blockIdx.x, b = blockIdx.y, tid = threadIdx.x, parts = gridDim.x;
    const SpPart part = sp_part(V, parts, p);
    SpRow& R = rows[b];
    uint32_t t;
    sp_u64 above;
    sp_decide(R, parts, 3, top_p, digit_mass, &t, &above, p == 0);
    const float* s = scratch + (size_t)b * V + part.first;
    const float* pr = scratch + ((size_t)n_rows + b) * V + part.first;
    sp_u64 gt = 0, one = 0;
    int eq = 0;
    each_strided8(s, part.n, tid, [&](int i, float v) {
        const uint32_t key = order_key(v);
        if (key > t) gt += sp_fixed(pr[i]);
        else if (key == t) { eq += 1; one = sp_fixed(pr[i]); }
    });
    if (tid == 0) { sh_gt = 0; sh_one = 0; sh_eq = 0; }
    __syncthreads();
    atomicAdd(&sh_gt, gt);
    atomicAdd(&sh_eq, eq);
    if (eq) atomicMax(&sh_one, one);
    __syncthreads();
    if (tid == 0) { R.mass_gt[p] = sh_gt; R.n_eq[p] = sh_eq; R.one_fx[p] = sh_one; }
}

__global__ void __launch_bounds__(SB)
sp_draw_kernel(const float* __restrict__ scratch, const SpRow* __restrict__ rows, int32_t* __restrict__ out,
               int V, int n_rows, int parts, float top_p, const uint64_t* __restrict__ seeds,
               const int32_t* __restrict__ counters) {
    __shared__ sp_u64 red_u[SB / ILLM_WAVE];
    __shared__ int red_i[SB / ILLM_WAVE];
    __shared__ int sh_i;
    const int b = blockIdx.x, tid = threadIdx.x;
    const SpRow& R = rows[b];
    const float* s = scratch + (size_t)b * V;
    const float* pr = scratch + ((size_t)n_rows + b) * V;
    const bool all = !(top_p < 1.0f);                    // every id stays
    // (every thread works these few numbers out for itself)
    sp_u64 total = 0;
    for (int q = 0; q < parts; ++q) total += R.ptotal[q];
    uint32_t t = 0;
    int cut = V, part_of_cut = parts, eq_in_cut_part = 0;
    sp_u64 one = 0, kept_total = total;
    if (!all) {
        sp_u64 need = (sp_u64)((double)top_p * (double)total);
        need = need > 0 ? need : 1;
        t = R.t[4];
        const sp_u64 above = R.above[4];
        int n_eq = 0;
        for (int q = 0; q < parts; ++q) { n_eq += R.n_eq[q]; one = one ? one : R.one_fx[q]; }
        // ids at the threshold key that stay: as many as still needed to reach top_p, the lowest ids
        long long m = one > 0 ? (long long)((need - above + one - 1) / one) : n_eq;
        m = m < 1 ? 1 : (m > n_eq ? n_eq : m);
        kept_total = above + (sp_u64)m * one;
        int before = 0;
        for (int q = 0; q < parts; ++q) {
            if (m > before && m <= before + R.n_eq[q]) { part_of_cut = q; eq_in_cut_part = (int)m - before; }
            before += R.n_eq[q];
        }
        // the id of that last one: the eq_in_cut_part-th id at the key in its part
        const SpPart part = sp_part(V, parts, part_of_cut);
        const int chunk = (part.n + SB - 1) / SB;
        const int lo = part.first + min(part.n, tid * chunk), hi = min(part.first + part.n, lo + chunk);
        int mine = 0;
        for (int i = lo; i < hi; ++i) mine += order_key(s[i]) == t ? 1 : 0;
        int all_eq;
        const int bef = block_exclusive_scan<int>(mine, red_i, &all_eq);
        __syncthreads();
        if (tid == 0) sh_i = part.first + part.n - 1;
        __syncthreads();
        if (eq_in_cut_part > bef && eq_in_cut_part <= bef + mine) {
            int c = bef;
            for (int i = lo; i < hi; ++i)
                if (order_key(s[i]) == t && ++c == eq_in_cut_part) { sh_i = i; break; }
        }
        __syncthreads();
        cut = sh_i;
        __syncthreads();
    }
    auto stays = [&](int i) {
        if (all) return true;
        const uint32_t key = order_key(s[i]);
        return key > t || (key == t && i <= cut);
    };
    // the part that holds the target, by the parts' kept masses in id order
    const float u = uniform_from(seeds[b], counters[b]);
    sp_u64 target = (sp_u64)((double)u * (double)kept_total);
    target = target < kept_total ? target : (kept_total ? kept_total - 1 : 0);
    int pt = parts - 1;
    sp_u64 before_part = 0;
    {
        sp_u64 acc = 0;
        bool found = false;
        for (int q = 0; q < parts; ++q) {
            const sp_u64 km = all ? R.ptotal[q]
                                  : R.mass_gt[q] + one * (sp_u64)(q < part_of_cut ? R.n_eq[q]
                                                                  : (q == part_of_cut ? eq_in_cut_part : 0));
            if (!found && target < acc + km) { pt = q; before_part = acc; found = true; }
            acc += km;
        }
    }
    const sp_u64 rem = target - before_part;
    const SpPart part = sp_part(V, parts, pt);
    const int chunk = (part.n + SB - 1) / SB;
    const int lo = part.first + min(part.n, tid * chunk), hi = min(part.first + part.n, lo + chunk);
    sp_u64 mine = 0;
    for (int i = lo; i < hi; ++i)
        if (stays(i)) mine += sp_fixed(pr[i]);
    sp_u64 part_total;
    const sp_u64 bef = block_exclusive_scan<sp_u64>(mine, red_u, &part_total);
    __syncthreads();
    if (tid == 0) sh_i = -1;
    __syncthreads();
    if (mine > 0 && rem >= bef && rem < bef + mine) {
        sp_u64 c = bef;
        int pick = -1;
        for (int i = lo; i < hi; ++i) {
            if (!stays(i)) continue;
            pick = i;
            c += sp_fixed(pr[i]);
            if (rem < c) break;
        }
        atomicMax(&sh_i, pick);
    }
    __syncthreads();
    if (sh_i < 0) {
        // (the target lies past the part's last kept id only if the sums disagree: take that id)
        int lastk = -1;
        for (int i = lo; i < hi; ++i)
            if (stays(i) && sp_fixed(pr[i]) > 0) lastk = i;
        atomicMax(&sh_i, lastk);
        __syncthreads();
    }
    if (tid == 0) out[b] = sh_i < 0 ? 0 : sh_i;
}

extern "C" int illm_sample_long_row_bytes(void) { return ILLM_SAMPLE_LONG_ROW_BYTES; }

extern "C" int illm_sample_long(const float* logits, float* scratch, void* rows, int32_t* out, int B,
                                int V, float temp, float top_p, float repeat_penalty,
                                const int32_t* last_tokens, int n_last, const uint64_t* seeds,
                                const int32_t* counters, void* stream) {
    if (B < 0 || B > 65535 || V < 16384 || !(temp > 0.f) || !(top_p > 0.f) || !(repeat_penalty > 0.f) ||
        n_last < 0 || n_last > 256 || !seeds || !counters || !scratch || !rows)
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    // parts of 4,096 ids or more, about 512 blocks in all
    int parts = V / 4096;
    parts = parts > SP_MAX_PARTS ? SP_MAX_PARTS : parts;
    while (parts > 2 && parts * B > 512) parts /= 2;
    hipStream_t st = (hipStream_t)stream;
    SpRow* R = (SpRow*)rows;
    const dim3 grid(parts, B);
    hipLaunchKernelGGL(sp_scale_kernel, grid, dim3(SB), 0, st, logits, scratch, R, V, temp,
                       repeat_penalty, last_tokens, n_last);
    hipLaunchKernelGGL(sp_mass_kernel, grid, dim3(SB), 0, st, scratch, R, V, B, top_p);
    if (top_p < 1.0f) {
        for (int level = 1; level <= 3; ++level)
            hipLaunchKernelGGL(sp_digit_kernel, grid, dim3(SB), 0, st, (const float*)scratch, R, V, B,
                               top_p, level);
        hipLaunchKernelGGL(sp_edge_kernel, grid, dim3(SB), 0, st, (const float*)scratch, R, V, B, top_p);
    }
    hipLaunchKernelGGL(sp_draw_kernel, dim3(B), dim3(SB), 0, st, (const float*)scratch, (const SpRow*)R,
                       out, V, B, parts, top_p, seeds, counters);
    return illm_launch_status();
}

extern "C" int illm_sample(const float* logits, float* scratch, int32_t* out, int B, int V,
                           float temp, int top_k, float top_p, float repeat_penalty,
                           const int32_t* last_tokens, int n_last, const uint64_t* seeds,
                           const int32_t* counters, void* stream) {
    if (B < 0 || V <= 0 || !(temp > 0.f) || !(top_p > 0.f) || !(repeat_penalty > 0.f) ||
        n_last < 0 || n_last > 256 || !seeds || !counters || !scratch)
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    if (top_k > 0 && top_k <= TOPK_PARTS_MAX_K && V >= 65536 && B <= 65535) {
        // a row in parts of 4,096 ids or more, about 512 blocks in all, then the merge (at 32,000
        // ids the second launch costs what the parts save: 60 us against 52)
        int parts = V / 4096;
        parts = parts > TOPK_MAX_PARTS ? TOPK_MAX_PARTS : parts;
        while (parts > 2 && parts * B > 512) parts /= 2;
        // (a part's ids: as sample_topk_kernel cuts the row)
        const int part_ids = ((V + parts - 1) / parts + 3) / 4 * 4;
        if (part_ids <= 8 * ILLM_WAVE * (SB / ILLM_WAVE))
            hipLaunchKernelGGL((sample_topk_kernel<true, 8>), dim3(parts, B), dim3(SB), 0, (hipStream_t)stream,
                               logits, scratch, out, V, temp, top_k, top_p, repeat_penalty, last_tokens,
                               n_last, seeds, counters);
        else
            hipLaunchKernelGGL((sample_topk_kernel<true, 0>), dim3(parts, B), dim3(SB), 0, (hipStream_t)stream,
                               logits, scratch, out, V, temp, top_k, top_p, repeat_penalty, last_tokens,
                               n_last, seeds, counters);
        hipLaunchKernelGGL(sample_topk_merge_kernel, dim3(B), dim3(SB), 0, (hipStream_t)stream, scratch,
                           out, V, parts, top_k, top_p, seeds, counters);
    } else if (top_k > 0 && top_k <= SB && top_k < V && V <= 32 * ILLM_WAVE * (SB / ILLM_WAVE))
        hipLaunchKernelGGL((sample_topk_kernel<false, 32>), dim3(B), dim3(SB), 0, (hipStream_t)stream, logits,
                           scratch, out, V, temp, top_k, top_p, repeat_penalty, last_tokens, n_last,
                           seeds, counters);
    else if (top_k > 0 && top_k <= SB && top_k < V)
        hipLaunchKernelGGL((sample_topk_kernel<false, 0>), dim3(B), dim3(SB), 0, (hipStream_t)stream, logits,
                           scratch, out, V, temp, top_k, top_p, repeat_penalty, last_tokens, n_last,
                           seeds, counters);
    else if (V <= SAMPLE_REG_IDS * SB)
        hipLaunchKernelGGL(sample_kernel<true>, dim3(B), dim3(SB), 0, (hipStream_t)stream, logits,
                           scratch, out, V, temp, top_k, top_p, repeat_penalty, last_tokens, n_last,
                           seeds, counters);
    else
        hipLaunchKernelGGL(sample_kernel<false>, dim3(B), dim3(SB), 0, (hipStream_t)stream, logits,
                           scratch, out, V, temp, top_k, top_p, repeat_penalty, last_tokens, n_last,
                           seeds, counters);
    return illm_launch_status();
}

// Causal attention in float32 arithmetic for any head size up to 256, any number
// of heads and groups, float32 or bfloat16 storage: one kernel for whole prompts
// (keys and values of the step itself) and one for a single new token per sequence
// over the paged cache.  These are the kernels of the 32-bit path and the
// fallback for sizes the MFMA kernels do not take.  Float32 prompts with head sizes
// 32 to 128 take a third kernel, on the matrix cores' float32 instruction.
//
// What they compute is the reference's chain scores -> scale and mask -> softmax
// -> context (src/core/op.cpp:485-498; src/kern/naive/naive.cpp:606-632, :531-553,
// :209-240, :664-691), with query head h reading kv head h / (heads / kv_heads)
// (naive.cpp:576-604).  The reference materialises the scores [heads, S, P+S]
// (op.cpp:323-326); here they live tile by tile with a running max and sum.
#include <math.h>

#include "api.h"
#include "api_test.h"
#include "common.h"

#define AQ 32  // query rows of a block
#define AK 32  // keys of a tile
#define NEG_INF (-INFINITY)

// Where a step's rows go on from tokens the cache already holds (PAGED): keys and values are
// read from the paged cache, which holds the step's own rows too by then, at absolute positions;
// row r of sequence b stands at position seq_start[b] + r.
struct AttnPages {
    const void* kcache;
    const void* vcache;
    const int32_t* page_table;
    const int32_t* seq_slot;
    const int32_t* seq_start;
    int table_stride, page_size, ring;
};

// grid (query tiles, heads, sequences); 256 threads: 8 per query row.
template <bool PAGED>
__global__ void __launch_bounds__(256)
attn_prefill_generic_kernel(const void* __restrict__ qkv, void* __restrict__ out, int dt,
                            const int32_t* __restrict__ cu, int nh, int nkv, int hd, float scale,
                            int window, AttnPages pg) {
    extern __shared__ float smem[];
    const int hp = hd + 1;
    float* qs = smem;            // [AQ][hp]
    float* ks = qs + AQ * hp;    // [AK][hp]
    float* vs = ks + AK * hp;    // [AK][hp]
    float* ps = vs + AK * hp;    // [AQ][AK + 1]
    const int b = blockIdx.z, h = blockIdx.y;
    const int start = cu[b], len = cu[b + 1] - start;
    const int q0 = blockIdx.x * AQ;
    if (q0 >= len) return;
    const int pos0 = PAGED ? pg.seq_start[b] : 0;       // position of the sequence's first row
    const int slot = PAGED ? pg.seq_slot[b] : 0;
    const int total = pos0 + len;                       // keys of the sequence after this step
    const int kvh = h / (nh / nkv);
    const size_t rowlen = (size_t)(nh + 2 * nkv) * hd;
    const int tid = threadIdx.x, i = tid >> 3, g = tid & 7;

    for (int e = tid; e < AQ * hd; e += 256) {
        const int r = e / hd, d = e - r * hd;
        qs[r * hp + d] = (q0 + r < len)
                             ? ld_f(qkv, dt, (size_t)(start + q0 + r) * rowlen + (size_t)h * hd + d)
                             : 0.f;
    }
    float m_i = NEG_INF, l_i = 0.f;
    float acc[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) acc[k] = 0.f;
    const int qrow = q0 + i;                            // row within the sequence's rows of the step
    const int qpos = pos0 + qrow;                       // its position
    const int k_hi = min(total, pos0 + q0 + AQ);
    int k_lo = window > 0 ? max(0, pos0 + q0 - window + 1) : 0;
    k_lo = (k_lo / AK) * AK;

    for (int k0 = k_lo; k0 < k_hi; k0 += AK) {
        __syncthreads();
        for (int e = tid; e < AK * hd; e += 256) {
            const int r = e / hd, d = e - r * hd;
            float kv = 0.f, vv = 0.f;
            if (k0 + r < total) {
                if (PAGED) {
                    const size_t at = cache_row_offset(pg.page_table, pg.table_stride, slot, k0 + r,
                                                       pg.page_size, pg.ring, nkv, kvh, hd) + d;
                    kv = ld_f(pg.kcache, dt, at);
                    vv = ld_f(pg.vcache, dt, at);
                } else {
                    const size_t base = (size_t)(start + k0 + r) * rowlen;
                    kv = ld_f(qkv, dt, base + (size_t)(nh + kvh) * hd + d);
                    vv = ld_f(qkv, dt, base + (size_t)(nh + nkv + kvh) * hd + d);
                }
            }
            ks[r * hp + d] = kv;
            vs[r * hp + d] = vv;
        }
        __syncthreads();
        float s[4];
        float tm = NEG_INF;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int j = g + 8 * c, kj = k0 + j;
            float a = 0.f;
            for (int d = 0; d < hd; ++d) a = fmaf(qs[i * hp + d], ks[j * hp + d], a);
            const bool ok = qrow < len && kj <= qpos && (window <= 0 || kj > qpos - window);
            s[c] = ok ? a * scale : NEG_INF;
            tm = fmaxf(tm, s[c]);
        }
        tm = fmaxf(tm, __shfl_xor(tm, 1, ILLM_WAVE));
        tm = fmaxf(tm, __shfl_xor(tm, 2, ILLM_WAVE));
        tm = fmaxf(tm, __shfl_xor(tm, 4, ILLM_WAVE));
        const float m_new = fmaxf(m_i, tm);
        const float alpha = (m_new == NEG_INF) ? 1.f : expf(m_i - m_new);
        float psum = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float p = (s[c] == NEG_INF) ? 0.f : expf(s[c] - m_new);
            ps[i * (AK + 1) + g + 8 * c] = p;
            psum += p;
        }
        psum += __shfl_xor(psum, 1, ILLM_WAVE);
        psum += __shfl_xor(psum, 2, ILLM_WAVE);
        psum += __shfl_xor(psum, 4, ILLM_WAVE);
        l_i = l_i * alpha + psum;
        m_i = m_new;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const int d = g + 8 * k;
            if (d < hd) {
                float a = acc[k] * alpha;
                for (int j = 0; j < AK; ++j) a = fmaf(ps[i * (AK + 1) + j], vs[j * hp + d], a);
                acc[k] = a;
            }
        }
    }
    if (qrow < len) {
        const float inv = 1.0f / l_i;
        const size_t ob = (size_t)(start + qrow) * nh * hd + (size_t)h * hd;
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const int d = g + 8 * k;
            if (d < hd) st_f(out, dt, ob + d, acc[k] * inv);
        }
    }
}

// The same attention for float32 storage and head sizes 32, 64, 96 and 128 on the matrix cores'
// float32 instruction (MFMA 32x32x2: float32 operands, products and sums), 8 times the kernel
// above at 2,048 tokens.  grid (tiles of 128 queries, heaviest first; heads; sequences); a wave
// takes 32 queries.  Both products are kept transposed so that a lane's column is its query:
// scores^T = K . Q^T puts the 16 scores of query (lane % 32) into a lane and its partner 32 lanes
// on (max and sum: one exchange), and in context^T = V^T . P^T the lane's own 16 weights are the
// second operand as they stand, the keys of a step being 8 g + v for the lower half of the wave
// and 8 g + 4 + v for the upper.  Keys and values go through LDS 32 keys at a time (K padded by
// one float a row); the next tile's loads are in flight while this one is multiplied.
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
#define FQ 128  // query rows of a block
#define FK 32   // keys of a tile

template <int HD, bool PAGED>
__global__ void __launch_bounds__(256, 2)
attn_prefill_f32_mfma_kernel(const float* __restrict__ qkv, float* __restrict__ out,
                             const int32_t* __restrict__ cu, int nh, int nkv, float scale,
                             int window, AttnPages pg) {
    constexpr int KLD = HD + 1;
    constexpr int NT = HD / 32;                  // tiles of 32 dims; float4 of a thread a tile
    __shared__ float ks[FK * KLD];
    __shared__ __align__(16) float vs[FK * HD];
    const int b = blockIdx.z, h = blockIdx.y;
    const int start = cu[b], len = cu[b + 1] - start;
    const int q0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * FQ;
    if (q0 >= len) return;
    const int pos0 = PAGED ? pg.seq_start[b] : 0;
    const int slot = PAGED ? pg.seq_slot[b] : 0;
    const int total = pos0 + len;
    const int kvh = h / (nh / nkv);
    const size_t rowlen = (size_t)(nh + 2 * nkv) * HD;
    const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
    const int col = lane & 31, half = lane >> 5;
    const int qrow = q0 + 32 * wave + col;                 // row within the step's rows of the sequence
    const int qpos = pos0 + qrow;
    const bool wave_has_rows = q0 + 32 * wave < len;

    // the query row: dims 2 s + half
    float q[HD / 2];
    {
        const float4* src = (const float4*)(qkv + (size_t)(start + min(qrow, len - 1)) * rowlen + (size_t)h * HD);
#pragma unroll
        for (int j = 0; j < HD / 4; ++j) {
            const float4 x = src[j];
            q[2 * j] = half ? x.y : x.x;
            q[2 * j + 1] = half ? x.w : x.z;
        }
    }
    const float* kbase = PAGED ? (const float*)pg.kcache : qkv + (size_t)(nh + kvh) * HD;
    const float* vbase = PAGED ? (const float*)pg.vcache : qkv + (size_t)(nh + nkv + kvh) * HD;
    f32x4_t kreg[NT], vreg[NT];                  // (native vectors: arrays of HIP's float4 stay in memory)
    auto fetch = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const int e = tid + 256 * i, row = e / (HD / 4), dq = e % (HD / 4);
            const int kj = min(k0 + row, total - 1);       // keys past the end: a valid row, masked below
            const size_t at = (PAGED ? cache_row_offset(pg.page_table, pg.table_stride, slot, kj,
                                                        pg.page_size, pg.ring, nkv, kvh, HD)
                                     : (size_t)(start + kj) * rowlen) + 4 * dq;
            kreg[i] = *(const f32x4_t*)(kbase + at);
            vreg[i] = *(const f32x4_t*)(vbase + at);
        }
    };
    auto stage = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const int e = tid + 256 * i, row = e / (HD / 4), dq = e % (HD / 4);
            float* kd = ks + row * KLD + 4 * dq;
            kd[0] = kreg[i].x; kd[1] = kreg[i].y; kd[2] = kreg[i].z; kd[3] = kreg[i].w;
            *(f32x4_t*)(vs + row * HD + 4 * dq) = vreg[i];
        }
    };
    f32x16_t o[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[t][v] = 0.f;
    float m_i = NEG_INF, l_i = 0.f;

    const int k_hi = min(total, pos0 + q0 + FQ);
    int k_lo = window > 0 ? max(0, pos0 + q0 - window + 1) : 0;
    k_lo = (k_lo / FK) * FK;
    const int wq_lo = pos0 + q0 + 32 * wave, wq_hi = wq_lo + 31;
    const int k_last = k_lo + ((k_hi - 1 - k_lo) / FK) * FK;
    fetch(k_lo);
    for (int k0 = k_lo; k0 < k_hi; k0 += FK) {
        __syncthreads();
        stage();
        __syncthreads();
        fetch(min(k0 + FK, k_last));              // (unconditional: the last tile is asked for twice)
        // a wave leaves out tiles that lie after all its queries or before all their windows
        if (!wave_has_rows || k0 > wq_hi || (window > 0 && k0 + FK - 1 <= wq_lo - window)) continue;
        f32x16_t sc;
#pragma unroll
        for (int v = 0; v < 16; ++v) sc[v] = 0.f;
        const float* kr = ks + col * KLD + half;
#pragma unroll
        for (int s = 0; s < HD / 2; ++s)
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kr[2 * s], q[s], sc, 0, 0, 0);
        float tm = NEG_INF;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int kj = k0 + 8 * (v >> 2) + 4 * half + (v & 3);
            const bool ok = qrow < len && kj <= qpos && (window <= 0 || kj > qpos - window);
            sc[v] = ok ? sc[v] * scale : NEG_INF;
            tm = fmaxf(tm, sc[v]);
        }
        tm = fmaxf(tm, __shfl_xor(tm, 32, ILLM_WAVE));
        const float m_new = fmaxf(m_i, tm);
        const float alpha = (m_new == NEG_INF) ? 1.f : expf(m_i - m_new);
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            sc[v] = (sc[v] == NEG_INF) ? 0.f : expf(sc[v] - m_new);
            psum += sc[v];
        }
        psum += __shfl_xor(psum, 32, ILLM_WAVE);
        l_i = l_i * alpha + psum;
        m_i = m_new;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[t][v] *= alpha;
        const float* vr = vs + 4 * half * HD + col;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = 8 * (v >> 2) + (v & 3);         // + 4 * half, in vr
#pragma unroll
            for (int t = 0; t < NT; ++t)
                o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[key * HD + 32 * t], sc[v], o[t], 0, 0, 0);
        }
    }
    if (qrow < len) {
        const float inv = 1.0f / l_i;
        float* dst = out + (size_t)(start + qrow) * nh * HD + (size_t)h * HD + 4 * half;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *(float4*)(dst + 32 * t + 8 * g) = make_float4(o[t][4 * g] * inv, o[t][4 * g + 1] * inv,
                                                               o[t][4 * g + 2] * inv, o[t][4 * g + 3] * inv);
    }
}

static int g_attn_f32_mfma = 1;
extern "C" void illm_set_attn_f32_mfma(int on) { g_attn_f32_mfma = on ? 1 : 0; }

template <int HD, bool PAGED>
static int launch_prefill_f32_mfma(const void* qkv, void* out, const int32_t* cu_seqlens, int n_seqs,
                                   int max_len, int nh, int nkv, float scale, int window,
                                   const AttnPages& pg, hipStream_t stream) {
    hipLaunchKernelGGL((attn_prefill_f32_mfma_kernel<HD, PAGED>), dim3((max_len + FQ - 1) / FQ, nh, n_seqs),
                       dim3(256), 0, stream, (const float*)qkv, (float*)out, cu_seqlens, nh, nkv, scale,
                       window, pg);
    return illm_launch_status();
}

template <bool PAGED>
static int launch_prefill_generic(const void* qkv, void* out, int dt, const int32_t* cu_seqlens,
                                  int n_seqs, int max_len, int nh, int nkv, int hd, float scale,
                                  int window, const AttnPages& pg, hipStream_t stream) {
    if (n_seqs < 0 || max_len < 0 || nh <= 0 || nkv <= 0 || nh % nkv || hd <= 0 || hd > 256 ||
        !illm_dtype_ok(dt) || nh > 65535 || n_seqs > 65535)
        return ILLM_ERR_ARG;
    if (n_seqs == 0 || max_len == 0) return ILLM_OK;
    if (dt == ILLM_F32 && g_attn_f32_mfma) {
        switch (hd) {
            case 32: return launch_prefill_f32_mfma<32, PAGED>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, pg, stream);
            case 64: return launch_prefill_f32_mfma<64, PAGED>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, pg, stream);
            case 96: return launch_prefill_f32_mfma<96, PAGED>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, pg, stream);
            case 128: return launch_prefill_f32_mfma<128, PAGED>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, pg, stream);
            default: break;
        }
    }
    const size_t smem = ((size_t)(AQ + 2 * AK) * (hd + 1) + AQ * (AK + 1)) * sizeof(float);
    if (smem > 48 * 1024) {
        if (hipFuncSetAttribute((const void*)attn_prefill_generic_kernel<PAGED>,
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)smem) != hipSuccess) {
            (void)hipGetLastError();
            return ILLM_ERR_ARG;
        }
    }
    hipLaunchKernelGGL(attn_prefill_generic_kernel<PAGED>, dim3((max_len + AQ - 1) / AQ, nh, n_seqs),
                       dim3(256), smem, stream, qkv, out, dt, cu_seqlens, nh, nkv, hd, scale, window,
                       pg);
    return illm_launch_status();
}

extern "C" int illm_attn_prefill_generic(const void* qkv, void* out, int dt,
                                         const int32_t* cu_seqlens, int n_seqs, int max_len,
                                         int nh, int nkv, int hd, float scale, int window,
                                         void* stream) {
    return launch_prefill_generic<false>(qkv, out, dt, cu_seqlens, n_seqs, max_len, nh, nkv, hd,
                                         scale, window, AttnPages(), (hipStream_t)stream);
}

extern "C" int illm_attn_prefill_paged_generic(const void* qkv, void* out, int dt,
                                               const int32_t* cu_seqlens, const int32_t* seq_slot,
                                               const int32_t* seq_start, const void* kcache,
                                               const void* vcache, const int32_t* page_table,
                                               int table_stride, int page_size, int ring, int n_seqs,
                                               int max_len, int nh, int nkv, int hd, float scale,
                                               int window, void* stream) {
    if (!seq_slot || !seq_start || !kcache || !vcache || !page_table || table_stride <= 0 ||
        page_size <= 0)
        return ILLM_ERR_ARG;
    const AttnPages pg = {kcache, vcache, page_table, seq_slot, seq_start, table_stride, page_size, ring};
    return launch_prefill_generic<true>(qkv, out, dt, cu_seqlens, n_seqs, max_len, nh, nkv, hd,
                                        scale, window, pg, (hipStream_t)stream);
}

// ---------------------------------------------------------------- decode
// grid (heads, sequences, splits); 256 threads.  A split takes whole tiles of 256 keys aligned at
// absolute positions.  A wave takes eight keys at a time, in turn with the block's other waves;
// lane l holds dims l, l + 64, l + 128, l + 192 of the query and of its sums, so a key's or a
// value's row is read 256 bytes an instruction (a thread a key, walking its row by itself, took
// 155 us for 520 keys at head size 128: every load of a wave touched 64 rows), and the eight
// scores are summed over the wave together, each step handing half of them to the partner lane.
// The waves' (sums, max, weight) are combined in wave order at the end; each block leaves
// (acc[hd], max, sum) in `partial`.  Plain float32 arithmetic and expf.
// A wave asks for the keys and the values of its next eight keys together, before it works on
// the eight it has: one trip to memory a round instead of two, and that one beside the arithmetic.
template <int DT, int DL>                  // storage type; dims a lane holds (head sizes up to 64 DL)
__global__ void __launch_bounds__(256)
attn_decode_generic_kernel(const void* __restrict__ qkv, const void* __restrict__ kcache,
                           const void* __restrict__ vcache,
                           const int32_t* __restrict__ page_table, int table_stride,
                           int page_size, int ring, const int32_t* __restrict__ seq_slot,
                           const int32_t* __restrict__ seq_len, float* __restrict__ partial,
                           int nsplit, int nh, int nkv, int hd, float scale, int window) {
    constexpr int KU = 8;                  // keys a wave takes at a time
    __shared__ float wave_acc[4][256];
    __shared__ float wave_ml[4][2];
    const int h = blockIdx.x, b = blockIdx.y, sp = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int slot = seq_slot[b];
    const int len = seq_len[b];
    const int kvh = h / (nh / nkv);
    const size_t rowlen = (size_t)(nh + 2 * nkv) * hd;
    const int k_first = window > 0 ? max(0, len - window) : 0;
    const int first_tile = k_first / 256;
    const int n_tiles = (len + 255) / 256 - first_tile;
    const int per_split = (n_tiles + nsplit - 1) / nsplit;
    const int t_lo = first_tile + sp * per_split;
    const int t_hi = min(first_tile + n_tiles, t_lo + per_split);
    const int k_lo = max(k_first, t_lo * 256), k_hi = min(len, t_hi * 256);

    float q[DL], acc[DL];
    int dim[DL];                           // (a lane without a dim reads dim 0; its sums are dropped)
#pragma unroll
    for (int i = 0; i < DL; ++i) {
        const int d = lane + 64 * i;
        dim[i] = d < hd ? d : 0;
        q[i] = d < hd ? ld_f(qkv, DT, (size_t)b * rowlen + (size_t)h * hd + d) : 0.f;
        acc[i] = 0.f;
    }
    float m = NEG_INF, l = 0.f;
    // keys beyond the range read its last key again (an existing row) and get no weight
    auto load = [&](int k0, float (&kk)[KU][DL], float (&vv)[KU][DL]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < KU; ++j) {
            const size_t off = cache_row_offset(page_table, table_stride, slot, min(k0 + j, k_hi - 1),
                                                page_size, ring, nkv, kvh, hd);
#pragma unroll
            for (int i = 0; i < DL; ++i) {
                kk[j][i] = ld_f(kcache, DT, off + dim[i]);
                vv[j][i] = ld_f(vcache, DT, off + dim[i]);
            }
        }
    };
    auto work = [&](int k0, const float (&kk)[KU][DL], const float (&vv)[KU][DL]) __attribute__((always_inline)) {
        float part[KU];
#pragma unroll
        for (int j = 0; j < KU; ++j) {
            float a = 0.f;
#pragma unroll
            for (int i = 0; i < DL; ++i) a = fmaf(q[i], kk[j][i], a);
            part[j] = a;
        }
        // eight sums over 64 lanes: three steps that halve what a lane keeps (the sums whose
        // number has the lane's bit), then three plain ones; sum j ends in the lanes with
        // (lane & 7) == j
#pragma unroll
        for (int bit = 1, n = KU / 2; bit < KU; bit <<= 1, n >>= 1) {
            const bool up = (lane & bit) != 0;
#pragma unroll
            for (int k = 0; k < n; ++k) {
                const float keep = up ? part[2 * k + 1] : part[2 * k];
                const float send = up ? part[2 * k] : part[2 * k + 1];
                part[k] = keep + __shfl_xor(send, bit, ILLM_WAVE);
            }
        }
        float mine = part[0];
#pragma unroll
        for (int o = KU; o < 64; o <<= 1) mine += __shfl_xor(mine, o, ILLM_WAVE);
        float s[KU];
#pragma unroll
        for (int j = 0; j < KU; ++j) {
            const float v = __shfl(mine, j, ILLM_WAVE) * scale;
            s[j] = k0 + j < k_hi ? v : NEG_INF;
        }
        float mx = s[0];
#pragma unroll
        for (int j = 1; j < KU; ++j) mx = fmaxf(mx, s[j]);
        const float m_new = fmaxf(m, mx);          // finite: key k0 is in the range
        const float alpha = (m == NEG_INF) ? 0.f : expf(m - m_new);
        float psum = 0.f, pv[KU];
#pragma unroll
        for (int j = 0; j < KU; ++j) {
            pv[j] = (s[j] == NEG_INF) ? 0.f : expf(s[j] - m_new);
            psum += pv[j];
        }
        l = l * alpha + psum;
        m = m_new;
#pragma unroll
        for (int i = 0; i < DL; ++i) {
            float a = acc[i] * alpha;
#pragma unroll
            for (int j = 0; j < KU; ++j) a = fmaf(pv[j], vv[j][i], a);
            acc[i] = a;
        }
    };
    int k0 = k_lo + wave * KU;
    if (k0 < k_hi) {                                   // (else the wave has no key: k_hi - 1 may not be a row)
        float k_a[KU][DL], v_a[KU][DL], k_b[KU][DL], v_b[KU][DL];
        load(k0, k_a, v_a);
        while (true) {
            load(k0 + 4 * KU, k_b, v_b);               // (past the range: its last key again, not used)
            work(k0, k_a, v_a);
            k0 += 4 * KU;
            if (k0 >= k_hi) break;
            load(k0 + 4 * KU, k_a, v_a);
            work(k0, k_b, v_b);
            k0 += 4 * KU;
            if (k0 >= k_hi) break;
        }
    }
    // the waves' results, combined in wave order
#pragma unroll
    for (int i = 0; i < DL; ++i) wave_acc[wave][lane + 64 * i] = acc[i];
    if (lane == 0) {
        wave_ml[wave][0] = m;
        wave_ml[wave][1] = l;
    }
    __syncthreads();
    float mb = NEG_INF;
    for (int w = 0; w < 4; ++w) mb = fmaxf(mb, wave_ml[w][0]);
    float lb = 0.f, f[4];
    for (int w = 0; w < 4; ++w) {
        f[w] = (wave_ml[w][0] == NEG_INF) ? 0.f : expf(wave_ml[w][0] - mb);
        lb += f[w] * wave_ml[w][1];
    }
    float* pp = partial + (((size_t)b * nh + h) * nsplit + sp) * (size_t)(hd + 2);
    const int tid = threadIdx.x;
    if (tid < hd) {
        float a = 0.f;
        for (int w = 0; w < 4; ++w) a += f[w] * wave_acc[w][tid];
        pp[tid] = a;
    }
    if (tid == 0) {
        pp[hd] = mb;
        pp[hd + 1] = lb;
    }
}

// grid (heads, sequences): combine the splits' partial results.
__global__ void attn_decode_merge_kernel(const float* __restrict__ partial, void* __restrict__ out,
                                         int dt, int nsplit, int nh, int hd) {
    const int h = blockIdx.x, b = blockIdx.y;
    const float* pp = partial + ((size_t)b * nh + h) * nsplit * (size_t)(hd + 2);
    float m = NEG_INF;
    for (int s = 0; s < nsplit; ++s) m = fmaxf(m, pp[(size_t)s * (hd + 2) + hd]);
    float L = 0.f;
    for (int s = 0; s < nsplit; ++s) {
        const float ms = pp[(size_t)s * (hd + 2) + hd];
        if (ms != NEG_INF) L += expf(ms - m) * pp[(size_t)s * (hd + 2) + hd + 1];
    }
    const float inv = 1.0f / L;
    for (int d = threadIdx.x; d < hd; d += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < nsplit; ++s) {
            const float ms = pp[(size_t)s * (hd + 2) + hd];
            if (ms != NEG_INF) a += expf(ms - m) * pp[(size_t)s * (hd + 2) + d];
        }
        st_f(out, dt, ((size_t)b * nh + h) * hd + d, a * inv);
    }
}

extern "C" int illm_attn_decode_generic(const void* qkv, void* out, int dt, const void* kcache,
                                        const void* vcache, const int32_t* page_table,
                                        int table_stride, int page_size, int ring,
                                        const int32_t* seq_slot, const int32_t* seq_len,
                                        float* partial, int nsplit, int B, int nh, int nkv, int hd,
                                        float scale, int window, void* stream) {
    if (B < 0 || nh <= 0 || nkv <= 0 || nh % nkv || hd <= 0 || hd > 256 || !illm_dtype_ok(dt) ||
        nsplit <= 0 || nsplit > 65535 || B > 65535 || page_size <= 0 || table_stride <= 0)
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
#define ILLM_DECODE_GENERIC(DT, DL)                                                                   \
    hipLaunchKernelGGL((attn_decode_generic_kernel<DT, DL>), dim3(nh, B, nsplit), dim3(256), 0,       \
                       (hipStream_t)stream, qkv, kcache, vcache, page_table, table_stride, page_size, \
                       ring, seq_slot, seq_len, partial, nsplit, nh, nkv, hd, scale, window)
    const int dl = (hd + 63) / 64;
    if (dt == ILLM_F32) {
        if (dl == 1) ILLM_DECODE_GENERIC(ILLM_F32, 1);
        else if (dl == 2) ILLM_DECODE_GENERIC(ILLM_F32, 2);
        else ILLM_DECODE_GENERIC(ILLM_F32, 4);
    } else {
        if (dl == 1) ILLM_DECODE_GENERIC(ILLM_BF16, 1);
        else if (dl == 2) ILLM_DECODE_GENERIC(ILLM_BF16, 2);
        else ILLM_DECODE_GENERIC(ILLM_BF16, 4);
    }
#undef ILLM_DECODE_GENERIC
    hipLaunchKernelGGL(attn_decode_merge_kernel, dim3(nh, B), dim3(64), 0, (hipStream_t)stream,
                       (const float*)partial, out, dt, nsplit, nh, hd);
    return illm_launch_status();
}

// Decode attention for bfloat16: one new token per sequence over the paged cache.
//
// The step is bound by reading K and V once.  A 64-lane wave is a work unit: it
// walks tiles of keys of one (sequence, kv head), all query heads of the group at
// once, so K and V are read once per group.  LPR lanes share a key row with one
// 16-byte load each (8 head dims per lane); 64/LPR keys are covered by one load
// instruction, and a tile's loads are all issued before any is used.  Scores are
// reduced over the LPR lanes of a row, the running max / sum are wave-wide, and
// each lane accumulates P.V for its 8 dims over the keys of its row group; the
// groups are added once at the end.  The waves of a block take the tiles of their key range
// in turn and combine their results through LDS; splits of the key range across blocks
// (for few sequences) leave (acc, max, sum) for the merge kernel.
//
// Same chain as src/core/op.cpp:485-498 with S = 1, grouped as
// src/kern/naive/naive.cpp:576-604.
#include <math.h>

#include <mutex>

#include "api.h"
#include "api_test.h"
#include "common.h"

#define NEG_INF (-INFINITY)

// e^x for the softmax of bfloat16 rows: the hardware's base-2 exponential of x * log2(e), three
// instructions instead of the library routine's thirty; its relative error, about |x| * 6e-8, is
// far below what bfloat16 keeps.  (The float32 path has kernels of its own with expf.)
__device__ __forceinline__ float fexp(float x) {
    return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f);
}

__device__ __forceinline__ void unpack8(const illm_u32x4_t& v, float* f) {
    f[0] = __uint_as_float(v[0] << 16); f[1] = __uint_as_float(v[0] & 0xffff0000u);
    f[2] = __uint_as_float(v[1] << 16); f[3] = __uint_as_float(v[1] & 0xffff0000u);
    f[4] = __uint_as_float(v[2] << 16); f[5] = __uint_as_float(v[2] & 0xffff0000u);
    f[6] = __uint_as_float(v[3] << 16); f[7] = __uint_as_float(v[3] & 0xffff0000u);
}

__device__ __forceinline__ void unpack8(const uint4& v, float* f) {
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
    f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
    f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}

// Combining the results that the waves of a block left in LDS and writing them out, by the
// whole block: row (w, head) is at lds + (w * n_heads + head) * (hd + 4) floats and holds hd
// sums, then the wave's max and sum.  A thread takes 4 dims of one head and asks for all the
// waves' values at once (a wave beyond `waves` reads the last one's row again, with weight
// zero): one wave walking through heads and waves in turn took longer than a tile of keys.
// The block's heads are bh0, bh0 + 1, ... in the numbering b * nh + head; a wave's rows are
// row_heads apart, of which the first n_heads count.
#define DEC_MAXW 8
__device__ __forceinline__ void combine_block(const float* lds, int row_heads, int n_heads, int hd,
                                              int waves, bf16_t* out, float* partial, int nsplit,
                                              int sp, size_t bh0) {
    const int stride = hd + 4, per_head = hd / 4;
    for (int idx = threadIdx.x; idx < n_heads * per_head; idx += blockDim.x) {
        const int hl = idx / per_head, d = (idx % per_head) * 4;
        float mw[DEC_MAXW], lw[DEC_MAXW];
        float4 v[DEC_MAXW];
#pragma unroll
        for (int w = 0; w < DEC_MAXW; ++w) {
            const float* wr = lds + ((size_t)(w < waves ? w : waves - 1) * row_heads + hl) * stride;
            mw[w] = wr[hd];
            lw[w] = wr[hd + 1];
            v[w] = *(const float4*)(wr + d);
        }
        float mm = NEG_INF;
#pragma unroll
        for (int w = 0; w < DEC_MAXW; ++w) mm = fmaxf(mm, w < waves ? mw[w] : NEG_INF);
        float L = 0.f;
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int w = 0; w < DEC_MAXW; ++w) {
            const float wgt = (w < waves && mw[w] != NEG_INF) ? fexp(mw[w] - mm) : 0.f;
            L = fmaf(wgt, lw[w], L);
            a.x = fmaf(wgt, v[w].x, a.x); a.y = fmaf(wgt, v[w].y, a.y);
            a.z = fmaf(wgt, v[w].z, a.z); a.w = fmaf(wgt, v[w].w, a.w);
        }
        const size_t bh = bh0 + hl;
        if (nsplit == 1) {
            const float inv = 1.0f / L;
            *(uint2*)(out + bh * hd + d) =
                make_uint2(pack_bf16x2(a.x * inv, a.y * inv), pack_bf16x2(a.z * inv, a.w * inv));
        } else {
            float* pp = partial + (bh * nsplit + sp) * (size_t)(hd + 2);
            *(float2*)(pp + d) = make_float2(a.x, a.y);
            *(float2*)(pp + d + 2) = make_float2(a.z, a.w);
            if (d == 0) {
                pp[hd] = mm;
                pp[hd + 1] = L;
            }
        }
    }
}

template <bool B>
struct DecMore {
    static constexpr bool value = B;
};

// LPR: lanes per key row (power of two, 8 dims each, LPR * 8 >= head_dim).
// GC: query heads handled together (power of two >= heads per kv head, at most 8).
template <int LPR, int GC>
__global__ void __launch_bounds__(GC <= 4 ? 512 : 256)
attn_decode_bf16_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ out,
                        const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
                        const int32_t* __restrict__ page_table, int table_stride, int page_size,
                        int ring, const int32_t* __restrict__ seq_slot,
                        const int32_t* __restrict__ seq_len, float* __restrict__ partial,
                        int nsplit, int nh, int nkv, int hd, float scale, int window) {
    constexpr int KPI = 64 / LPR;              // keys per load instruction
    constexpr int NI = LPR < 16 ? LPR : 16;    // load instructions per tile
    constexpr int TK = NI * KPI;               // keys per tile
    extern __shared__ __attribute__((aligned(16))) float wave_res[];   // [waves][GC][hd + 4], used when waves > 1
    const int lane = threadIdx.x & 63, wave = wave_index(), waves = blockDim.x >> 6;
    const int q = lane / LPR, c = lane % LPR;
    const int G = nh / nkv;
    const int kvh = blockIdx.x % nkv, g0 = (blockIdx.x / nkv) * GC;
    const int b = blockIdx.y, sp = blockIdx.z;
    const int slot = seq_slot[b];
    const int len = seq_len[b];
    const int kf = window > 0 ? max(0, len - window) : 0;
    const bool dim_ok = c * 8 < hd;
    const size_t rowlen = (size_t)(nh + 2 * nkv) * hd;

    float qr[GC][8];
#pragma unroll
    for (int g = 0; g < GC; ++g) {
        const bool ok = dim_ok && (g0 + g < G);
        uint4 v = make_uint4(0, 0, 0, 0);
        if (ok) v = *(const uint4*)(qkv + (size_t)b * rowlen + (size_t)(kvh * G + g0 + g) * hd + c * 8);
        unpack8(v, qr[g]);
    }
    float m[GC], l[GC], acc[GC][8];
#pragma unroll
    for (int g = 0; g < GC; ++g) {
        m[g] = NEG_INF;
        l[g] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
    }

    const int t_first = kf / TK;
    const int n_tiles = (len + TK - 1) / TK - t_first;
    const int per = (n_tiles + nsplit - 1) / nsplit;
    const int t_lo = t_first + sp * per;
    const int t_hi = min(t_first + n_tiles, t_lo + per);

    // Where tile t of the sequence begins in the cache, for this lane: row q of the tile, dims
    // 8 c .. 8 c + 7 (a lane beyond the head's dims reads the last 8 again; its values are never
    // used).  A tile of TK keys lies within a page.
    const int c_read = dim_ok ? c : 0;
    auto tile_base = [&](int t) __attribute__((always_inline)) {
        const int k0 = t * TK;
        int lp = k0 / page_size;
        if (ring > 0) lp %= ring;
        const int phys = page_table[(size_t)slot * table_stride + lp];
        return (((size_t)phys * nkv + kvh) * page_size + (k0 % page_size)) * (size_t)hd;
    };
    // The loads of a tile are unconditional, so that the wait counts are exact and a tile's loads
    // stay in flight beside the arithmetic of the one before.  A load instruction whose rows all
    // lie beyond the sequence's length reads the rows of the last one that has a row again
    // (lines that are read anyway: no more bytes from memory; the choice is the same for the
    // whole wave, a scalar offset).  Rows beyond the length that a load does bring may hold anything: their
    // scores and values are replaced before use.
    illm_u32x4_t kreg[NI], vreg[NI];
    auto load_tile = [&](const bf16_t* __restrict__ cache, size_t base, int k0,
                         illm_u32x4_t (&reg)[NI]) __attribute__((always_inline)) {
        const bf16_t* src = cache + base + (size_t)q * hd + c_read * 8;
        const int r_max = ((len - k0 - 1) / KPI) * KPI;   // first row of the last instruction with a row that exists
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int r = min(j * KPI, r_max);            // (scalar arithmetic)
            reg[j] = __builtin_nontemporal_load((const illm_u32x4_t*)(src + (size_t)r * hd));
        }
    };
    // K of the next tile is asked for as soon as the scores have used this tile's K, V of the
    // next tile as soon as the sums have used this tile's V: each load has half a tile's
    // arithmetic to arrive in, and a wave holds one tile's registers.  The wave's last tile is a
    // copy of the loop's body that asks for nothing.
    // (With several heads a wave the registers do not hold that: the tile's loads are all asked
    // for at its beginning and used as they arrive.)
    constexpr bool AHEAD = GC == 1;
    const int t_begin = t_lo + wave;
    if (AHEAD && t_begin < t_hi) {
        const size_t base = tile_base(t_begin);
        load_tile(kcache, base, t_begin * TK, kreg);
        load_tile(vcache, base, t_begin * TK, vreg);
    }
    auto one_tile = [&](auto more, int t) __attribute__((always_inline)) {
        constexpr bool MORE = AHEAD && decltype(more)::value;
        const int k0 = t * TK;
        const int t_next = t + waves;
        size_t base_next = 0;
        if constexpr (MORE) base_next = tile_base(t_next);
        if constexpr (!AHEAD) {
            const size_t base = tile_base(t);
            load_tile(kcache, base, k0, kreg);
            load_tile(vcache, base, k0, vreg);
        }

        // scores: lane (q, c) ends up owning key k0 + c * KPI + q (if c < NI).  Every lane has a
        // share of NI dot products; instead of NI full reductions over the LPR lanes of a row,
        // each step halves what a lane keeps: at the step that pairs lanes c and c ^ b, the lane
        // keeps the products whose index has c's bit b and hands the others over.
        float s_own[GC];
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            float part[NI];
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                float kf8[8];
                unpack8(kreg[j], kf8);
                float p = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) p = fmaf(qr[g][i], kf8[i], p);
                part[j] = p;
            }
            // lanes beyond the NI that own a product (LPR > NI): plain sums first
#pragma unroll
            for (int o = NI; o < LPR; o <<= 1)
#pragma unroll
                for (int j = 0; j < NI; ++j) part[j] += __shfl_xor(part[j], o, ILLM_WAVE);
#pragma unroll
            for (int b = 1, n = NI / 2; b < NI; b <<= 1, n >>= 1) {
                const bool up = (c & b) != 0;
#pragma unroll
                for (int k = 0; k < n; ++k) {
                    const float keep = up ? part[2 * k + 1] : part[2 * k];
                    const float send = up ? part[2 * k] : part[2 * k + 1];
                    part[k] = keep + __shfl_xor(send, b, ILLM_WAVE);
                }
            }
            s_own[g] = part[0] * scale;
        }
        // (scheduling barriers: the compiler would move these loads down to the others)
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (MORE) load_tile(kcache, base_next, t_next * TK, kreg);
        __builtin_amdgcn_sched_barrier(0);
        const int key_own = k0 + c * KPI + q;
        const bool own_ok = (c < NI) && key_own < len && key_own >= kf;
        float p_own[GC];
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            const float s = own_ok ? s_own[g] : NEG_INF;
            const float m_new = fmaxf(m[g], wave_max(s));
            const float alpha = (m_new == NEG_INF) ? 1.f : fexp(m[g] - m_new);
            const float p = own_ok ? fexp(s - m_new) : 0.f;
            p_own[g] = p;
            l[g] = l[g] * alpha + wave_sum(p);
            m[g] = m_new;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] *= alpha;
        }
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int key = k0 + j * KPI + q;
            const bool ok = key < len && key >= kf;
            float vf8[8];
            unpack8(vreg[j], vf8);
#pragma unroll
            for (int g = 0; g < GC; ++g) {
                float pj = __shfl(p_own[g], q * LPR + j, ILLM_WAVE);
                pj = ok ? pj : 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[g][i] = fmaf(pj, ok ? vf8[i] : 0.f, acc[g][i]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (MORE) load_tile(vcache, base_next, t_next * TK, vreg);
        __builtin_amdgcn_sched_barrier(0);
    };
    if (t_begin < t_hi) {
        int t = t_begin;
        for (; t + waves < t_hi; t += waves) one_tile(DecMore<true>{}, t);
        one_tile(DecMore<false>{}, t);
    }
    // add the row groups' shares
#pragma unroll
    for (int g = 0; g < GC; ++g)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float a = acc[g][i];
#pragma unroll
            for (int o = LPR; o < 64; o <<= 1) a += __shfl_xor(a, o, ILLM_WAVE);
            acc[g][i] = a;
        }
    if (waves > 1) {
        // every wave leaves its result in LDS; wave 0 combines them
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            float* wr = wave_res + (size_t)(wave * GC + g) * (hd + 4);
            if (q == 0 && dim_ok) {
                *(float4*)(wr + c * 8) = make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
                *(float4*)(wr + c * 8 + 4) = make_float4(acc[g][4], acc[g][5], acc[g][6], acc[g][7]);
            }
            if (lane == 0) {
                wr[hd] = m[g];
                wr[hd + 1] = l[g];
            }
        }
        __syncthreads();
        combine_block(wave_res, GC, min(GC, G - g0), hd, waves, out, partial, nsplit, sp,
                      (size_t)b * nh + kvh * G + g0);
        return;
    }
#pragma unroll
    for (int g = 0; g < GC; ++g) {
        if (g0 + g >= G) continue;
        const int h = kvh * G + g0 + g;
        if (nsplit == 1) {
            if (q == 0 && dim_ok) {
                const float inv = 1.0f / l[g];
                uint4 o;
                o.x = pack_bf16x2(acc[g][0] * inv, acc[g][1] * inv);
                o.y = pack_bf16x2(acc[g][2] * inv, acc[g][3] * inv);
                o.z = pack_bf16x2(acc[g][4] * inv, acc[g][5] * inv);
                o.w = pack_bf16x2(acc[g][6] * inv, acc[g][7] * inv);
                *(uint4*)(out + ((size_t)b * nh + h) * hd + c * 8) = o;
            }
        } else {
            float* pp = partial + (((size_t)b * nh + h) * nsplit + sp) * (size_t)(hd + 2);
            if (q == 0 && dim_ok) {
#pragma unroll
                for (int i = 0; i < 8; ++i) pp[c * 8 + i] = acc[g][i];
            }
            if (lane == 0) {
                pp[hd] = m[g];
                pp[hd + 1] = l[g];
            }
        }
    }
}

// Grouped heads (several query heads per kv head), head_dim % 32 == 0: the scores of all the
// group's heads come from the matrix cores.  S^T[key][head] = K . Q^T with MFMA 16x16x32: the A
// operand is 16 keys x 32 dims straight from the cache (16 bytes per lane), the B operand the
// group's queries (kept in registers), and a lane ends up with 4 keys of one head, so the
// softmax statistics need two exchanges per tile.  P goes through a small LDS array to the
// lanes that own the V rows, which accumulate P.V as in the kernel above.
typedef __bf16 dbf16x8_t __attribute__((ext_vector_type(8)));
typedef float df32x4_t __attribute__((ext_vector_type(4)));

template <int HD, int GC>
__global__ void __launch_bounds__(GC <= 4 ? 512 : (GC <= 8 ? 256 : 128))
attn_decode_bf16_gqa_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ out,
                            const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
                            const int32_t* __restrict__ page_table, int table_stride,
                            int page_size, int ring, const int32_t* __restrict__ seq_slot,
                            const int32_t* __restrict__ seq_len, float* __restrict__ partial,
                            int nsplit, int nh, int nkv, float scale, int window) {
    constexpr int LPR = HD <= 32 ? 4 : (HD <= 64 ? 8 : (HD <= 128 ? 16 : 32));
    constexpr int KPI = 64 / LPR;
    constexpr int NI = LPR < 16 ? LPR : 16;
    constexpr int TK = NI * KPI;               // 64 keys (32 when a row needs 32 lanes)
    constexpr int NSUB = TK / 16;              // MFMA sub-tiles of 16 keys
    constexpr int KS = HD / 32;                // k-steps of 32 dims
    constexpr int PLD = 20;                    // floats per key row of P in LDS (16 heads + pad)
    // per wave 64 * PLD floats of P; after the tiles the same memory holds the waves' results
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int lane = threadIdx.x & 63, wave = wave_index(), waves = blockDim.x >> 6;
    float* ps = lds + (size_t)wave * 64 * PLD;
    const int r = lane & 15, q4 = lane >> 4;   // MFMA roles: key / head, and k group
    const int q = lane / LPR, c = lane % LPR;  // V row roles
    const int G = nh / nkv;
    const int chunks = (G + GC - 1) / GC;
    const int kvh = blockIdx.x / chunks, g0 = (blockIdx.x % chunks) * GC;
    const int b = blockIdx.y, sp = blockIdx.z;
    const int slot = seq_slot[b];
    const int len = seq_len[b];
    const int kf = window > 0 ? max(0, len - window) : 0;
    const bool dim_ok = c * 8 < HD;
    const size_t rowlen = (size_t)(nh + 2 * nkv) * HD;
    const bool head_ok = (r < GC) && (g0 + r < G);

    uint4 qf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        qf[s] = make_uint4(0, 0, 0, 0);
        if (head_ok)
            qf[s] = *(const uint4*)(qkv + (size_t)b * rowlen + (size_t)(kvh * G + g0 + r) * HD +
                                    s * 32 + q4 * 8);
    }
    float m = NEG_INF, l = 0.f;                // of head r (the same in the four k groups)
    float acc[GC][8];
#pragma unroll
    for (int g = 0; g < GC; ++g)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;

    const int t_first = kf / TK;
    const int n_tiles = (len + TK - 1) / TK - t_first;
    const int per = (n_tiles + nsplit - 1) / nsplit;
    const int t_lo = t_first + sp * per;
    const int t_hi = min(t_first + n_tiles, t_lo + per);

    for (int t = t_lo + wave; t < t_hi; t += waves) {
        const int k0 = t * TK;
        int lp = k0 / page_size;
        if (ring > 0) lp %= ring;
        const int phys = page_table[(size_t)slot * table_stride + lp];
        const size_t tile = (((size_t)phys * nkv + kvh) * page_size + (k0 % page_size)) * (size_t)HD;
        uint4 ka[NSUB][KS], vreg[NI];
#pragma unroll
        for (int sub = 0; sub < NSUB; ++sub)
#pragma unroll
            for (int s = 0; s < KS; ++s)
                ka[sub][s] = *(const uint4*)(kcache + tile + (size_t)(sub * 16 + r) * HD + s * 32 + q4 * 8);
#pragma unroll
        for (int j = 0; j < NI; ++j)
            vreg[j] = dim_ok ? *(const uint4*)(vcache + tile + (size_t)(j * KPI + q) * HD + c * 8)
                             : make_uint4(0, 0, 0, 0);
        // scores of 4 keys per sub-tile for head r
        float sv[NSUB][4];
        float mx = NEG_INF;
#pragma unroll
        for (int sub = 0; sub < NSUB; ++sub) {
            df32x4_t a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; ++s)
                a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const dbf16x8_t*)&ka[sub][s],
                                                            *(const dbf16x8_t*)&qf[s], a, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = k0 + sub * 16 + 4 * q4 + i;
                const bool ok = key < len && key >= kf;
                sv[sub][i] = ok ? a[i] * scale : NEG_INF;
                mx = fmaxf(mx, sv[sub][i]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, ILLM_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, ILLM_WAVE));
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == NEG_INF) ? 0.f : m_new;
        const float alpha = fexp(m - m_use);             // m = -inf gives 0 (nothing summed yet)
        float rs = 0.f;
        // P is private to the wave, whose LDS accesses run in program order: no barrier, only
        // a fence for the compiler
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int sub = 0; sub < NSUB; ++sub)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = (sv[sub][i] == NEG_INF) ? 0.f : fexp(sv[sub][i] - m_use);
                rs += p;
                ps[(sub * 16 + 4 * q4 + i) * PLD + r] = p;
            }
        rs += __shfl_xor(rs, 16, ILLM_WAVE);
        rs += __shfl_xor(rs, 32, ILLM_WAVE);
        l = l * alpha + rs;
        m = m_new;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            const float ag = __shfl(alpha, g, ILLM_WAVE);  // lane g holds head g's factor
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] *= ag;
        }
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int kt = j * KPI + q;
            const int key = k0 + kt;
            const bool ok = key < len && key >= kf;
            float vf8[8];
            unpack8(vreg[j], vf8);
#pragma unroll
            for (int i = 0; i < 8; ++i) vf8[i] = ok ? vf8[i] : 0.f;
#pragma unroll
            for (int g4 = 0; g4 < GC; g4 += 4) {
                const float4 pv = *(const float4*)(ps + kt * PLD + g4);
                const float pg[4] = {pv.x, pv.y, pv.z, pv.w};
#pragma unroll
                for (int gg = 0; gg < 4 && g4 + gg < GC; ++gg)
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        acc[g4 + gg][i] = fmaf(pg[gg], vf8[i], acc[g4 + gg][i]);
            }
        }
    }
#pragma unroll
    for (int g = 0; g < GC; ++g)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float a = acc[g][i];
#pragma unroll
            for (int o = LPR; o < 64; o <<= 1) a += __shfl_xor(a, o, ILLM_WAVE);
            acc[g][i] = a;
        }
    float lg[GC], mg[GC];
#pragma unroll
    for (int g = 0; g < GC; ++g) {
        lg[g] = __shfl(l, g, ILLM_WAVE);
        mg[g] = __shfl(m, g, ILLM_WAVE);
    }
    if (waves > 1) {
        __syncthreads();                       // every wave is done with its P
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            float* wr = lds + (size_t)(wave * GC + g) * (HD + 2);
            if (q == 0 && dim_ok) {
#pragma unroll
                for (int i = 0; i < 8; ++i) wr[c * 8 + i] = acc[g][i];
            }
            if (lane == 0) {
                wr[HD] = mg[g];
                wr[HD + 1] = lg[g];
            }
        }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            float mm = NEG_INF;
            for (int w = 0; w < waves; ++w) mm = fmaxf(mm, lds[(size_t)(w * GC + g) * (HD + 2) + HD]);
            float L = 0.f, a[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) a[i] = 0.f;
            for (int w = 0; w < waves; ++w) {
                const float* wr = lds + (size_t)(w * GC + g) * (HD + 2);
                const float mw = wr[HD];
                if (mw == NEG_INF) continue;
                const float wgt = fexp(mw - mm);
                L += wgt * wr[HD + 1];
                if (q == 0 && dim_ok) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) a[i] = fmaf(wgt, wr[c * 8 + i], a[i]);
                }
            }
            mg[g] = mm;
            lg[g] = L;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] = a[i];
        }
    }
#pragma unroll
    for (int g = 0; g < GC; ++g) {
        if (g0 + g >= G) continue;
        const int h = kvh * G + g0 + g;
        if (nsplit == 1) {
            if (q == 0 && dim_ok) {
                const float inv = 1.0f / lg[g];
                uint4 o;
                o.x = pack_bf16x2(acc[g][0] * inv, acc[g][1] * inv);
                o.y = pack_bf16x2(acc[g][2] * inv, acc[g][3] * inv);
                o.z = pack_bf16x2(acc[g][4] * inv, acc[g][5] * inv);
                o.w = pack_bf16x2(acc[g][6] * inv, acc[g][7] * inv);
                *(uint4*)(out + ((size_t)b * nh + h) * HD + c * 8) = o;
            }
        } else {
            float* pp = partial + (((size_t)b * nh + h) * nsplit + sp) * (size_t)(HD + 2);
            if (q == 0 && dim_ok) {
#pragma unroll
                for (int i = 0; i < 8; ++i) pp[c * 8 + i] = acc[g][i];
            }
            if (lane == 0) {
                pp[HD] = mg[g];
                pp[HD + 1] = lg[g];
            }
        }
    }
}

// Grouped heads, head_dim % 32 == 0 and <= 128: both products on the matrix cores.
//
// S^T[key][head] = K . Q^T as in the kernel above.  For O[head][dim] = P . V with MFMA 16x16x32
// the contraction runs over keys: lane (r, k-group q4) supplies 8 keys of head r as the A
// operand and lane (n, q4) 8 keys of ONE dim as the B operand, while V lies in the cache with
// the dims of a key contiguous.  Two things make that cheap.  The order of the keys within the
// contraction is free as long as A and B agree, so the 32 keys of an MFMA are taken in the order
// in which the first product left their scores: lane (r, q4) already holds head r's probabilities
// of keys 16 sub + 4 q4 + i (sub = 0..3, i = 0..3), and two sub-tiles of them are its A operand
// as they are: P never leaves the registers.  And lane (n, q4) loads, for the same 8 keys,
// the 8 dims 8 n .. 8 n + 7 (16 bytes of a row), an 8 x 8 block that it transposes in its own
// registers with byte permutes; row e of the transposed block is the B operand of the MFMA that
// gives dims 8 n + e of all 16 heads.  Eight MFMAs per 32 keys cover 128 dims, and a lane ends
// up with 4 heads x 8 consecutive dims.  A block takes up to 16 heads of a kv head.
// Measured on MI355X against the kernel above: a tile of 64 keys 1.4 us instead of 3.0 us at 4
// heads a group, and the same for 8 or 16; 8 sequences of 650 keys, 64/8 heads: 30 -> 20 us.
template <int HD>
__global__ void __launch_bounds__(512)
attn_decode_bf16_gqa_pv_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ out,
                               const bf16_t* __restrict__ kcache,
                               const bf16_t* __restrict__ vcache,
                               const int32_t* __restrict__ page_table, int table_stride,
                               int page_size, int ring, const int32_t* __restrict__ seq_slot,
                               const int32_t* __restrict__ seq_len, float* __restrict__ partial,
                               int nsplit, int nh, int nkv, float scale, int window) {
    constexpr int TK = 64;                     // keys per tile
    constexpr int KS = HD / 32;                // k-steps of 32 dims of the first product
    extern __shared__ __attribute__((aligned(16))) float lds[];   // the waves' results at the end
    const int lane = threadIdx.x & 63, wave = wave_index(), waves = blockDim.x >> 6;
    const int r = lane & 15, q4 = lane >> 4;
    const int G = nh / nkv;
    const int chunks = (G + 15) / 16;
    const int kvh = blockIdx.x / chunks, g0 = (blockIdx.x % chunks) * 16;
    const int GH = min(16, G - g0);            // heads of this block
    const int b = blockIdx.y, sp = blockIdx.z;
    const int slot = seq_slot[b];
    const int len = seq_len[b];
    const int kf = window > 0 ? max(0, len - window) : 0;
    const bool dim_ok = r * 8 < HD;            // this lane's 8 dims as an owner of V columns
    const size_t rowlen = (size_t)(nh + 2 * nkv) * HD;

    uint4 qf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        qf[s] = make_uint4(0, 0, 0, 0);
        if (r < GH)
            qf[s] = *(const uint4*)(qkv + (size_t)b * rowlen + (size_t)(kvh * G + g0 + r) * HD +
                                    s * 32 + q4 * 8);
    }
    float m = NEG_INF, l = 0.f;                // of head r (the same in the four k groups)
    df32x4_t o[8];                             // o[e][i]: head 4 q4 + i, dim 8 r + e
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (df32x4_t){0.f, 0.f, 0.f, 0.f};

    const int t_first = kf / TK;
    const int n_tiles = (len + TK - 1) / TK - t_first;
    const int per = (n_tiles + nsplit - 1) / nsplit;
    const int t_lo = t_first + sp * per;
    const int t_hi = min(t_first + n_tiles, t_lo + per);

    // Where tile t of the sequence begins in the cache (a tile of 64 keys lies within a page).
    auto tile_base = [&](int t) __attribute__((always_inline)) {
        const int k0 = t * TK;
        int lp = k0 / page_size;
        if (ring > 0) lp %= ring;
        const int phys = page_table[(size_t)slot * table_stride + lp];
        return (((size_t)phys * nkv + kvh) * page_size + (k0 % page_size)) * (size_t)HD;
    };
    // The loads of a tile are unconditional (exact wait counts: a tile's loads stay in flight
    // beside the arithmetic of the one before).  A load instruction brings 16 rows of one
    // sub-tile; one whose sub-tile lies wholly beyond the sequence's length reads the last
    // sub-tile that has a row again (lines that are read anyway; a scalar offset).  Rows beyond
    // the length that a load does bring may hold anything: their scores are replaced and their
    // values set to zero before use.
    illm_u32x4_t ka[4][KS], vr[2][8];
    const int r_read = dim_ok ? r : 0;         // (a lane beyond the head's dims: values never used)
    auto load_k = [&](size_t tile, int k0) __attribute__((always_inline)) {
        const int sub_max = (len - k0 - 1) / 16;
#pragma unroll
        for (int sub = 0; sub < 4; ++sub) {
            const int sb = min(sub, sub_max);
#pragma unroll
            for (int s = 0; s < KS; ++s)
                ka[sub][s] = *(const illm_u32x4_t*)(kcache + tile + (size_t)(sb * 16 + r) * HD + s * 32 + q4 * 8);
        }
    };
    // V: slot i of half hb is key (2 hb + i / 4) * 16 + 4 q4 + i % 4, the key whose score this
    // k group's lanes get at place i % 4 of sub-tile 2 hb + i / 4
    auto load_v = [&](size_t tile, int k0) __attribute__((always_inline)) {
        const int sub_max = (len - k0 - 1) / 16;
#pragma unroll
        for (int hb = 0; hb < 2; ++hb)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int sb = min(2 * hb + i / 4, sub_max);
                vr[hb][i] = *(const illm_u32x4_t*)(vcache + tile + (size_t)(sb * 16 + 4 * q4 + (i & 3)) * HD + r_read * 8);
            }
    };
    // K of the next tile is asked for as soon as the scores have used this tile's K, V of the
    // next tile as soon as the sums have used this tile's V; the wave's last tile is a copy of
    // the loop's body that asks for nothing.
    const int t_begin = t_lo + wave;
    if (t_begin < t_hi) {
        const size_t tile = tile_base(t_begin);
        load_k(tile, t_begin * TK);
        load_v(tile, t_begin * TK);
    }
    auto one_tile = [&](auto more, int t) __attribute__((always_inline)) {
        constexpr bool MORE = decltype(more)::value;
        const int k0 = t * TK;
        const int t_next = t + waves;
        size_t tile_next = 0;
        if constexpr (MORE) tile_next = tile_base(t_next);
        // scores of 4 keys per sub-tile for head r
        float sv[4][4];
        float mx = NEG_INF;
#pragma unroll
        for (int sub = 0; sub < 4; ++sub) {
            df32x4_t a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; ++s)
                a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const dbf16x8_t*)&ka[sub][s],
                                                            *(const dbf16x8_t*)&qf[s], a, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = k0 + sub * 16 + 4 * q4 + i;
                const bool ok = key < len && key >= kf;
                sv[sub][i] = ok ? a[i] * scale : NEG_INF;
                mx = fmaxf(mx, sv[sub][i]);
            }
        }
        // (scheduling barriers: the compiler would move these loads down to the others)
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (MORE) load_k(tile_next, t_next * TK);
        __builtin_amdgcn_sched_barrier(0);
        mx = fmaxf(mx, __shfl_xor(mx, 16, ILLM_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, ILLM_WAVE));
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == NEG_INF) ? 0.f : m_new;
        const float alpha = fexp(m - m_use);             // m = -inf gives 0 (nothing summed yet)
        float rs = 0.f;
        uint4 pa[2];                                     // head r's probabilities, two A operands
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
            float pf[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float sc = sv[2 * hb + i / 4][i & 3];
                pf[i] = (sc == NEG_INF) ? 0.f : fexp(sc - m_use);
                rs += pf[i];
            }
            pa[hb] = make_uint4(pack_bf16x2(pf[0], pf[1]), pack_bf16x2(pf[2], pf[3]),
                                pack_bf16x2(pf[4], pf[5]), pack_bf16x2(pf[6], pf[7]));
        }
        rs += __shfl_xor(rs, 16, ILLM_WAVE);
        rs += __shfl_xor(rs, 32, ILLM_WAVE);
        l = l * alpha + rs;
        m = m_new;
        // what this lane has summed belongs to heads 4 q4 + i, whose factors lanes 4 q4 + i hold
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float ai = __shfl(alpha, 4 * q4 + i, ILLM_WAVE);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e][i] *= ai;
        }
        if (k0 < kf || k0 + TK > len) {
            // a tile with keys before the window or beyond the length: their rows may hold
            // anything (NaN too), and a probability of zero would not undo that
#pragma unroll
            for (int hb = 0; hb < 2; ++hb)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int key = k0 + (2 * hb + i / 4) * 16 + 4 * q4 + (i & 3);
                    if (key < kf || key >= len) vr[hb][i] = (illm_u32x4_t){0u, 0u, 0u, 0u};
                }
        }
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                // row e of the transposed 8 keys x 8 dims block: dim 8 r + e of the 8 keys
                const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
                uint4 tr;
                const uint32_t* w0 = (const uint32_t*)&vr[hb][0];
                tr.x = __builtin_amdgcn_perm(((const uint32_t*)&vr[hb][1])[e >> 1], w0[e >> 1], sel);
                tr.y = __builtin_amdgcn_perm(((const uint32_t*)&vr[hb][3])[e >> 1],
                                             ((const uint32_t*)&vr[hb][2])[e >> 1], sel);
                tr.z = __builtin_amdgcn_perm(((const uint32_t*)&vr[hb][5])[e >> 1],
                                             ((const uint32_t*)&vr[hb][4])[e >> 1], sel);
                tr.w = __builtin_amdgcn_perm(((const uint32_t*)&vr[hb][7])[e >> 1],
                                             ((const uint32_t*)&vr[hb][6])[e >> 1], sel);
                o[e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const dbf16x8_t*)&pa[hb],
                                                               *(const dbf16x8_t*)&tr, o[e], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (MORE) load_v(tile_next, t_next * TK);
        __builtin_amdgcn_sched_barrier(0);
    };
    if (t_begin < t_hi) {
        int t = t_begin;
        for (; t + waves < t_hi; t += waves) one_tile(DecMore<true>{}, t);
        one_tile(DecMore<false>{}, t);
    }
    // this lane's heads 4 q4 + i: their max and sum from the lanes that hold them
    float lh[4], mh[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        lh[i] = __shfl(l, 4 * q4 + i, ILLM_WAVE);
        mh[i] = __shfl(m, 4 * q4 + i, ILLM_WAVE);
    }
    if (waves > 1) {
        // every wave leaves its result in LDS ([wave][head][HD + 4]); wave 0 combines them
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int hl = 4 * q4 + i;
            if (hl >= GH) continue;
            float* wr = lds + (size_t)(wave * GH + hl) * (HD + 4);
            if (dim_ok) {
                *(float4*)(wr + r * 8) = make_float4(o[0][i], o[1][i], o[2][i], o[3][i]);
                *(float4*)(wr + r * 8 + 4) = make_float4(o[4][i], o[5][i], o[6][i], o[7][i]);
            }
            if (r == 0) {
                wr[HD] = mh[i];
                wr[HD + 1] = lh[i];
            }
        }
        __syncthreads();
        combine_block(lds, GH, GH, HD, waves, out, partial, nsplit, sp,
                      (size_t)b * nh + kvh * G + g0);
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int hl = 4 * q4 + i;
        if (hl >= GH) continue;
        const int h = kvh * G + g0 + hl;
        if (nsplit == 1) {
            if (dim_ok) {
                const float inv = 1.0f / lh[i];
                uint4 ov;
                ov.x = pack_bf16x2(o[0][i] * inv, o[1][i] * inv);
                ov.y = pack_bf16x2(o[2][i] * inv, o[3][i] * inv);
                ov.z = pack_bf16x2(o[4][i] * inv, o[5][i] * inv);
                ov.w = pack_bf16x2(o[6][i] * inv, o[7][i] * inv);
                *(uint4*)(out + ((size_t)b * nh + h) * HD + r * 8) = ov;
            }
        } else {
            float* pp = partial + (((size_t)b * nh + h) * nsplit + sp) * (size_t)(HD + 2);
            if (dim_ok) {
#pragma unroll
                for (int e = 0; e < 8; ++e) pp[r * 8 + e] = o[e][i];
            }
            if (r == 0) {
                pp[HD] = mh[i];
                pp[HD + 1] = lh[i];
            }
        }
    }
}

// grid (heads, sequences), one wave: lane s holds split s's max and sum (nsplit <= 64), the
// weights are formed once, and splits that saw no key are skipped.
__global__ void __launch_bounds__(64)
attn_decode_bf16_merge_kernel(const float* __restrict__ partial, bf16_t* __restrict__ out,
                              int nsplit, int nh, int hd) {
    const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
    const float* pp = partial + ((size_t)b * nh + h) * nsplit * (size_t)(hd + 2);
    float ms = NEG_INF, ls = 0.f;
    if (lane < nsplit) {
        ms = pp[(size_t)lane * (hd + 2) + hd];
        ls = pp[(size_t)lane * (hd + 2) + hd + 1];
    }
    const float m = wave_max(ms);
    const float w = (ms == NEG_INF) ? 0.f : fexp(ms - m);
    const float inv = 1.0f / wave_sum(w * ls);
    for (int d = lane; d < hd; d += 64) {
        float a = 0.f;
        // eight splits' values are asked for at once (beyond the last: the last again, unused)
        for (int s0 = 0; s0 < nsplit; s0 += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int s = s0 + u < nsplit ? s0 + u : nsplit - 1;
                v[u] = pp[(size_t)s * (hd + 2) + d];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const float ws = __shfl(w, (s0 + u) & 63, ILLM_WAVE);
                a = (s0 + u < nsplit && ws != 0.f) ? fmaf(ws, v[u], a) : a;
            }
        }
        out[((size_t)b * nh + h) * hd + d] = f32_to_bf16(a * inv);
    }
}

template <int LPR, int GC>
static int launch_decode(const void* qkv, void* out, const void* kcache, const void* vcache,
                         const int32_t* page_table, int table_stride, int page_size, int ring,
                         const int32_t* seq_slot, const int32_t* seq_len, float* partial,
                         int nsplit, int waves, int B, int nh, int nkv, int hd, float scale,
                         int window, hipStream_t stream) {
    const int G = nh / nkv;
    const int chunks = (G + GC - 1) / GC;
    const int maxw = GC <= 4 ? 8 : 4;
    waves = waves < 1 ? 1 : (waves > maxw ? maxw : waves);
    const size_t smem = waves > 1 ? (size_t)waves * GC * (hd + 4) * sizeof(float) : 0;
    hipLaunchKernelGGL((attn_decode_bf16_kernel<LPR, GC>), dim3(nkv * chunks, B, nsplit),
                       dim3(64 * waves), smem, stream, (const bf16_t*)qkv, (bf16_t*)out, (const bf16_t*)kcache,
                       (const bf16_t*)vcache, page_table, table_stride, page_size, ring, seq_slot,
                       seq_len, partial, nsplit, nh, nkv, hd, scale, window);
    if (nsplit > 1)
        hipLaunchKernelGGL(attn_decode_bf16_merge_kernel, dim3(nh, B), dim3(64), 0, stream,
                           (const float*)partial, (bf16_t*)out, nsplit, nh, hd);
    return illm_launch_status();
}

template <int LPR>
static int launch_decode_g(int gc, const void* qkv, void* out, const void* kcache,
                           const void* vcache, const int32_t* page_table, int table_stride,
                           int page_size, int ring, const int32_t* seq_slot,
                           const int32_t* seq_len, float* partial, int nsplit, int waves, int B,
                           int nh, int nkv, int hd, float scale, int window, hipStream_t stream) {
#define GO(GC_)                                                                                   \
    return launch_decode<LPR, GC_>(qkv, out, kcache, vcache, page_table, table_stride, page_size, \
                                   ring, seq_slot, seq_len, partial, nsplit, waves, B, nh, nkv,  \
                                   hd, scale, window, stream)
    switch (gc) {
        case 1: GO(1);
        case 2: GO(2);
        case 4: GO(4);
        default: GO(8);
    }
#undef GO
}

// Sizes this kernel takes: bfloat16, head_dim a multiple of 8 up to 256, a page size that
// is a multiple of 64.  Anything else: ILLM_ERR_ARG (the caller uses the generic kernel).
// `waves`: waves per block that share a key range (clamped to what registers and LDS allow);
// `nsplit`: key ranges per sequence, combined by the merge kernel when > 1.
static int GQA_PV_ON_MATRIX_CORES = 1;      // 0: the kernel with P.V on the vector units (tuning)
extern "C" void illm_set_gqa_pv_on_matrix_cores(int on) { GQA_PV_ON_MATRIX_CORES = on; }

extern "C" int illm_attn_decode_bf16(const void* qkv, void* out, const void* kcache,
                                     const void* vcache, const int32_t* page_table,
                                     int table_stride, int page_size, int ring,
                                     const int32_t* seq_slot, const int32_t* seq_len,
                                     float* partial, int nsplit, int waves, int B, int nh, int nkv,
                                     int hd, float scale, int window, void* stream) {
    if (B < 0 || nh <= 0 || nkv <= 0 || nh % nkv || hd <= 0 || hd > 256 || hd % 8 ||
        page_size <= 0 || page_size % 64 || nsplit <= 0 || nsplit > 64 || B > 65535 ||
        table_stride <= 0 || (nsplit > 1 && !partial))
        return ILLM_ERR_ARG;
    if (B == 0) return ILLM_OK;
    const int G = nh / nkv;
    if (G > 1 && hd % 32 == 0 && hd <= 128 && GQA_PV_ON_MATRIX_CORES) {
        const int chunks = (G + 15) / 16, gh = G < 16 ? G : 16;
        const dim3 grid(nkv * chunks, B, nsplit);
        int wq = waves < 1 ? 1 : (waves > 8 ? 8 : waves);
        while (wq > 1 && (size_t)wq * gh * (hd + 4) * sizeof(float) > 64 * 1024) --wq;
        const size_t smem = wq > 1 ? (size_t)wq * gh * (hd + 4) * sizeof(float) : 0;
#define GQA_PV(HD_)                                                                                \
    hipLaunchKernelGGL((attn_decode_bf16_gqa_pv_kernel<HD_>), grid, dim3(64 * wq), smem,           \
                       (hipStream_t)stream, (const bf16_t*)qkv, (bf16_t*)out,                      \
                       (const bf16_t*)kcache, (const bf16_t*)vcache, page_table, table_stride,     \
                       page_size, ring, seq_slot, seq_len, partial, nsplit, nh, nkv, scale, window)
        switch (hd) {
            case 32: GQA_PV(32); break;
            case 64: GQA_PV(64); break;
            case 96: GQA_PV(96); break;
            default: GQA_PV(128); break;
        }
#undef GQA_PV
        if (nsplit > 1)
            hipLaunchKernelGGL(attn_decode_bf16_merge_kernel, dim3(nh, B), dim3(64), 0,
                               (hipStream_t)stream, (const float*)partial, (bf16_t*)out, nsplit, nh,
                               hd);
        return illm_launch_status();
    }
    if (G > 1 && hd % 32 == 0) {
        int gcq = 2;
        while (gcq < G && gcq < 16) gcq <<= 1;
        const int chunks = (G + gcq - 1) / gcq;
        const dim3 grid(nkv * chunks, B, nsplit);
        // waves of a block: bounded by the registers a head group needs and by 64 KB of LDS
        int wq = waves < 1 ? 1 : waves;
        const int maxw = gcq <= 4 ? 8 : (gcq <= 8 ? 4 : 2);
        wq = wq > maxw ? maxw : wq;
        size_t smem = 0;
        for (;; --wq) {
            const size_t p_bytes = (size_t)wq * 64 * 20 * sizeof(float);
            const size_t r_bytes = wq > 1 ? (size_t)wq * gcq * (hd + 2) * sizeof(float) : 0;
            smem = p_bytes > r_bytes ? p_bytes : r_bytes;
            if (smem <= 64 * 1024 || wq == 1) break;
        }
#define GQA(HD_, GC_)                                                                              \
    hipLaunchKernelGGL((attn_decode_bf16_gqa_kernel<HD_, GC_>), grid, dim3(64 * wq), smem,         \
                       (hipStream_t)stream, (const bf16_t*)qkv, (bf16_t*)out,                      \
                       (const bf16_t*)kcache, (const bf16_t*)vcache, page_table, table_stride,     \
                       page_size, ring, seq_slot, seq_len, partial, nsplit, nh, nkv, scale, window)
#define GQA_HD(HD_)                                                                                \
    do {                                                                                           \
        if (gcq == 2) GQA(HD_, 2);                                                                 \
        else if (gcq == 4) GQA(HD_, 4);                                                            \
        else if (gcq == 8) GQA(HD_, 8);                                                            \
        else GQA(HD_, 16);                                                                         \
    } while (0)
        switch (hd) {
            case 32: GQA_HD(32); break;
            case 64: GQA_HD(64); break;
            case 96: GQA_HD(96); break;
            case 128: GQA_HD(128); break;
            case 160: GQA_HD(160); break;
            case 192: GQA_HD(192); break;
            case 224: GQA_HD(224); break;
            default: GQA_HD(256); break;
        }
#undef GQA_HD
#undef GQA
        if (nsplit > 1)
            hipLaunchKernelGGL(attn_decode_bf16_merge_kernel, dim3(nh, B), dim3(64), 0,
                               (hipStream_t)stream, (const float*)partial, (bf16_t*)out, nsplit, nh,
                               hd);
        return illm_launch_status();
    }
    int gc = 1;
    while (gc < G && gc < 8) gc <<= 1;
    int lpr = 1;
    while (lpr * 8 < hd) lpr <<= 1;
    hipStream_t st = (hipStream_t)stream;
#define GO(LPR_)                                                                                   \
    return launch_decode_g<LPR_>(gc, qkv, out, kcache, vcache, page_table, table_stride, page_size, \
                                 ring, seq_slot, seq_len, partial, nsplit, waves, B, nh, nkv, hd,  \
                                 scale, window, st)
    switch (lpr) {
        case 1: GO(1);
        case 2: GO(2);
        case 4: GO(4);
        case 8: GO(8);
        case 16: GO(16);
        default: GO(32);
    }
#undef GO
}

// ---------------------------------------------------------------------------------------------
// The same decode attention for callers that cannot allocate device memory: the split results go
// through a file-scope array instead of a workspace argument.  Each GPU holds its own copy of the
// array at its own address, which the host learns once per device from the runtime; host code
// never passes the array's name to a kernel.
static __device__ __align__(256) float scratch[ILLM_DECODE_SCRATCH_BYTES / sizeof(float)];

#define ILLM_MAX_DEVICES 64
static float* scratch_of_device[ILLM_MAX_DEVICES];     // null until the device's first call
static std::mutex scratch_lock;

// The address of `scratch` on the device that holds `out` (the device the kernels will run on,
// whichever is current for the calling thread), looked up at that device's first call with that
// device current.
static int scratch_of(const void* out, float** p) {
    int dev = -1;
    hipPointerAttribute_t attr;
    if (out && hipPointerGetAttributes(&attr, out) == hipSuccess) dev = attr.device;
    else {
        (void)hipGetLastError();                        // not a pointer the runtime knows: fall back
        if (hipGetDevice(&dev) != hipSuccess) return ILLM_ERR_LAUNCH;
    }
    if (dev < 0 || dev >= ILLM_MAX_DEVICES) return ILLM_ERR_LAUNCH;
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (!scratch_of_device[dev]) {
        int current = -1;
        if (hipGetDevice(&current) != hipSuccess) return ILLM_ERR_LAUNCH;
        if (current != dev && hipSetDevice(dev) != hipSuccess) return ILLM_ERR_LAUNCH;
        void* q = nullptr;
        const hipError_t rc = hipGetSymbolAddress(&q, HIP_SYMBOL(scratch));
        if (current != dev && hipSetDevice(current) != hipSuccess) return ILLM_ERR_LAUNCH;
        if (rc != hipSuccess || !q) return ILLM_ERR_LAUNCH;
        scratch_of_device[dev] = (float*)q;
    }
    *p = scratch_of_device[dev];
    return ILLM_OK;
}

extern "C" int illm_attn_decode_bf16_static(const void* qkv, void* out, const void* kcache,
                                            const void* vcache, const int32_t* page_table,
                                            int table_stride, int page_size, int ring,
                                            const int32_t* seq_slot, const int32_t* seq_len,
                                            int nsplit, int waves, int B, int nh, int nkv, int hd,
                                            float scale, int window, void* stream) {
    if (B < 0 || nh <= 0 || nsplit <= 0 || hd <= 0) return ILLM_ERR_ARG;
    float* partial = nullptr;
    if (nsplit > 1) {
        const size_t need = (size_t)B * nh * nsplit * (size_t)(hd + 2) * sizeof(float);
        if (need > ILLM_DECODE_SCRATCH_BYTES) return ILLM_ERR_SCRATCH;
        const int rc = scratch_of(out, &partial);
        if (rc != ILLM_OK) return rc;
    }
    // every (sequence, head, split) entry that the merge reads is written by the first kernel of
    // this call (a split without keys leaves max = -inf, sum = 0), so nothing has to be cleared
    return illm_attn_decode_bf16(qkv, out, kcache, vcache, page_table, table_stride, page_size, ring,
                                 seq_slot, seq_len, partial, nsplit, waves, B, nh, nkv, hd, scale,
                                 window, stream);
}

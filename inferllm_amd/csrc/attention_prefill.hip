// Causal attention of whole prompts for bfloat16 on the matrix cores (MFMA 32x32x16),
// head sizes that are multiples of 16 up to 256 (the last block of 32 dims of the second
// product is half used when the size is no multiple of 32), any number of heads and groups,
// ragged batches.
//
// A block of 4 waves takes 128 consecutive query rows of one (sequence, head); a
// wave owns 32 of them.  Everything is computed transposed, so that a lane owns one
// query column: S^T = K . Q^T puts 32 keys of one query in a lane's accumulator, the
// running max and sum of the softmax need no reduction across lanes beyond one
// exchange between the two half-waves, and the accumulator layout of P^T is already
// the B-operand layout of the second product O^T = V^T . P^T: P never leaves
// registers.  K tiles (64 keys) go through LDS as they are; V tiles are transposed on
// their way into LDS so that 8 consecutive keys of one head dim are contiguous.  Q is
// read once into registers.  Scores and statistics are float32; exponentials are
// base 2 with log2(e) folded into the scale.
//
// The next tile's K and V are on their way from global memory (into registers) while the
// current tile is multiplied.  Blocks are numbered so that the query blocks of one
// (sequence, head) run on the same XCD (consecutive block ids go round the 8 XCDs) and
// share K and V in its L2, and so that every XCD starts with its heaviest (last) query
// blocks and ends with the middle ones.
//
// The chain is src/core/op.cpp:485-498 (scores, scale + mask, softmax, context) with
// grouped heads as src/kern/naive/naive.cpp:576-604.
#include <math.h>

#include <mutex>

#include "api.h"
#include "api_test.h"
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

#define PF_BN 64      // keys per tile
#define PF_BM 128     // query rows per block
#define NEG_INF (-INFINITY)

// PAGED: the step's rows go on from tokens the cache already holds.  Keys and values are read
// from the paged cache (which holds the step's own rows too by then) at absolute positions, a
// tile of 64 keys being one page or an aligned part of one; row r of sequence b stands at
// position seq_start[b] + r.
struct PfPages {
    const bf16_t* kcache;
    const bf16_t* vcache;
    const int32_t* page_table;
    const int32_t* seq_slot;
    const int32_t* seq_start;
    int table_stride, page_size, ring;
};

template <int HD, bool PAGED>
__global__ void __launch_bounds__(256, (HD <= 128 ? 2 : 1))
attn_prefill_mfma_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ out,
                         const int32_t* __restrict__ cu, int n_qblk, int nh, int nkv,
                         float scale_log2, int window, int hb_per_xcd, int n_hb, int zigzag,
                         PfPages pg) {
    constexpr int KLD = HD + 8;        // K tile row stride: 16 bytes of padding
    constexpr int VLD = PF_BN + 4;     // V^T row stride
    constexpr int KS = HD / 16;        // k-steps of the first product
    constexpr int DB = (HD + 31) / 32; // 32-row blocks of O^T (the last one half used when HD % 32 == 16)
    constexpr int CH = HD / 8;         // 16-byte chunks of a row
    __shared__ __attribute__((aligned(16))) bf16_t ks[PF_BN * KLD];
    __shared__ __attribute__((aligned(16))) bf16_t vts[DB * 32 * VLD];

    // XCD x takes the (sequence, head) pairs [x * hb_per_xcd, (x + 1) * hb_per_xcd); within
    // it, slots run over those pairs first and over query blocks, last block first, second
    const int xcd = blockIdx.x % 8, slot_id = blockIdx.x / 8;
    const int hb = xcd * hb_per_xcd + slot_id % hb_per_xcd;
    if (hb >= n_hb) return;
    // heavy half first (last query blocks, descending), then the light half ascending: when
    // all blocks are resident at once, the blocks that share a CU add up to about the same
    // (`zigzag`); with more blocks than fit at once, plain heaviest-first is better
    const int qi = slot_id / hb_per_xcd, top = zigzag ? (n_qblk + 1) / 2 : n_qblk;
    const int qb = qi < top ? n_qblk - 1 - qi : qi - top;
    const int h = hb % nh, b = hb / nh;
    const int start = cu[b], len = cu[b + 1] - start;
    const int q0 = qb * PF_BM;
    if (q0 >= len) return;
    const int pos0 = PAGED ? pg.seq_start[b] : 0;       // position of the sequence's first row
    const int slot = PAGED ? pg.seq_slot[b] : 0;
    const int total = pos0 + len;                       // keys of the sequence after this step
    const int kvh = h / (nh / nkv);
    const size_t rowlen = (size_t)(nh + 2 * nkv) * HD;
    const int tid = threadIdx.x, wave = wave_index(), lane = tid & 63;
    const int lq = lane & 31, half = lane >> 5;
    const int q_row0 = q0 + wave * 32;
    const int q = q_row0 + lq;                          // row within the sequence's rows
    const int qc = q < len ? q : len - 1;
    const int qp = pos0 + q;                            // its position

    if constexpr (HD % 32 != 0) {       // rows of V^T beyond the head size: operands of sums nobody stores
        for (int e = threadIdx.x; e < (DB * 32 - HD) * VLD; e += 256) vts[HD * VLD + e] = 0;
    }
    uint4 qf[KS];
    {
        const bf16_t* qp = qkv + (size_t)(start + qc) * rowlen + (size_t)h * HD + half * 8;
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = *(const uint4*)(qp + s * 16);
    }
    f32x16_t o[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[d][i] = 0.f;
    float m = NEG_INF, l = 0.f;

    const int k_end = min(total, pos0 + q0 + PF_BM);
    int k_begin = window > 0 ? max(0, pos0 + q0 - window + 1) : 0;
    k_begin = (k_begin / PF_BN) * PF_BN;
    const int wk_end = min(total, pos0 + q_row0 + 32);              // this wave's last key + 1
    const int wk_begin = window > 0 ? max(0, pos0 + q_row0 - window + 1) : 0;

    constexpr int NLD = (PF_BN * CH + 255) / 256;   // 16-byte pieces of K (and of V) per thread
    uint4 kpre[NLD], vpre[NLD];
    auto fetch = [&](int k0) {
        size_t page_base = 0;                           // PAGED: the tile's page, this kv head
        if (PAGED) {
            int lp = k0 / pg.page_size;
            if (pg.ring > 0) lp %= pg.ring;
            const int phys = pg.page_table[(size_t)slot * pg.table_stride + lp];
            page_base = ((size_t)phys * nkv + kvh) * pg.page_size;
        }
#pragma unroll
        for (int it = 0; it < NLD; ++it) {
            const int u = tid + it * 256;
            const int key = ((u >> 6) & 3) * 16 + (u & 15);
            const int ch = min((u >> 8) * 4 + ((u >> 4) & 3), CH - 1);   // (HD % 32 == 16: the last round's upper half loads a chunk again)
            const int krow = min(k0 + key, total - 1);
            if (PAGED) {
                const size_t at = (page_base + krow % pg.page_size) * HD + ch * 8;
                kpre[it] = *(const uint4*)(pg.kcache + at);
                vpre[it] = *(const uint4*)(pg.vcache + at);
            } else {
                const bf16_t* src = qkv + (size_t)(start + krow) * rowlen;
                kpre[it] = *(const uint4*)(src + (size_t)(nh + kvh) * HD + ch * 8);
                vpre[it] = *(const uint4*)(src + (size_t)(nh + nkv + kvh) * HD + ch * 8);
            }
        }
    };
    if (k_begin < k_end) fetch(k_begin);
    for (int k0 = k_begin; k0 < k_end; k0 += PF_BN) {
        __syncthreads();
        // K tile as it is, V tile transposed; a wave instruction covers 16 keys x 4 chunks
#pragma unroll
        for (int it = 0; it < NLD; ++it) {
            const int u = tid + it * 256;
            const int key = ((u >> 6) & 3) * 16 + (u & 15);
            const int ch = (u >> 8) * 4 + ((u >> 4) & 3);
            if (HD % 32 != 0 && ch >= CH) continue;
            const uint4 kv = kpre[it], vv = vpre[it];
            *(uint4*)(ks + key * KLD + ch * 8) = kv;
            bf16_t* vd = vts + (ch * 8) * VLD + key;
            vd[0 * VLD] = (bf16_t)(vv.x & 0xffffu); vd[1 * VLD] = (bf16_t)(vv.x >> 16);
            vd[2 * VLD] = (bf16_t)(vv.y & 0xffffu); vd[3 * VLD] = (bf16_t)(vv.y >> 16);
            vd[4 * VLD] = (bf16_t)(vv.z & 0xffffu); vd[5 * VLD] = (bf16_t)(vv.z >> 16);
            vd[6 * VLD] = (bf16_t)(vv.w & 0xffffu); vd[7 * VLD] = (bf16_t)(vv.w >> 16);
        }
        __syncthreads();
        if (k0 + PF_BN < k_end) fetch(k0 + PF_BN);
        if (k0 >= wk_end || k0 + PF_BN <= wk_begin) continue;       // nothing visible to this wave

        // S^T[key][q] for two sub-tiles of 32 keys
        f32x16_t s[2];
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[sub][i] = 0.f;
            const bf16_t* kp = ks + (sub * 32 + lq) * KLD + half * 8;
#pragma unroll
            for (int st = 0; st < KS; ++st) {
                const uint4 a = *(const uint4*)(kp + st * 16);
                s[sub] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&a,
                                                                 *(const bf16x8_t*)&qf[st], s[sub],
                                                                 0, 0, 0);
            }
        }
        const bool need_mask = (k0 + PF_BN > pos0 + q_row0 + 1) || (k0 + PF_BN > total) || (window > 0);
        float mx = NEG_INF;
        if (need_mask) {                 // the same for the whole wave: one branch, two bodies
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = k0 + sub * 32 + 8 * (i >> 2) + 4 * half + (i & 3);
                    const bool ok = key <= qp && key < total && (window <= 0 || key > qp - window);
                    const float v = ok ? s[sub][i] * scale_log2 : NEG_INF;
                    s[sub][i] = v;
                    mx = fmaxf(mx, v);
                }
        } else {
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float v = s[sub][i] * scale_log2;
                    s[sub][i] = v;
                    mx = fmaxf(mx, v);
                }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, ILLM_WAVE));
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == NEG_INF) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m - m_use);
        float rs = 0.f;
        uint4 pb[2][2];
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            float p[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                p[i] = __builtin_amdgcn_exp2f(s[sub][i] - m_use);
                rs += p[i];
            }
#pragma unroll
            for (int mf = 0; mf < 2; ++mf) {
                pb[sub][mf].x = pack_bf16x2(p[8 * mf + 0], p[8 * mf + 1]);
                pb[sub][mf].y = pack_bf16x2(p[8 * mf + 2], p[8 * mf + 3]);
                pb[sub][mf].z = pack_bf16x2(p[8 * mf + 4], p[8 * mf + 5]);
                pb[sub][mf].w = pack_bf16x2(p[8 * mf + 6], p[8 * mf + 7]);
            }
        }
        l = l * alpha + rs;
        m = m_new;
        if (__any(alpha != 1.f)) {          // the running max moved for some query of the wave
#pragma unroll
            for (int d = 0; d < DB; ++d)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[d][i] *= alpha;
        }
        // O^T[d][q] += V^T[d][keys] . P^T[keys][q]
#pragma unroll
        for (int d = 0; d < DB; ++d) {
            const bf16_t* vp = vts + (d * 32 + lq) * VLD + 4 * half;
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int mf = 0; mf < 2; ++mf) {
                    const uint2 lo = *(const uint2*)(vp + sub * 32 + 16 * mf);
                    const uint2 hi = *(const uint2*)(vp + sub * 32 + 16 * mf + 8);
                    const uint4 a = make_uint4(lo.x, lo.y, hi.x, hi.y);
                    o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&a,
                                                                   *(const bf16x8_t*)&pb[sub][mf],
                                                                   o[d], 0, 0, 0);
                }
        }
    }
    l += __shfl_xor(l, 32, ILLM_WAVE);
    if (q < len) {
        const float inv = 1.0f / l;
        bf16_t* op = out + (size_t)(start + q) * nh * HD + (size_t)h * HD + 4 * half;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) {
                if (d * 32 + 8 * b4 >= HD) continue;
                uint2 v;
                v.x = pack_bf16x2(o[d][4 * b4 + 0] * inv, o[d][4 * b4 + 1] * inv);
                v.y = pack_bf16x2(o[d][4 * b4 + 2] * inv, o[d][4 * b4 + 3] * inv);
                *(uint2*)(op + d * 32 + 8 * b4) = v;
            }
    }
}

// The same for head sizes up to 128 with two LDS buffers and one barrier a tile: while a tile is
// multiplied the next one, already in registers, is written to the other buffer and the one
// after it is asked for.  It keeps the vector instructions beside the products few: K and V^T
// rows are padded and the loop is unrolled over the two buffers, so every LDS address is a
// register fixed for the whole kernel plus an immediate offset; the tile's K and V rows are read
// at per-thread byte offsets, fixed as well, from a base that moves with the tile (scalar
// arithmetic), clamped only in a sequence's last tile; V is transposed in registers, 4 keys x 8
// dims a thread, with one byte permute a pair, and written as 8-byte runs of 4 keys; within a
// tile of 64 keys the runs are placed in the order in which the first product leaves the scores
// of a lane (keys 16 m + 4 h + {0..3} and + 8 + {0..3} for half-wave h), so that the A operand of
// the second product is one 16-byte read.  Two buffers of padded rows are 70 KB at head size 128
// (two blocks a compute unit fit in its 160 KB).
template <int B>
struct PfBuf {
    static constexpr int v = B;
};

template <int HD, bool PAGED>
__global__ void __launch_bounds__(256, 2)
attn_prefill_mfma2_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ out,
                          const int32_t* __restrict__ cu, int n_qblk, int nh, int nkv,
                          float scale_log2, int window, int hb_per_xcd, int n_hb, int zigzag,
                          PfPages pg) {
    constexpr int KS = HD / 16;        // k-steps of the first product
    constexpr int DB = HD / 32;        // 32-row blocks of O^T
    constexpr int UK = HD / 8;         // 16-byte units in a K row
    constexpr int KLD = HD + 8;        // K row stride: 16 bytes of padding
    constexpr int VLD = PF_BN + 8;     // V^T row stride
    constexpr int K_TILE = PF_BN * KLD;
    constexpr int BUF = K_TILE + HD * VLD;         // elements of a buffer: K, then V^T
    constexpr int NLD = (PF_BN * UK) / 256;        // K units a thread (HD / 32)
    extern __shared__ __attribute__((aligned(16))) bf16_t pf_lds[];

    const int xcd = blockIdx.x % 8, slot_id = blockIdx.x / 8;
    const int hb = xcd * hb_per_xcd + slot_id % hb_per_xcd;
    if (hb >= n_hb) return;
    const int qi = slot_id / hb_per_xcd, top = zigzag ? (n_qblk + 1) / 2 : n_qblk;
    const int qb = qi < top ? n_qblk - 1 - qi : qi - top;
    const int h = hb % nh, b = hb / nh;
    const int start = cu[b], len = cu[b + 1] - start;
    const int q0 = qb * PF_BM;
    if (q0 >= len) return;
    // PAGED: the rows stand at positions pos0 .. and see the keys 0 .. of the sequence's cache
    const int slot = PAGED ? pg.seq_slot[b] : 0;
    const int pos0 = PAGED ? pg.seq_start[b] : 0;
    const int total = pos0 + len;                       // keys of the sequence after this step
    const int kvh = h / (nh / nkv);
    const size_t rowlen = (size_t)(nh + 2 * nkv) * HD;
    const uint32_t row_bytes = PAGED ? (uint32_t)(HD * 2) : (uint32_t)(rowlen * 2);   // of a key's row
    const int tid = threadIdx.x, wave = wave_index(), lane = tid & 63;
    const int lq = lane & 31, half = lane >> 5;
    const int q_row0 = q0 + wave * 32;
    const int q = q_row0 + lq;                          // row within the sequence's rows
    const int qc = q < len ? q : len - 1;
    const int qp = pos0 + q;                            // its position

    illm_u32x4_t qf[KS];
    {
        const bf16_t* qp = qkv + (size_t)(start + qc) * rowlen + (size_t)h * HD + half * 8;
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = *(const illm_u32x4_t*)(qp + s * 16);
    }
    // Q is asked for before the first tile and stays there (a scheduling barrier): the wait for
    // that tile then covers Q, and the loop's products wait for no load.  Asked for later, every
    // round's first product would wait for the tile after next, which is on its way by then.
    __builtin_amdgcn_sched_barrier(0);
    f32x16_t o[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[d][i] = 0.f;
    float m = NEG_INF, l = 0.f;

    const int k_end = min(total, pos0 + q0 + PF_BM);
    int k_begin = window > 0 ? max(0, pos0 + q0 - window + 1) : 0;
    k_begin = (k_begin / PF_BN) * PF_BN;
    const int wk_end = min(total, pos0 + q_row0 + 32);              // this wave's last key + 1
    const int wk_begin = window > 0 ? max(0, pos0 + q_row0 - window + 1) : 0;

    // Staging.  K: this thread brings chunks chq + 4 it (it < NLD) of key `skey`.  V: keys
    // 4 g .. 4 g + 3, dims 8 c .. 8 c + 7 (threads with c >= UK, at head sizes below 128, bring
    // chunk UK - 1 again and write nothing).
    const int skey = ((tid >> 6) & 3) * 16 + (tid & 15), chq = (tid >> 4) & 3;
    const int vc = (tid >> 4) < UK ? (tid >> 4) : UK - 1, vg = tid & 15;
    const bool v_writes = (tid >> 4) < UK;
    // where the group's 4 keys go in the row of 64, so that the second product's operand, a
    // lane's 8 keys in the order in which the first product leaves them, is one 16-byte read:
    // bits (sub, sub, m, a, h) -> (.., h, a)
    const int vpg = (vg & 12) | ((vg & 1) << 1) | ((vg >> 1) & 1);
    // (not PAGED: the keys are the step's own rows; PAGED: a tile of 64 keys is a page or an
    // aligned part of one, found through the page table when the tile is asked for)
    const char* const kg = (const char*)(qkv + (size_t)start * rowlen + (size_t)(nh + kvh) * HD);
    const char* const vg_base = (const char*)(qkv + (size_t)start * rowlen + (size_t)(nh + nkv + kvh) * HD);
    const uint32_t koff_whole = (uint32_t)skey * row_bytes + chq * 16;
    const uint32_t voff_whole = (uint32_t)(4 * vg) * row_bytes + vc * 16;
    bf16_t* const kw = pf_lds + skey * KLD + chq * 8;                 // + it * 32
    bf16_t* const vw = pf_lds + K_TILE + (8 * vc) * VLD + vpg * 4;    // + dim * VLD
    const bf16_t* const kr = pf_lds + lq * KLD + half * 8;            // + sub * 32 * KLD + st * 16
    const bf16_t* const vr = pf_lds + K_TILE + lq * VLD + half * 8;   // + d * 32 * VLD + (sub * 4 + mf * 2) * 8

    illm_u32x4_t kpre[NLD], vpre0, vpre1, vpre2, vpre3;
    auto fetch = [&](int k0) __attribute__((always_inline)) {
        uint32_t ko = koff_whole, v0 = voff_whole, v1 = voff_whole + row_bytes,
                 v2 = voff_whole + 2 * row_bytes, v3 = voff_whole + 3 * row_bytes;
        if (k0 + PF_BN > total) {                  // the sequence's last tile: rows clamped
            const int last = total - 1 - k0;
            ko = (uint32_t)min(skey, last) * row_bytes + chq * 16;
            v0 = (uint32_t)min(4 * vg + 0, last) * row_bytes + vc * 16;
            v1 = (uint32_t)min(4 * vg + 1, last) * row_bytes + vc * 16;
            v2 = (uint32_t)min(4 * vg + 2, last) * row_bytes + vc * 16;
            v3 = (uint32_t)min(4 * vg + 3, last) * row_bytes + vc * 16;
        }
        const char* kt;
        const char* vt;
        if (PAGED) {
            int lp = k0 / pg.page_size;
            if (pg.ring > 0) lp %= pg.ring;
            const int phys = pg.page_table[(size_t)slot * pg.table_stride + lp];
            const size_t at = (((size_t)phys * nkv + kvh) * pg.page_size + k0 % pg.page_size) * (size_t)(HD * 2);
            kt = (const char*)pg.kcache + at;
            vt = (const char*)pg.vcache + at;
        } else {
            kt = kg + (size_t)k0 * row_bytes;
            vt = vg_base + (size_t)k0 * row_bytes;
        }
#pragma unroll
        for (int it = 0; it < NLD; ++it) kpre[it] = *(const illm_u32x4_t*)(kt + ko + it * 64);
        vpre0 = *(const illm_u32x4_t*)(vt + v0);
        vpre1 = *(const illm_u32x4_t*)(vt + v1);
        vpre2 = *(const illm_u32x4_t*)(vt + v2);
        vpre3 = *(const illm_u32x4_t*)(vt + v3);
    };
    auto stage = [&](auto bc) __attribute__((always_inline)) {
        constexpr int off = decltype(bc)::v * BUF;
#pragma unroll
        for (int it = 0; it < NLD; ++it) *(illm_u32x4_t*)(kw + off + it * 32) = kpre[it];
        if (v_writes) {
#pragma unroll
            for (int dp = 0; dp < 4; ++dp) {                 // dims 2 dp and 2 dp + 1 of the chunk
                const uint32_t a0 = vpre0[dp], a1 = vpre1[dp], a2 = vpre2[dp], a3 = vpre3[dp];
                uint2 even, odd;
                even.x = __builtin_amdgcn_perm(a1, a0, 0x05040100u);
                even.y = __builtin_amdgcn_perm(a3, a2, 0x05040100u);
                odd.x = __builtin_amdgcn_perm(a1, a0, 0x07060302u);
                odd.y = __builtin_amdgcn_perm(a3, a2, 0x07060302u);
                *(uint2*)(vw + off + (2 * dp) * VLD) = even;
                *(uint2*)(vw + off + (2 * dp + 1) * VLD) = odd;
            }
        }
    };
    // One tile of 64 keys at k0 from buffer B; then the next tile, already in registers, goes
    // into the other buffer and the one after it is asked for.
    auto tile = [&](auto bc, int k0) __attribute__((always_inline)) {
        constexpr int B = decltype(bc)::v;
        if (k0 < wk_end && k0 + PF_BN > wk_begin) {                 // something visible to this wave
            const bf16_t* kb = kr + B * BUF;
            const bf16_t* vb = vr + B * BUF;
            // S^T[key][q] for two sub-tiles of 32 keys (their sums alternate, so that no product
            // waits for the one before it)
            f32x16_t s[2];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[sub][i] = 0.f;
#pragma unroll
            for (int st = 0; st < KS; ++st)
#pragma unroll
                for (int sub = 0; sub < 2; ++sub) {
                    const illm_u32x4_t a = *(const illm_u32x4_t*)(kb + sub * 32 * KLD + st * 16);
                    s[sub] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&a,
                                                                     *(const bf16x8_t*)&qf[st],
                                                                     s[sub], 0, 0, 0);
                }
            const bool need_mask = (k0 + PF_BN > pos0 + q_row0 + 1) || (k0 + PF_BN > total) || (window > 0);
            float mx = NEG_INF;
            if (need_mask) {                 // the same for the whole wave: one branch, two bodies
#pragma unroll
                for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int key = k0 + sub * 32 + 8 * (i >> 2) + 4 * half + (i & 3);
                        const bool ok = key <= qp && key < total && (window <= 0 || key > qp - window);
                        const float v = ok ? s[sub][i] : NEG_INF;
                        s[sub][i] = v;
                        mx = fmaxf(mx, v);
                    }
            } else {
#pragma unroll
                for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[sub][i]);
            }
            // The reference point of the exponentials (in scaled units: the scale is positive and
            // is applied inside the exponential's argument, one multiply-add a score) follows the
            // running max only when that has grown by more than 8, a factor of 256: until then
            // the weights are at most 256, which float32 sums and bfloat16 weights hold as well
            // as weights up to 1, and the sums need no rescaling (with random scores some query
            // of a wave has a new max in most tiles: 64 multiplications a lane).  The division
            // by the sum of the weights at the end makes the result the same.
            mx = fmaxf(mx, __shfl_xor(mx, 32, ILLM_WAVE)) * scale_log2;
            const float m_new = (mx > m + 8.0f || m == NEG_INF) ? fmaxf(m, mx) : m;
            const float m_use = (m_new == NEG_INF) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m - m_use);
            float rs = 0.f;
            illm_u32x4_t pb[2][2];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                float p[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    p[i] = __builtin_amdgcn_exp2f(fmaf(s[sub][i], scale_log2, -m_use));
                    rs += p[i];
                }
#pragma unroll
                for (int mf = 0; mf < 2; ++mf)
#pragma unroll
                    for (int w = 0; w < 4; ++w)
                        pb[sub][mf][w] = pack_bf16x2(p[8 * mf + 2 * w], p[8 * mf + 2 * w + 1]);
            }
            l = l * alpha + rs;
            m = m_new;
            if (__any(alpha != 1.f)) {          // the reference moved for some query of the wave
#pragma unroll
                for (int d = 0; d < DB; ++d)
#pragma unroll
                    for (int i = 0; i < 16; ++i) o[d][i] *= alpha;
            }
            // O^T[d][q] += V^T[d][keys] . P^T[keys][q]: 8 keys of a lane are one 16-byte unit
            // (the blocks of dims innermost: consecutive products add to different sums)
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int mf = 0; mf < 2; ++mf)
#pragma unroll
                    for (int d = 0; d < DB; ++d) {
                        const illm_u32x4_t a =
                            *(const illm_u32x4_t*)(vb + d * 32 * VLD + (sub * 4 + mf * 2) * 8);
                        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&a,
                                                                       *(const bf16x8_t*)&pb[sub][mf],
                                                                       o[d], 0, 0, 0);
                    }
        }
        if (k0 + PF_BN < k_end) {
            stage(PfBuf<1 - B>{});
            if (k0 + 2 * PF_BN < k_end) fetch(k0 + 2 * PF_BN);
        }
        __syncthreads();
    };

    // (k_begin <= q0 < k_end: there is a first tile.  Were this under a condition, the loop's
    // wait counts would provide for a way in on which Q has not arrived.)
    fetch(k_begin);
    __builtin_amdgcn_sched_barrier(0);
    stage(PfBuf<0>{});
    if (k_begin + PF_BN < k_end) fetch(k_begin + PF_BN);
    __syncthreads();
    for (int k0 = k_begin; k0 < k_end; k0 += 2 * PF_BN) {
        tile(PfBuf<0>{}, k0);
        if (k0 + PF_BN >= k_end) break;
        tile(PfBuf<1>{}, k0 + PF_BN);
    }
    l += __shfl_xor(l, 32, ILLM_WAVE);
    if (q < len) {
        const float inv = 1.0f / l;
        bf16_t* op = out + (size_t)(start + q) * nh * HD + (size_t)h * HD + 4 * half;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) {
                uint2 v;
                v.x = pack_bf16x2(o[d][4 * b4 + 0] * inv, o[d][4 * b4 + 1] * inv);
                v.y = pack_bf16x2(o[d][4 * b4 + 2] * inv, o[d][4 * b4 + 3] * inv);
                *(uint2*)(op + d * 32 + 8 * b4) = v;
            }
    }
}

// Tuning and tests: 0 sends head sizes up to 128 to the kernel with one LDS buffer always, 2 to the
// one with two buffers always (the scale must be positive); 1 (default): two buffers for head
// sizes 64 to 128 and sequences of 1,024 keys or more.
static int PF_TWO_BUFFERS = 1;
extern "C" void illm_set_prefill_two_buffers(int on) { PF_TWO_BUFFERS = on; }

// The two-buffer kernel needs more LDS than a kernel may have without asking: asked for once per
// device and head size.
template <int HD, bool PAGED>
static int prefill2_lds_ready(size_t bytes) {
    static bool ready[64] = {};
    static std::mutex lock;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return ILLM_ERR_LAUNCH;
    std::lock_guard<std::mutex> hold(lock);
    if (!ready[dev]) {
        if (hipFuncSetAttribute((const void*)attn_prefill_mfma2_kernel<HD, PAGED>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
            return ILLM_ERR_LAUNCH;
        ready[dev] = true;
    }
    return ILLM_OK;
}


template <int HD>
static int launch_prefill(const void* qkv, void* out, const int32_t* cu, int n_seqs, int max_len,
                          int nh, int nkv, float scale, int window, hipStream_t st,
                          const PfPages* pg = nullptr) {
    const int n_qblk = (max_len + PF_BM - 1) / PF_BM;
    const long long n_hb = (long long)nh * n_seqs;
    const long long hb_per_xcd = (n_hb + 7) / 8;
    const long long blocks = 8 * hb_per_xcd * n_qblk;
    if (blocks > 0x7fffffffLL) return ILLM_ERR_ARG;
    if constexpr (HD <= 128 && HD % 32 == 0) {
        // measured at 32 heads of size 128: 2,048 keys 81 -> 71 us, 4,096 keys 228 -> 193, 8,192
        // keys (8 groups) 704 -> 615; size 64, 2,048 keys 46.7 -> 42.7; four sequences of 1,024
        // 66 -> 64; eight of 512 lose (45 -> 48: a tile more of set-up before the first product).
        // (steps that go on from the cache: `max_len` is the most rows a sequence brings, which
        // see at least as many keys)
        if (PF_TWO_BUFFERS == 2 || (PF_TWO_BUFFERS == 1 && HD >= 64 && max_len >= 1024 && scale > 0.f)) {
            const size_t lds = (size_t)2 * (PF_BN * (HD + 8) + HD * (PF_BN + 8)) * sizeof(bf16_t);
            const int rc = pg ? prefill2_lds_ready<HD, true>(lds) : prefill2_lds_ready<HD, false>(lds);
            if (rc != ILLM_OK) return rc;
            if (pg)
                hipLaunchKernelGGL((attn_prefill_mfma2_kernel<HD, true>), dim3((unsigned)blocks), dim3(256), lds,
                                   st, (const bf16_t*)qkv, (bf16_t*)out, cu, n_qblk, nh, nkv,
                                   scale * 1.44269504088896340736f, window, (int)hb_per_xcd, (int)n_hb,
                                   hb_per_xcd * n_qblk <= 64 ? 1 : 0, *pg);
            else
                hipLaunchKernelGGL((attn_prefill_mfma2_kernel<HD, false>), dim3((unsigned)blocks), dim3(256), lds,
                                   st, (const bf16_t*)qkv, (bf16_t*)out, cu, n_qblk, nh, nkv,
                                   scale * 1.44269504088896340736f, window, (int)hb_per_xcd, (int)n_hb,
                                   hb_per_xcd * n_qblk <= 64 ? 1 : 0, PfPages());
            return illm_launch_status();
        }
    }
    if (pg) {
        hipLaunchKernelGGL((attn_prefill_mfma_kernel<HD, true>), dim3((unsigned)blocks), dim3(256), 0,
                           st, (const bf16_t*)qkv, (bf16_t*)out, cu, n_qblk, nh, nkv,
                           scale * 1.44269504088896340736f, window, (int)hb_per_xcd, (int)n_hb,
                           hb_per_xcd * n_qblk <= 64 ? 1 : 0, *pg);
        return illm_launch_status();
    }
    hipLaunchKernelGGL((attn_prefill_mfma_kernel<HD, false>), dim3((unsigned)blocks), dim3(256), 0, st,
                       (const bf16_t*)qkv, (bf16_t*)out, cu, n_qblk, nh, nkv,
                       scale * 1.44269504088896340736f, window, (int)hb_per_xcd, (int)n_hb,
                       hb_per_xcd * n_qblk <= 64 ? 1 : 0, PfPages());   // 32 CUs of an XCD, two blocks each
    return illm_launch_status();
}

// Takes bfloat16 and a head_dim that is a multiple of 16 up to 256; else ILLM_ERR_ARG.
extern "C" int illm_attn_prefill_bf16(const void* qkv, void* out, const int32_t* cu_seqlens,
                                      int n_seqs, int max_len, int nh, int nkv, int hd,
                                      float scale, int window, void* stream) {
    if (n_seqs < 0 || max_len < 0 || nh <= 0 || nkv <= 0 || nh % nkv || hd <= 0 || hd > 256 ||
        hd % 16)
        return ILLM_ERR_ARG;
    if (n_seqs == 0 || max_len == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
    switch (hd) {
        case 32: return launch_prefill<32>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 64: return launch_prefill<64>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 96: return launch_prefill<96>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 128: return launch_prefill<128>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 160: return launch_prefill<160>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 192: return launch_prefill<192>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 224: return launch_prefill<224>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 16: return launch_prefill<16>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 48: return launch_prefill<48>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 80: return launch_prefill<80>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 112: return launch_prefill<112>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 144: return launch_prefill<144>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 176: return launch_prefill<176>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 208: return launch_prefill<208>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        case 240: return launch_prefill<240>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
        default: return launch_prefill<256>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st);
    }
}

// The same where the step's rows go on from tokens the cache already holds: keys and values from
// the paged cache (bfloat16, pages of a multiple of 64 rows), row r of sequence b at position
// seq_start[b] + r.  The step's own keys and values must be in the cache already.
extern "C" int illm_attn_prefill_paged_bf16(const void* qkv, void* out, const int32_t* cu_seqlens,
                                            const int32_t* seq_slot, const int32_t* seq_start,
                                            const void* kcache, const void* vcache,
                                            const int32_t* page_table, int table_stride,
                                            int page_size, int ring, int n_seqs, int max_len, int nh,
                                            int nkv, int hd, float scale, int window, void* stream) {
    if (n_seqs < 0 || max_len < 0 || nh <= 0 || nkv <= 0 || nh % nkv || hd <= 0 || hd > 256 ||
        hd % 16 || !seq_slot || !seq_start || !kcache || !vcache || !page_table ||
        table_stride <= 0 || page_size <= 0 || page_size % PF_BN)
        return ILLM_ERR_ARG;
    if (n_seqs == 0 || max_len == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
    const PfPages pg = {(const bf16_t*)kcache, (const bf16_t*)vcache, page_table, seq_slot, seq_start,
                        table_stride, page_size, ring};
    switch (hd) {
        case 32: return launch_prefill<32>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 64: return launch_prefill<64>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 96: return launch_prefill<96>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 128: return launch_prefill<128>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 160: return launch_prefill<160>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 192: return launch_prefill<192>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 224: return launch_prefill<224>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 16: return launch_prefill<16>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 48: return launch_prefill<48>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 80: return launch_prefill<80>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 112: return launch_prefill<112>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 144: return launch_prefill<144>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 176: return launch_prefill<176>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 208: return launch_prefill<208>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        case 240: return launch_prefill<240>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
        default: return launch_prefill<256>(qkv, out, cu_seqlens, n_seqs, max_len, nh, nkv, scale, window, st, &pg);
    }
}

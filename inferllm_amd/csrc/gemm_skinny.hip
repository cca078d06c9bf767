// Y[M, N] = X[M, K] . W[N, K]^T for few rows (M <= 64, decoding), bfloat16 operands,
// float32 accumulation on the matrix cores.  The product is bound by reading W once.
//
// MFMA 16x16x32: the A operand is a 16-row tile of W, the B operand 16 rows of X.
// Lane (r = lane % 16, q = lane / 16) needs 8 consecutive k of row r at k0 + 8 q.
// X is read like that straight from global memory (it is small and stays in cache).
// W is used once and is read as a stream: non-temporal loads of whole 128-byte
// lines (8 lanes a row), put into operand order through a wave-private piece of
// LDS.  Reading W in operand order directly (64 bytes of 16 rows per instruction)
// measured 4.7 TB/s on a 180 MB matrix, whole lines 6.5 TB/s.  A wave owns NTB
// tiles of 16 W rows and all MT tiles of 16 X rows.  The waves of a block split K
// in interleaved pieces of U k-steps (U * 64 bytes of each W row at a time) and
// add their results through LDS in wave order, so the sum has a fixed order.
// Lanes of X rows >= M read row M - 1 and their results are dropped.
//
// The reference calls cublasSgemm with M = 1 here (src/kern/gpu/kernel_gpu.cu:420-435).
#include "api.h"
#include "api_test.h"
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// U: k-steps (of 32) per wave iteration, i.e. U * 64 contiguous bytes of each W row.
// MAXW: most waves a block may have (register budget: 512 / (MAXW / 4) per lane).
// What a block's tiles are and what happens to the sums:
//   SK_PLAIN     NTB consecutive tiles of 16 rows of W; Y = sums.
//   SK_GATE_UP   (NTB == 1) W is [gate rows (N) | up rows (N)]; the tile is 8 gate rows and the
//                same 8 up rows and Y[M, N] = silu(gate) * up.
//   SK_QKV_ROPE  (NTB == 1) W is [q heads | k heads | v heads]; the tile of a block of a q or k head
//                is 8 rows and their 8 rotation partners (hd/2 further); the block rotates the
//                pairs by the row's position and writes q to Y and k to the paged cache; a block
//                of a v head takes 16 consecutive rows and writes them to the cache.
enum { SK_PLAIN = 0, SK_GATE_UP = 1, SK_QKV_ROPE = 2 };

struct SkRope {
    const float* cos_sin;        // [max_pos][hd/2][2]
    const int32_t* row_pos;      // [M]
    const int32_t* row_slot;     // [M]
    bf16_t* kcache;
    bf16_t* vcache;
    const int32_t* page_table;
    int table_stride, page_size, ring, nh, nkv, hd;
};

// The residual add and the RMS norm between two products of few rows, without kernels of their
// own (M <= 16).  The producing product (SK_PLAIN, float32 Y) adds its result to the residual
// rows Y; if `nw` is given it also leaves xb = bfloat16(y * nw), the next product's operand up to
// the row's scale, and the sum of y^2 over its 16 columns in ssq[m][its block].  The consuming
// product gets xb as X and `ssq`: every result of row m is scaled by
// 1 / sqrt(sum_p ssq[m][p] / K + eps), which is the row's norm since the scale is common to all k.
struct SkResidual {
    int accumulate;              // producer: Y += product
    const void* nw;              // producer: norm weight [N] (bfloat16 or float32) or null
    int nw_dt;
    bf16_t* xb;                  // producer: [M, N]
    float* ssq_out;              // producer: [M, gridDim.x]
    const float* ssq;            // consumer: [M, parts] or null
    int parts;
    float eps;
};

// TILED (NTB == 1, K % 32 == 0): W is a copy laid out for this kernel, [tile][k-step][16 rows][32 k]
// with tile = blockIdx.x holding the 16 rows that block works on (in its mode's order): a load
// instruction then reads 1 KB that is contiguous and already in operand order, so the lines need
// no reordering in LDS.  Measured at the 7B shapes: 6 to 17 % less time than from row-major W.
// ONE_SHOT: a wave asks for its whole share of K at once and holds no second piece (for K that
// the block's waves cover in one piece each: the product of a short K is bound by the round
// trips of a wave's pieces, not by bandwidth).
template <int MT, int NTB, int SK_U, int MAXW, int MODE, bool TILED, bool ONE_SHOT = false>
__global__ void __launch_bounds__(64 * MAXW)
gemm_skinny_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                   void* __restrict__ Y, int y_dt, int M, int N, int K, SkRope rope,
                   SkResidual res) {
    constexpr bool DUAL = MODE == SK_GATE_UP;
    // a wave's piece of LDS: first the staging of its W lines (NTB * SK_U KB, not TILED), then
    // its sums
    constexpr int SK_REGION_FLOATS = NTB * ((!TILED && SK_U > MT) ? SK_U : MT) * 256;
    extern __shared__ float red[];   // [waves][SK_REGION_FLOATS]
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int waves = blockDim.x >> 6;
    const int r = lane & 15, q = lane >> 4;
    // consumer: the last wave, which has the fewest pieces of K if they do not divide evenly, adds
    // up the rows' sums of squares (a row's parts as one load of the whole wave) while the others
    // already stream W; the scales wait in LDS for the end
    float* row_rs = red + (size_t)waves * SK_REGION_FLOATS;      // [16]
    if (res.ssq && wave == waves - 1) {
        // all rows' loads are asked for at once; then 16 sums over the wave in one halving
        // exchange (a lane keeps the rows that share its bit), after which lane m has row m's
        float t[16];
#pragma unroll
        for (int m = 0; m < 16; ++m) t[m] = 0.f;
        const bool by4 = (res.parts & 3) == 0;
        for (int p = lane * 4; p < res.parts; p += 256) {
            float4 v[16];
#pragma unroll
            for (int m = 0; m < 16; ++m) {
                v[m] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (m < M) {
                    const float* at = res.ssq + (size_t)m * res.parts + p;
                    if (by4) {
                        v[m] = *(const float4*)at;
                    } else {
                        v[m].x = at[0];
                        if (p + 1 < res.parts) v[m].y = at[1];
                        if (p + 2 < res.parts) v[m].z = at[2];
                        if (p + 3 < res.parts) v[m].w = at[3];
                    }
                }
            }
#pragma unroll
            for (int m = 0; m < 16; ++m) t[m] += (v[m].x + v[m].y) + (v[m].z + v[m].w);
        }
#pragma unroll
        for (int b = 1, n = 8; b < 16; b <<= 1, n >>= 1) {
            const bool up = (lane & b) != 0;
#pragma unroll
            for (int k = 0; k < n; ++k) {
                const float keep = up ? t[2 * k + 1] : t[2 * k];
                const float send = up ? t[2 * k] : t[2 * k + 1];
                t[k] = keep + __shfl_xor(send, b, ILLM_WAVE);
            }
        }
        float tot = t[0];
        tot += __shfl_xor(tot, 16, ILLM_WAVE);
        tot += __shfl_xor(tot, 32, ILLM_WAVE);
        if (lane < 16) row_rs[lane] = 1.0f / sqrtf(tot / (float)K + res.eps);
    }
    const int n_base = blockIdx.x * (DUAL ? 8 * NTB : 16 * NTB);
    int tile_row[NTB];           // SK_PLAIN: first W row of each of the block's tiles
#pragma unroll
    for (int nt = 0; nt < NTB; ++nt) tile_row[nt] = n_base + nt * 16;
    // the other modes (NTB == 1): the first 8 rows of the tile and the second 8 are apart (a load
    // instruction reads 8 rows)
    int rot_head = -1, rot_j = 0, row_lo = 0, row_hi = 0;
    if (DUAL) {
        row_lo = n_base;
        row_hi = N + n_base;
    }
    if (MODE == SK_QKV_ROPE) {
        const int tph = rope.hd / 16, n_rot = (rope.nh + rope.nkv) * tph;
        if ((int)blockIdx.x < n_rot) {
            rot_head = blockIdx.x / tph;
            rot_j = blockIdx.x % tph;
            row_lo = rot_head * rope.hd + 8 * rot_j;
            row_hi = row_lo + rope.hd / 2;
        } else {
            row_lo = (rope.nh + rope.nkv) * rope.hd + 16 * ((int)blockIdx.x - n_rot);
            row_hi = row_lo + 8;
        }
    }

    // producer: the threads that will add to the residual rows fetch their 4 values and the norm
    // weights now, so that they arrive while W is streamed
    float pre_y[4] = {0.f, 0.f, 0.f, 0.f}, pre_nw[4] = {0.f, 0.f, 0.f, 0.f};
    if (MODE == SK_PLAIN && res.accumulate && threadIdx.x < 64 && (int)(threadIdx.x & 15) < M) {
        const int n0 = tile_row[0] + (threadIdx.x >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n0 + i < N) {
                pre_y[i] = ((const float*)Y)[(size_t)(threadIdx.x & 15) * N + n0 + i];
                if (res.nw) pre_nw[i] = ld_f(res.nw, res.nw_dt, n0 + i);
            }
    }

    // SK_QKV_ROPE: the threads that will write the results fetch what that needs (position,
    // angles, the cache row's address) now, so that it arrives while W is streamed
    float pre_cs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    size_t pre_off = 0;
    if (MODE == SK_QKV_ROPE && threadIdx.x < 64 && (int)(threadIdx.x & 15) < M) {
        const int mrow = threadIdx.x & 15, ro = (threadIdx.x >> 4) * 4;
        const int pos = rope.row_pos[mrow], slot = rope.row_slot[mrow];
        if (rot_head >= 0) {
            if (ro < 8) {
                const float4* cs =
                    (const float4*)(rope.cos_sin + (size_t)pos * rope.hd + 2 * (8 * rot_j + ro));
                const float4 c0 = cs[0], c1 = cs[1];
                pre_cs[0] = c0.x; pre_cs[1] = c0.y; pre_cs[2] = c0.z; pre_cs[3] = c0.w;
                pre_cs[4] = c1.x; pre_cs[5] = c1.y; pre_cs[6] = c1.z; pre_cs[7] = c1.w;
                if (rot_head >= rope.nh)
                    pre_off = cache_row_offset(rope.page_table, rope.table_stride, slot, pos,
                                               rope.page_size, rope.ring, rope.nkv,
                                               rot_head - rope.nh, rope.hd) + 8 * rot_j + ro;
            }
        } else {
            const int vrow = row_lo - (rope.nh + rope.nkv) * rope.hd;
            pre_off = cache_row_offset(rope.page_table, rope.table_stride, slot, pos, rope.page_size,
                                       rope.ring, rope.nkv, vrow / rope.hd, rope.hd) + vrow % rope.hd + ro;
        }
    }

    // W is read in whole 128-byte lines: one load instruction takes 64 k of 8 rows (8 lanes a
    // row), two of them the 16 rows of a tile.  `wline[nt][h]` is this lane's row of half h.
    const bf16_t* wline[NTB][2];
#pragma unroll
    for (int nt = 0; nt < NTB; ++nt)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int n = tile_row[nt] + (lane >> 3) + 8 * h;
            if (MODE != SK_PLAIN) n = (h ? row_hi : row_lo) + (DUAL ? 8 * nt : 0) + (lane >> 3);
            const int last = DUAL ? (h + 1) * N - 1 : N - 1;
            n = n < last ? n : last;
            wline[nt][h] = W + (size_t)n * K;
        }
    const bf16_t* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int mm = mt * 16 + r;
        mm = mm < M ? mm : M - 1;
        xrow[mt] = X + (size_t)mm * K;
    }
    f32x4_t acc[NTB][MT];
#pragma unroll
    for (int nt = 0; nt < NTB; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

    // The matrix cores want lane (r, q) to hold k-chunk q of row r, so the lines go through this
    // wave's own piece of LDS: written as loaded (lane = 8 * row + chunk, contiguous), read back
    // in operand order.  Chunks are swizzled within their row by (row / 2) % 8 so that both
    // directions are free of bank conflicts.  Only this wave touches the piece: the LDS unit
    // handles a wave's accesses in order, no barrier is needed.
    uint4* stage = (uint4*)red + (size_t)wave * (SK_REGION_FLOATS / 4);
    const int w_row = lane >> 3, w_chunk = lane & 7;
    // TILED: this lane's 8 values of k-step 0 of the block's first tile; a last block may have
    // fewer than NTB tiles (SK_GATE_UP with NTB > 1)
    const bf16_t* wtile = W + (size_t)blockIdx.x * NTB * ((K + 31) / 32) * 512 + (r * 4 + q) * 8;
    bool tile_ok[NTB];
#pragma unroll
    for (int nt = 0; nt < NTB; ++nt) tile_ok[nt] = DUAL ? n_base + 8 * nt < N : tile_row[nt] < N || MODE != SK_PLAIN;

    const int ksteps = (K + 31) / 32;
    const int stride = waves * SK_U;
    uint4 a[NTB][SK_U], b[MT][SK_U];
    auto load = [&](int s0, uint4 (&aa)[NTB][SK_U], uint4 (&bb)[MT][SK_U]) {
#pragma unroll
        for (int u = 0; u < SK_U; ++u) {
            // K is a multiple of 8: a lane's 8 values are all in or all out
            const int kw = (s0 + (u & ~1)) * 32 + w_chunk * 8;
#pragma unroll
            for (int nt = 0; nt < NTB; ++nt) {
                if (TILED)
                    aa[nt][u] = (s0 + u < ksteps && tile_ok[nt])
                                    ? ld16_stream(wtile + ((size_t)nt * ksteps + s0 + u) * 512)
                                    : make_uint4(0, 0, 0, 0);
                else aa[nt][u] = kw < K ? ld16_stream(wline[nt][u & 1] + kw) : make_uint4(0, 0, 0, 0);
            }
            const int k = (s0 + u) * 32 + q * 8;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                bb[mt][u] = k < K ? *(const uint4*)(xrow[mt] + k) : make_uint4(0, 0, 0, 0);
        }
    };
    int s0 = wave * SK_U;
    if (s0 < ksteps) load(s0, a, b);
    for (; s0 < ksteps; s0 += stride) {
        // the next piece is on its way while this one is multiplied
        uint4 an[ONE_SHOT ? 1 : NTB][SK_U], bn[ONE_SHOT ? 1 : MT][SK_U];
        const bool more = !ONE_SHOT && s0 + stride < ksteps;
        if constexpr (ONE_SHOT) {
            if (s0 != wave * SK_U) load(s0, a, b);       // (a K longer than one piece a wave)
        } else {
            if (more) load(s0 + stride, an, bn);
        }
        if (!TILED) {
#pragma unroll
            for (int u = 0; u < SK_U; ++u) {
                const int row = w_row + 8 * (u & 1);
#pragma unroll
                for (int nt = 0; nt < NTB; ++nt)
                    stage[(nt * (SK_U / 2) + (u >> 1)) * 128 + row * 8 +
                          (w_chunk ^ ((row >> 1) & 7))] = a[nt][u];
            }
        }
#pragma unroll
        for (int u = 0; u < SK_U; ++u)
#pragma unroll
            for (int nt = 0; nt < NTB; ++nt) {
                const uint4 am = TILED ? a[nt][u]
                                       : stage[(nt * (SK_U / 2) + (u >> 1)) * 128 + r * 8 +
                                               (((u & 1) * 4 + q) ^ ((r >> 1) & 7))];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        *(const bf16x8_t*)&am, *(bf16x8_t*)&b[mt][u], acc[nt][mt], 0, 0, 0);
            }
        if constexpr (!ONE_SHOT) {
            if (more) {
#pragma unroll
                for (int u = 0; u < SK_U; ++u) {
#pragma unroll
                    for (int nt = 0; nt < NTB; ++nt) a[nt][u] = an[nt][u];
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) b[mt][u] = bn[mt][u];
                }
            }
        }
    }
    // acc[nt][mt][i] = Y[m = mt*16 + r][n = n_base + nt*16 + q*4 + i]
    constexpr int PER_WAVE = SK_REGION_FLOATS;
    if (waves > 1 || MODE != SK_PLAIN) {
#pragma unroll
        for (int nt = 0; nt < NTB; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                *(f32x4_t*)(red + (size_t)wave * PER_WAVE + ((nt * MT + mt) * 64 + lane) * 4) =
                    acc[nt][mt];
        __syncthreads();
    }
    // consumer (MT == 1): the scale of X row m16
    auto row_scale = [&](int m16) { return res.ssq ? row_rs[m16] : 1.0f; };
    if (MODE == SK_QKV_ROPE) {
        // NTB == 1, MT == 1: lane (m, g) of the first wave's threads owns rows 4 g .. 4 g + 3 of
        // the tile for X row m; rows 8 .. 15 of a rotated tile are the partners of rows 0 .. 7
        const int mrow = threadIdx.x & 15, ro = (threadIdx.x >> 4) * 4;
        if (threadIdx.x >= 64 || mrow >= M || (rot_head >= 0 && ro >= 8)) return;
        auto total = [&](int l2) {
            f32x4_t t = *(f32x4_t*)(red + l2 * 4);
            for (int w = 1; w < waves; ++w) {
                const f32x4_t o = *(f32x4_t*)(red + (size_t)w * PER_WAVE + l2 * 4);
                t[0] += o[0]; t[1] += o[1]; t[2] += o[2]; t[3] += o[3];
            }
            return t;
        };
        const float rs = row_scale(mrow);
        f32x4_t lo = total(threadIdx.x);
        lo[0] *= rs; lo[1] *= rs; lo[2] *= rs; lo[3] *= rs;
        if (rot_head >= 0) {
            f32x4_t hi = total(threadIdx.x + 32);
            hi[0] *= rs; hi[1] *= rs; hi[2] *= rs; hi[3] *= rs;
            float y0[4], y1[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float c = pre_cs[2 * i], sn = pre_cs[2 * i + 1];
                y0[i] = lo[i] * c - hi[i] * sn;
                y1[i] = lo[i] * sn + hi[i] * c;
            }
            bf16_t* dst = rot_head < rope.nh ? (bf16_t*)Y + (size_t)mrow * N + row_lo + ro
                                             : rope.kcache + pre_off;
            *(uint2*)dst = make_uint2(pack_bf16x2(y0[0], y0[1]), pack_bf16x2(y0[2], y0[3]));
            *(uint2*)(dst + rope.hd / 2) =
                make_uint2(pack_bf16x2(y1[0], y1[1]), pack_bf16x2(y1[2], y1[3]));
        } else {
            *(uint2*)(rope.vcache + pre_off) =
                make_uint2(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]));
        }
        return;
    }
    if (DUAL) {
        // rows 0 .. 7 of a tile are gate rows, rows 8 .. 15 the up rows of the same outputs; a
        // thread takes one X row's 4 outputs of one tile
        for (int grp = threadIdx.x; grp < NTB * MT * 32; grp += blockDim.x) {
            const int l2 = grp & 31, mt = (grp >> 5) % MT, nt = (grp >> 5) / MT;
            const int mrow = mt * 16 + (l2 & 15), n0 = n_base + 8 * nt + (l2 >> 4) * 4;
            if (mrow >= M) continue;
            const int e = ((nt * MT + mt) * 64 + l2) * 4;
            f32x4_t g = *(f32x4_t*)(red + e), u = *(f32x4_t*)(red + e + 128);
            for (int w = 1; w < waves; ++w) {
                const f32x4_t og = *(f32x4_t*)(red + (size_t)w * PER_WAVE + e);
                const f32x4_t ou = *(f32x4_t*)(red + (size_t)w * PER_WAVE + e + 128);
                g[0] += og[0]; g[1] += og[1]; g[2] += og[2]; g[3] += og[3];
                u[0] += ou[0]; u[1] += ou[1]; u[2] += ou[2]; u[3] += ou[3];
            }
            const float rs = row_scale(l2 & 15);
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n0 + i < N) {
                    const float gi = g[i] * rs;
                    st_f(Y, y_dt, (size_t)mrow * N + n0 + i, (gi / (1.0f + expf(-gi))) * (u[i] * rs));
                }
        }
        return;
    }
    // every thread of the block sums some of the (mt, lane) groups over the waves, tile by tile
    for (int grp = threadIdx.x; grp < MT * 64; grp += blockDim.x) {
        const int l2 = grp & 63, mt = grp >> 6;
        f32x4_t v[NTB];
#pragma unroll
        for (int nt = 0; nt < NTB; ++nt) {
            if (waves > 1) {
                const int e = ((nt * MT + mt) * 64 + l2) * 4;
                v[nt] = *(f32x4_t*)(red + e);
                for (int w = 1; w < waves; ++w) {
                    const f32x4_t o = *(f32x4_t*)(red + (size_t)w * PER_WAVE + e);
                    v[nt][0] += o[0]; v[nt][1] += o[1]; v[nt][2] += o[2]; v[nt][3] += o[3];
                }
            } else {
                // one wave: thread == lane, and grp walks this lane's own mt tiles
                v[nt] = acc[nt][0];
#pragma unroll
                for (int b2 = 1; b2 < MT; ++b2)
                    if (b2 == mt) v[nt] = acc[nt][b2];
            }
        }
        const int mrow = mt * 16 + (l2 & 15);
        if (res.accumulate) {
            // producer (MT == 1, NTB == 1: the threads are the first wave, all of it takes part
            // in the exchange below): Y += sums; operand and sum of squares for the next norm
            const int n0 = tile_row[0] + (l2 >> 4) * 4;
            float sq = 0.f;
            if (mrow < M) {
                // grp == threadIdx.x here: the thread that fetched pre_y and pre_nw
                float y[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    y[i] = pre_y[i] + v[0][i];
                    if (res.nw && n0 + i < N) sq = fmaf(y[i], y[i], sq);
                }
                const size_t at = (size_t)mrow * N + n0;
                if (n0 + 3 < N && (N & 3) == 0) {
                    *(float4*)((float*)Y + at) = make_float4(y[0], y[1], y[2], y[3]);
                    if (res.nw)
                        *(uint2*)(res.xb + at) = make_uint2(pack_bf16x2(y[0] * pre_nw[0], y[1] * pre_nw[1]),
                                                            pack_bf16x2(y[2] * pre_nw[2], y[3] * pre_nw[3]));
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n0 + i < N) {
                            ((float*)Y)[at + i] = y[i];
                            if (res.nw) res.xb[at + i] = f32_to_bf16(y[i] * pre_nw[i]);
                        }
                }
            }
            if (res.nw) {
                sq += __shfl_xor(sq, 16, ILLM_WAVE);
                sq += __shfl_xor(sq, 32, ILLM_WAVE);
                if (l2 < 16 && mrow < M) res.ssq_out[(size_t)mrow * gridDim.x + blockIdx.x] = sq;
            }
            continue;
        }
        if (mrow >= M) continue;
        const float rs = MT == 1 ? row_scale(l2 & 15) : 1.0f;
#pragma unroll
        for (int nt = 0; nt < NTB; ++nt) {
            const int n0 = tile_row[nt] + (l2 >> 4) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n0 + i < N) st_f(Y, y_dt, (size_t)mrow * N + n0 + i, v[nt][i] * rs);
        }
    }
}

static const SkResidual SK_NO_RESIDUAL = {0, nullptr, ILLM_BF16, nullptr, nullptr, nullptr, 0, 0.f};

template <int MT, int NTB, int U, int MODE = SK_PLAIN, bool TILED = false, bool ONE_SHOT = false>
static int launch_skinny(const void* X, const void* W, void* Y, int y_dt, int M, int N, int K,
                         int waves, hipStream_t st, SkRope rope = SkRope(),
                         SkResidual res = SK_NO_RESIDUAL) {
    constexpr bool DUAL = MODE == SK_GATE_UP;
    // registers a lane needs: operands of two pieces in flight (one if ONE_SHOT) and the accumulators
    constexpr int REGS = (ONE_SHOT ? 1 : 2) * (NTB + MT) * U * 4 + NTB * 8 + NTB * MT * 4 + 40;
    constexpr int MAXW = REGS <= 128 ? 16 : (REGS <= 256 ? 8 : 4);
    waves = waves > MAXW ? MAXW : waves;
    const int rows_per_block = DUAL ? 8 * NTB : 16 * NTB;
    const int blocks = (N + rows_per_block - 1) / rows_per_block;
    const size_t smem = (size_t)waves * NTB * ((!TILED && U > MT) ? U : MT) * 1024 + 64;
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, NTB, U, MAXW, MODE, TILED, ONE_SHOT>), dim3(blocks), dim3(64 * waves),
                       smem, st, (const bf16_t*)X, (const bf16_t*)W, Y, y_dt, M, N, K, rope, res);
    return illm_launch_status();
}

// Measured on MI355X at the LLaMA-2-7B shapes: 16 W rows per block and about this many waves
// on the chip are best for M <= 16; wider row tiles only pay when X has many rows.
static const int SK_WAVES_ON_CHIP = 2400;
// A block of the tiled gate|up and plain products takes two tiles from 1024 tiles on.
static bool two_tiles_a_block(int blocks) { return blocks >= 1024; }
static int SK_ONE_SHOT = 1;           // tuning: 0 switches the one-piece-per-wave variant off
extern "C" void illm_set_skinny_one_shot(int on) { SK_ONE_SHOT = on; }
static const int SK_WAVES_ON_CHIP_TILED = 3072;      // from the tiled copy (no staging in LDS)

static int clamp_waves(int w, int ntb, int mt, int u, int K) {
    const int ksteps = (K + 31) / 32;
    const int max_by_k = (ksteps + u - 1) / u;           // more waves than k pieces would idle
    const int lds_cap = 60 / (ntb * (u > mt ? u : mt));     // 64 KB of LDS a block, some left for the scales
    w = w > 16 ? 16 : w;
    w = w > lds_cap ? lds_cap : w;
    w = w > max_by_k ? max_by_k : w;
    return w < 1 ? 1 : w;
}

// The product from the matrix itself (no tiled copy) with the tile shape given: 16 * ntb rows of
// W a block, u * 64 bytes of a W row per wave iteration, waves per block (clamped to what LDS
// and K allow).  Up to 16 rows of X take ntb = 1, more take 2; u = 4 (measured best).
static int skinny_from_matrix(const void* X, const void* W, void* Y, int y_dt, int M,
                              int N, int K, int ntb, int u, int waves, void* stream) {
    if (M <= 0 || M > 64 || N <= 0 || K <= 0 || (K % 8) || !illm_dtype_ok(y_dt))
        return ILLM_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int mt = (M + 15) / 16;
    waves = clamp_waves(waves, ntb, mt, u, K);
#define GO(MT_, NTB_, U_)                                                                     \
    if (mt == MT_ && ntb == NTB_ && u == U_)                                                  \
        return launch_skinny<MT_, NTB_, U_>(X, W, Y, y_dt, M, N, K, waves, st)
    GO(1, 1, 4); GO(2, 2, 4); GO(3, 2, 4); GO(4, 2, 4);
#undef GO
    return ILLM_ERR_ARG;
}

static bool scale_args_ok(const float* ssq, int parts, int M) {
    return !ssq || (parts > 0 && M <= 16);
}

// Takes bfloat16 X and W, M in 1..64, K a multiple of 8.  Otherwise ILLM_ERR_ARG.
// ssq != null (M <= 16): row m of the result is scaled by 1 / sqrt(sum_p ssq[m][p] / K + eps).
// Wt != null: the tiled copy of W (see the kernel), used for M <= 16 and K % 32 == 0.
static bool use_tiled(const void* Wt, int M, int K) { return Wt && M <= 16 && K % 32 == 0; }

extern "C" int illm_gemm_skinny_bf16(const void* X, const void* W, const void* Wt, void* Y, int y_dt,
                                     int M, int N, int K, const float* ssq, int parts, float eps,
                                     int waves_wanted, void* stream) {
    if (M <= 0 || M > 64 || N <= 0 || K <= 0 || (K % 8) || !illm_dtype_ok(y_dt) ||
        !scale_args_ok(ssq, parts, M))
        return ILLM_ERR_ARG;
    const int ntb = M <= 16 ? 1 : 2, u = 4;
    const int blocks = (N + 16 * ntb - 1) / (16 * ntb);
    const int on_chip = use_tiled(Wt, M, K) ? SK_WAVES_ON_CHIP_TILED : SK_WAVES_ON_CHIP;
    int waves = waves_wanted > 0 ? waves_wanted : (on_chip + blocks / 2) / blocks;
    waves = waves < 1 ? 1 : waves;
    if (!ssq && !use_tiled(Wt, M, K))
        return skinny_from_matrix(X, W, Y, y_dt, M, N, K, ntb, u, waves, stream);
    SkResidual res = SK_NO_RESIDUAL;
    res.ssq = ssq; res.parts = parts; res.eps = eps;
    waves = clamp_waves(waves, 1, 1, 4, K);
    if (use_tiled(Wt, M, K)) {
        // with many tiles (the head) a block takes two: X is read half as often
        if (two_tiles_a_block(blocks)) {
            const int blocks2 = (blocks + 1) / 2;
            int w2 = waves_wanted > 0 ? waves_wanted : (on_chip + blocks2 / 2) / blocks2;
            return launch_skinny<1, 2, 4, SK_PLAIN, true>(X, Wt, Y, y_dt, M, N, K,
                                                          clamp_waves(w2 < 1 ? 1 : w2, 2, 1, 4, K),
                                                          (hipStream_t)stream, SkRope(), res);
        }
        return launch_skinny<1, 1, 4, SK_PLAIN, true>(X, Wt, Y, y_dt, M, N, K, waves,
                                                      (hipStream_t)stream, SkRope(), res);
    }
    return launch_skinny<1, 1, 4>(X, W, Y, y_dt, M, N, K, waves, (hipStream_t)stream, SkRope(), res);
}

// Y[M, N] (float32) += X . W^T for M <= 16 bfloat16 rows: a block's output projection with the
// residual add.  nw != null: also xb[M, N] = bfloat16(Y * nw) and ssq_out[M][ceil(N / 16)], the
// sums of Y^2 over each block's 16 columns, for a product that takes the norm (see SkResidual).
extern "C" int illm_gemm_skinny_add(const void* X, const void* W, const void* Wt, float* Y, int M,
                                    int N, int K, const void* nw, int nw_dt, void* xb,
                                    float* ssq_out, int waves_wanted, void* stream) {
    if (M <= 0 || M > 16 || N <= 0 || K <= 0 || (K % 8) || !Y ||
        (nw && (!illm_dtype_ok(nw_dt) || !xb || !ssq_out)))
        return ILLM_ERR_ARG;
    const int blocks = (N + 15) / 16;
    const int on_chip = use_tiled(Wt, M, K) ? SK_WAVES_ON_CHIP_TILED : SK_WAVES_ON_CHIP;
    int waves = waves_wanted > 0 ? waves_wanted : (on_chip + blocks / 2) / blocks;
    waves = clamp_waves(waves < 1 ? 1 : waves, 1, 1, 4, K);
    SkResidual res = SK_NO_RESIDUAL;
    res.accumulate = 1; res.nw = nw; res.nw_dt = nw_dt; res.xb = (bf16_t*)xb; res.ssq_out = ssq_out;
    if (use_tiled(Wt, M, K)) {
        // a K of at most 8 pieces of 16 k-steps (4096) and few enough tiles that a block has the
        // chip's compute unit to itself: 8 waves, each with its whole share of K in flight at once
        if (SK_ONE_SHOT && K <= 8 * 16 * 32 && blocks <= 512 && waves_wanted <= 0)
            return launch_skinny<1, 1, 16, SK_PLAIN, true, true>(
                X, Wt, Y, ILLM_F32, M, N, K, (K / 32 + 15) / 16, (hipStream_t)stream, SkRope(), res);
        return launch_skinny<1, 1, 4, SK_PLAIN, true>(X, Wt, Y, ILLM_F32, M, N, K, waves,
                                                      (hipStream_t)stream, SkRope(), res);
    }
    return launch_skinny<1, 1, 4>(X, W, Y, ILLM_F32, M, N, K, waves, (hipStream_t)stream, SkRope(),
                                  res);
}

// Y[M, F] = silu(X . Wg^T) * (X . Wu^T) with W = [Wg (F rows) | Wu (F rows)], [2F, K]:
// the gate and up products and the SiLU-multiply in one kernel (src/core/graph.cpp:57-79).
// ssq: as for illm_gemm_skinny_bf16.
extern "C" int illm_gemm_skinny_gateup_silu(const void* X, const void* W, const void* Wt, void* Y,
                                            int y_dt, int M, int F, int K, const float* ssq,
                                            int parts, float eps, int waves_wanted, void* stream) {
    if (M <= 0 || M > 64 || F <= 0 || K <= 0 || (K % 8) || !illm_dtype_ok(y_dt) ||
        !scale_args_ok(ssq, parts, M))
        return ILLM_ERR_ARG;
    SkResidual res = SK_NO_RESIDUAL;
    res.ssq = ssq; res.parts = parts; res.eps = eps;
    hipStream_t st = (hipStream_t)stream;
    const int mt = (M + 15) / 16;
    const int blocks = (F + 7) / 8;
    // measured at F = 11008, K = 4096: 4 to 8 waves a block are within 1 % of each other, 2 are
    // 6 % slower; from the tiled copy 3 are best (at 8 rows 10 % better than 6)
    const int on_chip = use_tiled(Wt, M, K) ? 4096 : 8192;
    int waves = waves_wanted > 0 ? waves_wanted : (on_chip + blocks / 2) / blocks;
    waves = clamp_waves(waves < 1 ? 1 : waves, 1, mt, 4, K);
    if (use_tiled(Wt, M, K)) {
        // with many tiles a block takes two: X is read half as often (measured at F = 11008, 8 and
        // 16 rows: 36 -> 31 us and 46 -> 33 us; one row: no change)
        if (two_tiles_a_block(blocks)) {
            const int blocks2 = (F + 15) / 16;
            int w2 = waves_wanted > 0 ? waves_wanted : (1400 + blocks2 / 2) / blocks2;
            w2 = clamp_waves(w2 < 1 ? 1 : w2, 2, mt, 4, K);
            return launch_skinny<1, 2, 4, SK_GATE_UP, true>(X, Wt, Y, y_dt, M, F, K, w2, st, SkRope(), res);
        }
        return launch_skinny<1, 1, 4, SK_GATE_UP, true>(X, Wt, Y, y_dt, M, F, K, waves, st, SkRope(), res);
    }
    if (mt == 1 && two_tiles_a_block(blocks)) {
        const int blocks2 = (F + 15) / 16;
        int w2 = waves_wanted > 0 ? waves_wanted : (1400 + blocks2 / 2) / blocks2;
        w2 = clamp_waves(w2 < 1 ? 1 : w2, 2, mt, 4, K);
        return launch_skinny<1, 2, 4, SK_GATE_UP>(X, W, Y, y_dt, M, F, K, w2, st, SkRope(), res);
    }
    switch (mt) {
        case 1: return launch_skinny<1, 1, 4, SK_GATE_UP>(X, W, Y, y_dt, M, F, K, waves, st, SkRope(), res);
        case 2: return launch_skinny<2, 1, 4, SK_GATE_UP>(X, W, Y, y_dt, M, F, K, waves, st);
        case 3: return launch_skinny<3, 1, 4, SK_GATE_UP>(X, W, Y, y_dt, M, F, K, waves, st);
        default: return launch_skinny<4, 1, 4, SK_GATE_UP>(X, W, Y, y_dt, M, F, K, waves, st);
    }
}

// Decode step of an attention layer's input side in one kernel: Y = X . Wqkv^T, the q and k heads
// rotated (pairs (i, i + hd/2), all hd dims) by the angles at row_pos[m], q written to
// Y[M, (nh + 2 nkv) hd] (its k and v parts are left untouched), k and v written to the paged cache
// of row_slot[m].  M <= 16, hd % 16 == 0, K % 8 == 0, bfloat16.  ssq: as for illm_gemm_skinny_bf16.
extern "C" int illm_qkv_rope_store_skinny(const void* X, const void* W, const void* Wt, void* Y,
                                          int M, int K,
                                          const float* cos_sin, int max_pos,
                                          const int32_t* row_pos, const int32_t* row_slot,
                                          void* kcache, void* vcache, const int32_t* page_table,
                                          int table_stride, int page_size, int ring, int nh, int nkv,
                                          int hd, const float* ssq, int parts, float eps,
                                          int waves_wanted, void* stream) {
    if (!scale_args_ok(ssq, parts, M)) return ILLM_ERR_ARG;
    SkResidual res = SK_NO_RESIDUAL;
    res.ssq = ssq; res.parts = parts; res.eps = eps;
    if (M <= 0 || M > 16 || K <= 0 || (K % 8) || nh <= 0 || nkv <= 0 || hd <= 0 || (hd % 16) ||
        !cos_sin || max_pos <= 0 || !row_pos || !row_slot || !kcache || !vcache || !page_table ||
        table_stride <= 0 || page_size <= 0)
        return ILLM_ERR_ARG;
    SkRope rope = {cos_sin, row_pos, row_slot, (bf16_t*)kcache, (bf16_t*)vcache, page_table,
                   table_stride, page_size, ring, nh, nkv, hd};
    const int N = (nh + 2 * nkv) * hd;
    const int blocks = N / 16;
    int waves = waves_wanted > 0 ? waves_wanted : (SK_WAVES_ON_CHIP + blocks / 2) / blocks;
    waves = clamp_waves(waves < 1 ? 1 : waves, 1, 1, 4, K);
    if (use_tiled(Wt, M, K))
        return launch_skinny<1, 1, 4, SK_QKV_ROPE, true>(X, Wt, Y, ILLM_BF16, M, N, K, waves,
                                                         (hipStream_t)stream, rope, res);
    return launch_skinny<1, 1, 4, SK_QKV_ROPE>(X, W, Y, ILLM_BF16, M, N, K, waves,
                                               (hipStream_t)stream, rope, res);
}

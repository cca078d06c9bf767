// Products of 9 to 128 rows with the wide matrices of a block (q|k|v, gate|up, the head) and what
// follows them in one kernel: Y = X[M, K] . W[N, K]^T from the tiled copy of W
// ([tile of 16 rows][K / 32][16 rows][32 k], see gemm_skinny.hip), bfloat16 operands, float32
// accumulation on the matrix cores (MFMA 16x16x32), then per mode
//   GR_PLAIN     Y = sums (bfloat16 or float32),
//   GR_GATE_UP   tiles of 8 gate rows and the same 8 up rows: Y[M, F] = silu(gate) * up,
//   GR_QKV_ROPE  tiles of 8 rows of a q or k head and their 8 rotation partners, then tiles of
//                16 v rows: q and k rotated by the row's position, q into Y, k and v into the
//                paged cache.
//
// With this many rows a wave that reads X for itself is bound by X (gemm_skinny.hip), and the
// vendor GEMM, which the reference would call here (cublasSgemm,
// src/kern/gpu/kernel_gpu.cu:420-435, then elementwise kernels :183-209 and :343-372), reads
// these matrices at half the memory's speed and leaves the rotation and the SiLU-multiply to
// kernels of their own.  Here a block is TB tiles x KP parts of K: wave (t, p) streams tile t's
// share p of K from the tiled copy straight into operand registers, three pieces of 64 k ahead; the
// TB waves of a part share the part's piece of X through LDS (written as loaded in 16-byte units,
// swizzled within a row, two buffers, one barrier a piece).  K is cut inside the block, not over
// blocks: the parts' sums are added through LDS in part order (a fixed order of summation) and
// the waves of part 0 finish their tile in registers: a rotation pair, or a gate and its up row,
// lie 32 lanes apart in the accumulator.
//
// What bounds these products at 32 to 64 rows is X, not W: every block reads all of X from the
// L2 cache, and with few tiles a block that is more bytes than the block's share of W (measured
// at 64 rows of a 22016 x 4096 gate|up: 45 us with blocks of 3 tiles, 33 us when X comes from
// the L1 cache instead, 33 us with blocks of 6 tiles).  So the host gives a block as many tiles
// (2 to 8) as still fill the chip's compute units in whole rounds.
#include <math.h>

#include "api.h"
#include "api_test.h"
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

enum { GR_PLAIN = 0, GR_GATE_UP = 1, GR_QKV_ROPE = 2 };

struct GrRope {
    const float* cos_sin;        // [max_pos][hd/2][2]
    const int32_t* row_pos;      // [M]
    const int32_t* row_slot;     // [M]
    bf16_t* kcache;
    bf16_t* vcache;
    const int32_t* page_table;
    int table_stride, page_size, ring, nh, nkv, hd;
};

// X is bfloat16(x * norm weight) of residual rows whose sums of squares lie in ssq[M][parts]
// (gemm_skinny.hip, SkResidual): row m of the result is scaled by
// 1 / sqrt(sum_p ssq[m][p] / K + eps).  Up to 16 rows only.
struct GrScale {
    const float* ssq;
    int parts;
    float eps;
};

// GR_PIECE: k-steps of 32 in a piece.  A block of four or more tiles has at most two parts of K,
// one of two or three tiles up to four.
template <int MT, int TB, int MODE, int GR_PIECE>
__global__ void __launch_bounds__(64 * TB * (TB >= 4 ? 2 : 4) / (MT > 4 ? 2 : 1))
gemm_rows_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ Wt, void* __restrict__ Y,
                 int y_dt, int M, int N, int K, int tiles, int kp, GrRope rope, GrScale scale) {
    constexpr int UNITS = MT * 16 * GR_PIECE * 4;            // 16-byte units of a part's X piece
    constexpr int XU = (UNITS + TB * 64 - 1) / (TB * 64);    // units a thread stages
    extern __shared__ uint4 lds[];       // X pieces [kp][2][UNITS]; afterwards the parts' sums
    float* row_rs = (float*)(lds + (size_t)kp * 2 * UNITS);   // [16], behind the pieces (MT == 1)
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int r = lane & 15, q = lane >> 4;
    const int tl = wave % TB, part = wave / TB;
    const int tile = blockIdx.x * TB + tl;
    const bool tile_ok = tile < tiles;
    const int ksteps = K / 32;
    const int pieces = (ksteps + GR_PIECE - 1) / GR_PIECE;
    const int per = (pieces + kp - 1) / kp;                  // pieces a part takes
    const int p_begin = part * per;
    int p_end = p_begin + per;
    p_end = p_end < pieces ? p_end : pieces;

    if (MT == 1 && scale.ssq && wave == TB * kp - 1) {
        // the scale of every X row, by the last wave while the others already stream W: all
        // rows' loads are asked for at once, then one sum over the wave a row
        float t[16];
#pragma unroll
        for (int m = 0; m < 16; ++m) t[m] = 0.f;
        for (int p = lane; p < scale.parts; p += 64) {
            float v[16];
#pragma unroll
            for (int m = 0; m < 16; ++m)
                v[m] = m < M ? scale.ssq[(size_t)m * scale.parts + p] : 0.f;
#pragma unroll
            for (int m = 0; m < 16; ++m) t[m] += v[m];
        }
        float mine = 0.f;
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            const float sum = wave_sum(t[m]);
            if (lane == m) mine = sum;
        }
        if (lane < 16) row_rs[lane] = 1.0f / sqrtf(mine / (float)K + scale.eps);
    }

    // staging of the part's X piece: unit u = row u / 8, 8 k at (u % 8) * 8; rows >= M read row
    // M - 1 and their results are dropped.  Where the part's threads do not divide the piece, the
    // threads left over bring a unit a second time (the same bytes to the same place).
    const int tp = tl * 64 + lane;                           // thread within its part
    const bf16_t* xsrc[XU];
    int x_dst[XU], x_k[XU];
#pragma unroll
    for (int j = 0; j < XU; ++j) {
        const int u = (tp + j * TB * 64) % UNITS;
        constexpr int UPR = GR_PIECE * 4;                    // units in a row of the piece
        const int row = u / UPR, c = u % UPR;
        const int m = row < M ? row : M - 1;
        xsrc[j] = X + (size_t)m * K;
        x_k[j] = c * 8;
        x_dst[j] = part * 2 * UNITS + row * UPR + (c ^ (row & (UPR - 1)));
    }
    uint4* xs = lds + (size_t)part * 2 * UNITS;
    const bf16_t* wsrc = Wt + (size_t)tile * ksteps * 512 + (r * 4 + q) * 8;

    // Loads are unconditional (piece indices clamped; K is a multiple of the piece, so nothing
    // lies beyond it), and every stage of the loop below names its registers statically, so that
    // the compiler's wait counts leave the newer loads in flight while the oldest is used: a wave
    // has three pieces of W and two of X on their way at any time.  Loads return in the order of
    // issue, and the wait count the compiler puts before a stage is the fewer of what the
    // prologue and what the round before leave behind the load it needs: the prologue therefore
    // issues its loads in the very order the stages would have (scheduling barriers keep the
    // compiler from sorting them), or the first stage of every round would wait for all loads.
    const int p_last = (p_end > p_begin ? p_end : pieces) - 1;         // a piece that exists
    const bf16_t* wtile = tile_ok ? wsrc : Wt + (r * 4 + q) * 8;       // no tile: tile 0, dropped
#define GR_LOAD_X(P, XG)                                                                          \
    {                                                                                             \
        const int pc_ = (P) < p_last ? (P) : p_last;                                              \
        _Pragma("unroll") for (int j = 0; j < XU; ++j)                                            \
            XG[j] = *(const illm_u32x4_t*)(xsrc[j] + (size_t)pc_ * (GR_PIECE * 32) + x_k[j]);            \
    }
#define GR_LOAD_W(P, A)                                                                           \
    {                                                                                             \
        const int pc_ = (P) < p_last ? (P) : p_last;                                              \
        _Pragma("unroll") for (int u = 0; u < GR_PIECE; ++u)                                      \
            A[u] = __builtin_nontemporal_load((const illm_u32x4_t*)(wtile + (size_t)(pc_ * GR_PIECE + u) * 512));                       \
    }

    // GR_QKV_ROPE: what the waves of part 0 need to finish their tile (positions, angles, cache
    // pages) is asked for around the first pieces of W, two dependent loads deep, and has long
    // arrived when the sums are complete.  Indices are clamped, so every lane loads something.
    int rot_head = -1, rot_j = 0, e_pos[MT], e_slot[MT], e_page[MT];
    float cs[MT][8];
    const bool finishes = MODE == GR_QKV_ROPE && part == 0;
    if (finishes) {
        const int tph = rope.hd / 16, n_rot = (rope.nh + rope.nkv) * tph;
        if (tile_ok && tile < n_rot) {
            rot_head = tile / tph;
            rot_j = tile % tph;
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r < M ? mt * 16 + r : M - 1;
            e_pos[mt] = rope.row_pos[m];
            e_slot[mt] = rope.row_slot[m];
        }
    }

    f32x4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    // (native vector types: arrays of the runtime's uint4 struct are not always kept in registers)
    illm_u32x4_t xr0[XU], xr1[XU], xr2[XU], xr3[XU];
    illm_u32x4_t wr0[GR_PIECE], wr1[GR_PIECE], wr2[GR_PIECE], wr3[GR_PIECE];
    GR_LOAD_W(p_begin, wr0)
    __builtin_amdgcn_sched_barrier(0);
    GR_LOAD_X(p_begin, xr0)
    __builtin_amdgcn_sched_barrier(0);
    GR_LOAD_W(p_begin + 1, wr1)
    __builtin_amdgcn_sched_barrier(0);
    GR_LOAD_X(p_begin + 1, xr1)
    __builtin_amdgcn_sched_barrier(0);
    GR_LOAD_W(p_begin + 2, wr2)
    __builtin_amdgcn_sched_barrier(0);
    if (finishes) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const float4* c4 = (const float4*)(rope.cos_sin + (size_t)e_pos[mt] * rope.hd +
                                               2 * (8 * rot_j + 4 * (q & 1)));
            const float4 c0 = c4[0], c1 = c4[1];
            cs[mt][0] = c0.x; cs[mt][1] = c0.y; cs[mt][2] = c0.z; cs[mt][3] = c0.w;
            cs[mt][4] = c1.x; cs[mt][5] = c1.y; cs[mt][6] = c1.z; cs[mt][7] = c1.w;
            int lp = e_pos[mt] / rope.page_size;
            if (rope.ring > 0) lp %= rope.ring;
            e_page[mt] = rope.page_table[(size_t)e_slot[mt] * rope.table_stride + lp];
        }
    }
    // A stage of a round of four: piece p = p_begin + I.  It first asks for X two pieces and W
    // three pieces on, then waits for its own piece of X.  One barrier a piece is enough with two
    // buffers: whoever writes buffer BUF again, two pieces on, has passed the next piece's
    // barrier, which every wave reaches only after it has finished reading this one.
#define GR_STAGE(I, BUF, XCUR, XNEXT, WCUR, WNEXT)                                                \
    {                                                                                             \
        const int p = p_begin + (I);                                                              \
        GR_LOAD_X(p + 2, XNEXT)                                                                   \
        GR_LOAD_W(p + 3, WNEXT)                                                                   \
        _Pragma("unroll") for (int j = 0; j < XU; ++j)                                            \
            ((illm_u32x4_t*)lds)[(BUF) * UNITS + x_dst[j]] = XCUR[j];                             \
        __syncthreads();                                                                          \
        if (p < p_end) {                                                                          \
            _Pragma("unroll") for (int u = 0; u < GR_PIECE; ++u)                                  \
                _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                               \
                    const int row = mt * 16 + r;                                                  \
                    const uint4 b = xs[(BUF) * UNITS + row * (GR_PIECE * 4) +                     \
                                       ((u * 4 + q) ^ (row & (GR_PIECE * 4 - 1)))];               \
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(                            \
                        *(const bf16x8_t*)&WCUR[u], *(const bf16x8_t*)&b, acc[mt], 0, 0, 0);      \
                }                                                                                 \
        }                                                                                         \
    }
    for (int i = 0; i < per; i += 4) {                       // every wave runs the same rounds
        GR_STAGE(i, 0, xr0, xr2, wr0, wr3)
        GR_STAGE(i + 1, 1, xr1, xr3, wr1, wr0)
        GR_STAGE(i + 2, 0, xr2, xr0, wr2, wr1)
        GR_STAGE(i + 3, 1, xr3, xr1, wr3, wr2)
    }
#undef GR_STAGE
#undef GR_LOAD_X
#undef GR_LOAD_W
    __syncthreads();                                         // the X pieces are no longer read

    // the parts' sums, added in part order by the waves of part 0
    if (kp > 1) {
        f32x4_t* red = (f32x4_t*)lds;                        // [kp - 1][TB][MT][64]
        if (part > 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                red[(((size_t)(part - 1) * TB + tl) * MT + mt) * 64 + lane] = acc[mt];
        }
        __syncthreads();
        if (part > 0) return;
        for (int p = 1; p < kp; ++p)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const f32x4_t o = red[(((size_t)(p - 1) * TB + tl) * MT + mt) * 64 + lane];
                acc[mt][0] += o[0]; acc[mt][1] += o[1]; acc[mt][2] += o[2]; acc[mt][3] += o[3];
            }
    }
    if (!tile_ok) return;
    // acc[mt][i] = sum for X row mt * 16 + r and row 4 q + i of the tile

#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        f32x4_t v = acc[mt];
        if (MT == 1 && scale.ssq) {
            const float rs = row_rs[r < M ? r : 0];
            v[0] *= rs; v[1] *= rs; v[2] *= rs; v[3] *= rs;
        }
        if (MODE == GR_PLAIN) {
            if (m >= M) continue;
            const int n0 = tile * 16 + q * 4;
            const size_t at = (size_t)m * N + n0;
            if (n0 + 3 < N && (N & 3) == 0) {
                if (y_dt == ILLM_F32)
                    *(float4*)((float*)Y + at) = make_float4(v[0], v[1], v[2], v[3]);
                else
                    *(uint2*)((bf16_t*)Y + at) =
                        make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n0 + i < N) st_f(Y, y_dt, at + i, v[i]);
            }
        } else {
            // the partner rows (up rows, rotation partners) are held 32 lanes on; every lane
            // takes part in the exchange
            f32x4_t o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = __shfl_xor(v[i], 32, ILLM_WAVE);
            if (MODE == GR_GATE_UP) {
                if (m >= M || q >= 2) continue;
                const int n0 = tile * 8 + q * 4;             // N is F here
                float y[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) y[i] = (v[i] / (1.0f + expf(-v[i]))) * o[i];
                const size_t at = (size_t)m * N + n0;
                if (n0 + 3 < N && (N & 3) == 0 && y_dt == ILLM_BF16) {
                    *(uint2*)((bf16_t*)Y + at) =
                        make_uint2(pack_bf16x2(y[0], y[1]), pack_bf16x2(y[2], y[3]));
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n0 + i < N) st_f(Y, y_dt, at + i, y[i]);
                }
            } else {                                         // GR_QKV_ROPE, bfloat16 throughout
                if (m >= M) continue;
                if (rot_head >= 0) {
                    if (q >= 2) continue;
                    float y0[4], y1[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float c = cs[mt][2 * i], sn = cs[mt][2 * i + 1];
                        y0[i] = v[i] * c - o[i] * sn;
                        y1[i] = v[i] * sn + o[i] * c;
                    }
                    // the row of the cache: [page][kv head][row in page][head_dim]
                    const size_t c_off = (((size_t)e_page[mt] * rope.nkv + (rot_head - rope.nh)) *
                                              rope.page_size + e_pos[mt] % rope.page_size) * rope.hd +
                                         8 * rot_j + 4 * q;
                    bf16_t* dst = rot_head < rope.nh
                                      ? (bf16_t*)Y + (size_t)m * N + rot_head * rope.hd + 8 * rot_j + 4 * q
                                      : rope.kcache + c_off;
                    *(uint2*)dst = make_uint2(pack_bf16x2(y0[0], y0[1]), pack_bf16x2(y0[2], y0[3]));
                    *(uint2*)(dst + rope.hd / 2) =
                        make_uint2(pack_bf16x2(y1[0], y1[1]), pack_bf16x2(y1[2], y1[3]));
                } else {
                    const int vrow = (tile - (rope.nh + rope.nkv) * (rope.hd / 16)) * 16 + 4 * q;
                    const size_t c_off = (((size_t)e_page[mt] * rope.nkv + vrow / rope.hd) *
                                              rope.page_size + e_pos[mt] % rope.page_size) * rope.hd +
                                         vrow % rope.hd;
                    *(uint2*)(rope.vcache + c_off) =
                        make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
                }
            }
        }
    }
}

// Tiles a block takes (2 to 8) and parts of K (1, 2 or 4; a part has at least 4 pieces).  The
// blocks run in rounds of one a compute unit and a block's time grows with its tiles, so the tiles
// are those with the fewest rounds x tiles; among equals the most tiles with more than 16 rows
// (the less of X is read) and the fewest with up to 16 (X is small, more blocks start sooner).
// Measured at 16 to 64 rows of the q|k|v, gate|up and head matrices of the 7B, 8B and 70B shapes,
// where this picks the fastest or one within 3 % of it.  Blocks of up to three tiles cut K in two
// (six waves at least), larger ones do not.
static int GR_TB = 0, GR_KP = 0;          // tuning and tests: forced values (0: the choice below)
extern "C" void illm_set_rows_shape(int tb, int kp) {
    GR_TB = (tb >= 2 && tb <= 8) ? tb : 0;
    GR_KP = (kp == 1 || kp == 2 || kp == 4) ? kp : 0;
}

#define GR_PIECE_STEPS 2      // k-steps of 32 in a piece (pieces of 128 k measured no better at 16
                              // rows and worse at 64)

static void rows_shape(int tiles, int K, int mt, int* tb, int* kp) {
    const int cus = 256;
    int best_tb = 2;
    long long best = -1;
    for (int t = 2; t <= 8; ++t) {
        const int blocks = (tiles + t - 1) / t;
        const long long cost = (long long)((blocks + cus - 1) / cus) * t;
        if (best < 0 || cost < best || (cost == best && mt > 1)) {
            best = cost;
            best_tb = t;
        }
    }
    *tb = GR_TB ? GR_TB : best_tb;
    *kp = GR_KP ? GR_KP : (*tb <= 3 ? 2 : 1);
    const int kp_max = (*tb >= 4 ? 2 : 4) / (mt > 4 ? 2 : 1);   // the kernel's launch bounds
    if (*kp > kp_max) *kp = kp_max;
    const int pieces = (K / 32 + GR_PIECE_STEPS - 1) / GR_PIECE_STEPS;
    while (*kp > 1 && pieces / *kp < 4) *kp /= 2;
}

template <int MT, int MODE>
static int launch_rows(const bf16_t* x, const bf16_t* wt, void* y, int y_dt, int rows, int N, int K,
                       int tiles, const GrRope& rope, const GrScale& scale, hipStream_t st) {
    int tb, kp;
    rows_shape(tiles, K, MT, &tb, &kp);
    constexpr int ps = GR_PIECE_STEPS;
    const size_t x_bytes = (size_t)kp * 2 * MT * 16 * ps * 4 * 16 + (MT == 1 ? 64 : 0);
    const size_t red_bytes = (size_t)(kp - 1) * tb * MT * 64 * 16;
    const size_t smem = x_bytes > red_bytes ? x_bytes : red_bytes;
    const dim3 grid((tiles + tb - 1) / tb), block(64 * tb * kp);
#define GO(TB_, PS_)                                                                              \
    hipLaunchKernelGGL((gemm_rows_kernel<MT, TB_, MODE, PS_>), grid, block, smem, st, x, wt, y,   \
                       y_dt, rows, N, K, tiles, kp, rope, scale)
    switch (tb) {
        case 2: GO(2, GR_PIECE_STEPS); break;
        case 3: GO(3, GR_PIECE_STEPS); break;
        case 4: GO(4, GR_PIECE_STEPS); break;
        case 5: GO(5, GR_PIECE_STEPS); break;
        case 6: GO(6, GR_PIECE_STEPS); break;
        case 7: GO(7, GR_PIECE_STEPS); break;
        default: GO(8, GR_PIECE_STEPS); break;
    }
#undef GO
    return illm_launch_status();
}

static int GR_ROWS_A_LAUNCH = 128;        // tuning and tests: 64 or 128 rows of X a launch
extern "C" void illm_set_rows_a_launch(int rows) { GR_ROWS_A_LAUNCH = rows == 64 ? 64 : 128; }

template <int MODE>
static int rows_product(const void* X, const void* Wt, void* Y, int y_dt, int M, int N, int K,
                        int tiles, GrRope rope, const GrScale& scale, hipStream_t st) {
    // more rows than a launch takes: W is read again for each
    const size_t y_elem = y_dt == ILLM_F32 ? 4 : 2;
    const int a_launch = GR_ROWS_A_LAUNCH;
    for (int m0 = 0; m0 < M; m0 += a_launch) {
        const int rows = M - m0 < a_launch ? M - m0 : a_launch;
        const int mt = (rows + 15) / 16;
        const bf16_t* x = (const bf16_t*)X + (size_t)m0 * K;
        void* y = (char*)Y + (size_t)m0 * N * y_elem;
        GrRope rp = rope;
        if (MODE == GR_QKV_ROPE) {
            rp.row_pos += m0;
            rp.row_slot += m0;
        }
        int rc;
        switch (mt) {
            case 1: rc = launch_rows<1, MODE>(x, (const bf16_t*)Wt, y, y_dt, rows, N, K, tiles, rp, scale, st); break;
            case 2: rc = launch_rows<2, MODE>(x, (const bf16_t*)Wt, y, y_dt, rows, N, K, tiles, rp, scale, st); break;
            case 3: rc = launch_rows<3, MODE>(x, (const bf16_t*)Wt, y, y_dt, rows, N, K, tiles, rp, scale, st); break;
            case 4: rc = launch_rows<4, MODE>(x, (const bf16_t*)Wt, y, y_dt, rows, N, K, tiles, rp, scale, st); break;
            case 5: rc = launch_rows<5, MODE>(x, (const bf16_t*)Wt, y, y_dt, rows, N, K, tiles, rp, scale, st); break;
            case 6: rc = launch_rows<6, MODE>(x, (const bf16_t*)Wt, y, y_dt, rows, N, K, tiles, rp, scale, st); break;
            case 7: rc = launch_rows<7, MODE>(x, (const bf16_t*)Wt, y, y_dt, rows, N, K, tiles, rp, scale, st); break;
            default: rc = launch_rows<8, MODE>(x, (const bf16_t*)Wt, y, y_dt, rows, N, K, tiles, rp, scale, st); break;
        }
        if (rc != ILLM_OK) return rc;
    }
    return ILLM_OK;
}

static bool rows_args_ok(const void* X, const void* Wt, const void* Y, int M, int N, int K,
                         const float* ssq, int parts) {
    return X && Wt && Y && M > 0 && M <= 128 && N > 0 && K > 0 &&
           K % 64 == 0 && (!ssq || (parts > 0 && M <= 16));
}

extern "C" int illm_gemm_rows_bf16(const void* X, const void* Wt, void* Y, int y_dt, int M, int N,
                                   int K, const float* ssq, int parts, float eps, void* stream) {
    if (!rows_args_ok(X, Wt, Y, M, N, K, ssq, parts) || !illm_dtype_ok(y_dt)) return ILLM_ERR_ARG;
    const GrScale scale = {ssq, parts, eps};
    return rows_product<GR_PLAIN>(X, Wt, Y, y_dt, M, N, K, (N + 15) / 16, GrRope(), scale,
                                  (hipStream_t)stream);
}

extern "C" int illm_gemm_rows_gateup_silu(const void* X, const void* Wt, void* Y, int y_dt, int M,
                                          int F, int K, const float* ssq, int parts, float eps,
                                          void* stream) {
    if (!rows_args_ok(X, Wt, Y, M, F, K, ssq, parts) || !illm_dtype_ok(y_dt)) return ILLM_ERR_ARG;
    const GrScale scale = {ssq, parts, eps};
    return rows_product<GR_GATE_UP>(X, Wt, Y, y_dt, M, F, K, (F + 7) / 8, GrRope(), scale,
                                    (hipStream_t)stream);
}

extern "C" int illm_qkv_rope_store_rows(const void* X, const void* Wt, void* Y, int M, int K,
                                        const float* cos_sin, int max_pos, const int32_t* row_pos,
                                        const int32_t* row_slot, void* kcache, void* vcache,
                                        const int32_t* page_table, int table_stride, int page_size,
                                        int ring, int nh, int nkv, int hd, const float* ssq,
                                        int parts, float eps, void* stream) {
    const int N = (nh + 2 * nkv) * hd;
    if (!rows_args_ok(X, Wt, Y, M, N, K, ssq, parts) || !cos_sin || max_pos <= 0 || !row_pos ||
        !row_slot || !kcache || !vcache || !page_table || table_stride <= 0 || page_size <= 0 ||
        nh <= 0 || nkv <= 0 || hd <= 0 || hd % 16)
        return ILLM_ERR_ARG;
    const GrRope rope = {cos_sin, row_pos, row_slot, (bf16_t*)kcache, (bf16_t*)vcache, page_table,
                         table_stride, page_size, ring, nh, nkv, hd};
    const GrScale scale = {ssq, parts, eps};
    return rows_product<GR_QKV_ROPE>(X, Wt, Y, ILLM_BF16, M, N, K, N / 16, rope, scale,
                                     (hipStream_t)stream);
}

// Y[M, N] = X[M, K] . W[N, K]^T for up to 128 rows (decoding larger batches), bfloat16 operands,
// float32 accumulation on the matrix cores, from the tiled copy of W
// ([tile of 16 rows][K / 32][16 rows][32 k], see gemm_skinny.hip).
//
// With this many rows the few-rows kernel, whose waves each read X for themselves, is bound by
// X: every 16 rows of W bring all of X through the cache again (measured: time grows in
// proportion to M).  Here the four waves of a block take four neighbouring tiles of W over the
// same range of k, and X comes to them through LDS once per block: a piece of 128 k of all rows,
// written as it is loaded (16-byte units, swizzled within their row by the row's number so that
// both the write and the operand-order read are free of bank conflicts) and double-buffered, one
// barrier per piece.  A wave may take two tiles (NTB), which halves what is read from LDS and
// through the cache per byte of W.  W is streamed from the tiled copy straight into operand registers, one
// piece ahead.  K is split over blockIdx.y so that a matrix with few rows still fills the chip;
// each split writes its float32 sums to its own plane of Y ([splits][M][N]) and the kernel that
// uses them adds the planes in order, so the result has a fixed order of summation.
//
// The reference has one GEMM for every number of rows (cublasSgemm,
// src/kern/gpu/kernel_gpu.cu:420-435).
#include "api.h"
#include "api_test.h"
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define MID_PIECE_STEPS 4      // k-steps of 32 in a piece

template <int MT, int NTB>
__global__ void __launch_bounds__(256)
gemm_mid_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ Wt, void* __restrict__ Y,
                int y_dt, int M, int N, int K, int pieces_per_split, size_t plane_stride) {
    __shared__ uint4 xs[2][MT * 256];    // [buffer][row][16 units of 8 k]
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int r = lane & 15, q = lane >> 4;
    const int ksteps = K / 32;
    const int tiles = (N + 15) / 16;
    const int tile0 = (blockIdx.x * 4 + wave) * NTB;     // this wave's NTB tiles: tile0 ..
    const int pieces = (ksteps + MID_PIECE_STEPS - 1) / MID_PIECE_STEPS;
    const int p_begin = blockIdx.y * pieces_per_split;
    int p_end = p_begin + pieces_per_split;
    p_end = p_end < pieces ? p_end : pieces;

    // staging of X: thread t brings unit t % 16 of rows t / 16 + 16 j; rows >= M read row M - 1
    // and their results are dropped
    const int x_unit = threadIdx.x & 15, x_row = threadIdx.x >> 4;
    const bf16_t* xsrc[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) {
        int m = 16 * j + x_row;
        m = m < M ? m : M - 1;
        xsrc[j] = X + (size_t)m * K + x_unit * 8;
    }
    const int x_dst = x_row * 16 + (x_unit ^ x_row);
    const bf16_t* wsrc = Wt + (size_t)tile0 * ksteps * 512 + (r * 4 + q) * 8;
    bool tile_ok[NTB];
#pragma unroll
    for (int nt = 0; nt < NTB; ++nt) tile_ok[nt] = tile0 + nt < tiles;

    auto load_x = [&](int p, uint4 (&xg)[MT]) {
        const bool in = p * 128 + x_unit * 8 < K;
#pragma unroll
        for (int j = 0; j < MT; ++j)
            xg[j] = in ? *(const uint4*)(xsrc[j] + (size_t)p * 128) : make_uint4(0, 0, 0, 0);
    };
    auto load_w = [&](int p, uint4 (&a)[NTB][MID_PIECE_STEPS]) {
#pragma unroll
        for (int nt = 0; nt < NTB; ++nt)
#pragma unroll
            for (int u = 0; u < MID_PIECE_STEPS; ++u) {
                const int s = p * MID_PIECE_STEPS + u;
                a[nt][u] = (tile_ok[nt] && s < ksteps)
                               ? ld16_stream(wsrc + ((size_t)nt * ksteps + s) * 512)
                               : make_uint4(0, 0, 0, 0);
            }
    };

    f32x4_t acc[NTB][MT];
#pragma unroll
    for (int nt = 0; nt < NTB; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    uint4 xg[MT], a[NTB][MID_PIECE_STEPS];
    if (p_begin < p_end) {
        load_x(p_begin, xg);
        load_w(p_begin, a);
    }
    int buf = 0;
    for (int p = p_begin; p < p_end; ++p) {
#pragma unroll
        for (int j = 0; j < MT; ++j) xs[buf][j * 256 + x_dst] = xg[j];
        // one barrier a piece is enough with two buffers: whoever writes buffer `buf` again, two
        // pieces on, has passed the next piece's barrier, which every wave reaches only after it
        // has finished reading this one
        __syncthreads();
        uint4 an[NTB][MID_PIECE_STEPS];
        const bool more = p + 1 < p_end;
        if (more) {
            load_x(p + 1, xg);
            load_w(p + 1, an);
        }
#pragma unroll
        for (int u = 0; u < MID_PIECE_STEPS; ++u)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint4 b = xs[buf][(mt * 16 + r) * 16 + ((u * 4 + q) ^ r)];
#pragma unroll
                for (int nt = 0; nt < NTB; ++nt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        *(const bf16x8_t*)&a[nt][u], *(const bf16x8_t*)&b, acc[nt][mt], 0, 0, 0);
            }
        if (more) {
#pragma unroll
            for (int nt = 0; nt < NTB; ++nt)
#pragma unroll
                for (int u = 0; u < MID_PIECE_STEPS; ++u) a[nt][u] = an[nt][u];
        }
        buf ^= 1;
    }
    // acc[nt][mt][i] = sum for X row mt * 16 + r and W row (tile0 + nt) * 16 + 4 q + i
    const bool planes = gridDim.y > 1;
    const int dt = planes ? ILLM_F32 : y_dt;
    const size_t plane = planes ? (size_t)blockIdx.y * plane_stride : 0;
#pragma unroll
    for (int nt = 0; nt < NTB; ++nt) {
        if (!tile_ok[nt]) continue;
        const int n0 = (tile0 + nt) * 16 + q * 4;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            if (m >= M) continue;
            const f32x4_t v = acc[nt][mt];
            const size_t at = plane + (size_t)m * N + n0;
            if (n0 + 3 < N && (N & 3) == 0) {
                if (dt == ILLM_F32)
                    *(float4*)((float*)Y + at) = make_float4(v[0], v[1], v[2], v[3]);
                else
                    *(uint2*)((bf16_t*)Y + at) =
                        make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n0 + i < N) st_f(Y, dt, at + i, v[i]);
            }
        }
    }
}

// Tiles of 16 W rows a wave takes: two when the matrix has at least 512 tiles, where reading
// X from LDS once for two tiles pays (measured at 17 to 64 rows).  Splits of K: about
// MID_BLOCKS_WANTED blocks on the chip, the pieces spread evenly (no split is left empty),
// every split at least two pieces long.
static const int MID_BLOCKS_WANTED = 512;
static int MID_TILES_PER_WAVE = 0;       // 0: by the number of tiles; 1 or 2: forced (tuning)
extern "C" void illm_set_mid_tiles_per_wave(int n) { MID_TILES_PER_WAVE = (n == 1 || n == 2) ? n : 0; }

static int MID_ROWS_A_LAUNCH = 128;      // tuning and tests: 64 or 128 rows of X a launch
extern "C" void illm_set_mid_rows_a_launch(int rows) { MID_ROWS_A_LAUNCH = rows == 64 ? 64 : 128; }

static int mid_ntb(int N) {
    return MID_TILES_PER_WAVE ? MID_TILES_PER_WAVE : ((N + 15) / 16 >= 512 ? 2 : 1);
}

static int mid_blocks_x(int N) {
    const int per_block = 4 * mid_ntb(N);
    return ((N + 15) / 16 + per_block - 1) / per_block;
}

extern "C" int illm_gemm_mid_splits(int N, int K) {
    const int bx = mid_blocks_x(N);
    const int pieces = (K / 32 + MID_PIECE_STEPS - 1) / MID_PIECE_STEPS;
    int s = (MID_BLOCKS_WANTED + bx / 2) / bx;
    s = s > pieces / 2 ? pieces / 2 : s;
    s = s < 1 ? 1 : s;
    const int per = (pieces + s - 1) / s;
    return (pieces + per - 1) / per;
}

// Takes bfloat16 X [M, K] with M in 1..128 and the tiled copy Wt of W [N, K], K a multiple of 32.  splits == 1: Y is [M, N] of y_dt.
// splits > 1: Y is float32 [splits][M][N], whose planes the caller adds up.  Otherwise
// ILLM_ERR_ARG.
extern "C" int illm_gemm_mid_bf16(const void* X, const void* Wt, void* Y, int y_dt, int M, int N,
                                  int K, int splits, void* stream) {
    if (M <= 0 || M > 128 || N <= 0 || K <= 0 || (K % 32) || splits < 1 || !illm_dtype_ok(y_dt) ||
        !X || !Wt || !Y)
        return ILLM_ERR_ARG;
    const int pieces = (K / 32 + MID_PIECE_STEPS - 1) / MID_PIECE_STEPS;
    if (splits > pieces) return ILLM_ERR_ARG;
    const int per = (pieces + splits - 1) / splits;
    const dim3 grid(mid_blocks_x(N), splits);
    hipStream_t st = (hipStream_t)stream;
    const int ntb = mid_ntb(N);
    const size_t y_elem = (splits > 1 || y_dt == ILLM_F32) ? 4 : 2;
    const size_t plane_stride = (size_t)M * N;
    const int a_launch = MID_ROWS_A_LAUNCH;
    for (int m0 = 0; m0 < M; m0 += a_launch) {
        const int rows = M - m0 < a_launch ? M - m0 : a_launch;
        const int mt = (rows + 15) / 16;
        const bf16_t* x = (const bf16_t*)X + (size_t)m0 * K;
        void* y = (char*)Y + (size_t)m0 * N * y_elem;
        bool launched = false;
#define GO(MT_, NTB_)                                                                         \
        if (mt == MT_ && ntb == NTB_) {                                                       \
            hipLaunchKernelGGL((gemm_mid_kernel<MT_, NTB_>), grid, dim3(256), 0, st, x,       \
                               (const bf16_t*)Wt, y, y_dt, rows, N, K, per, plane_stride);    \
            launched = true;                                                                  \
        }
        GO(1, 1) GO(2, 1) GO(3, 1) GO(4, 1) GO(1, 2) GO(2, 2) GO(3, 2) GO(4, 2)
        GO(5, 1) GO(6, 1) GO(7, 1) GO(8, 1) GO(5, 2) GO(6, 2) GO(7, 2) GO(8, 2)
#undef GO
        if (!launched) return ILLM_ERR_ARG;
        const int rc = illm_launch_status();
        if (rc != ILLM_OK) return rc;
    }
    return ILLM_OK;
}

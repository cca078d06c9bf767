// Y[M, N] = X[M, K] . W[N, K]^T for any sizes and any mix of float32 / bfloat16
// storage, accumulated in float32 with plain multiply-adds (no matrix cores, no
// reduced-precision mode).  Each output element is summed over k in ascending
// order, whatever its row's place in the batch, so a row gives the same bits
// whether it comes alone or among others.  This is the matrix product of the
// 32-bit path and the fallback for shapes the MFMA kernels do not take.  Two more
// kernels below serve the 32-bit path's common cases faster, both in float32
// throughout: few rows (W read once) and many rows (the matrix cores' float32
// instruction).
//
// The reference's float product is the same sum (src/kern/naive/naive.cpp:363-379);
// its GPU path calls cublasSgemm (src/kern/gpu/kernel_gpu.cu:420-435).
#include "api.h"
#include "api_test.h"
#include "common.h"

#define GT 64   // tile of outputs per block (GT x GT)
#define GK 16   // depth of a k step

__global__ void __launch_bounds__(256)
gemm_generic_kernel(const void* __restrict__ X, int x_dt, const void* __restrict__ W, int w_dt,
                    void* __restrict__ Y, int y_dt, int M, int N, int K) {
    __shared__ float xs[GK][GT + 1];
    __shared__ float ws[GK][GT + 1];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GK) {
        // 64 rows x 16 k per operand, 1024 elements, 4 per thread
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int idx = threadIdx.x + e * 256;
            const int r = idx >> 4, kk = idx & 15;
            const int k = k0 + kk;
            const int m = m0 + r, n = n0 + r;
            xs[kk][r] = (m < M && k < K) ? ld_f(X, x_dt, (size_t)m * K + k) : 0.f;
            ws[kk][r] = (n < N && k < K) ? ld_f(W, w_dt, (size_t)n * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) st_f(Y, y_dt, (size_t)m * N + n, acc[i][j]);
        }
    }
}

extern "C" int illm_gemm_generic(const void* X, int x_dt, const void* W, int w_dt, void* Y,
                                 int y_dt, int M, int N, int K, void* stream) {
    if (M < 0 || N <= 0 || K <= 0 || !illm_dtype_ok(x_dt) || !illm_dtype_ok(w_dt) ||
        !illm_dtype_ok(y_dt))
        return ILLM_ERR_ARG;
    if (M == 0) return ILLM_OK;
    const int gy = (M + GT - 1) / GT;
    if (gy > 65535) return ILLM_ERR_ARG;
    hipLaunchKernelGGL(gemm_generic_kernel, dim3((N + GT - 1) / GT, gy), dim3(256), 0,
                       (hipStream_t)stream, X, x_dt, W, w_dt, Y, y_dt, M, N, K);
    return illm_launch_status();
}


// ---------------------------------------------------------------- many rows, float32
// The same product for float32 X and W with K a multiple of 16, on the matrix cores' float32
// instruction (MFMA 32x32x2: float32 operands, float32 products and sums; nothing is rounded to
// a shorter type).  The multiply-add tile above reaches 45 TFLOP/s, 0.57 of what the vector units
// give without packed instructions; the matrix cores' float32 rate is twice the vector units'.
// A block of four waves takes 128 x 128 outputs, a wave 64 x 64 (2 x 2 MFMA tiles); both
// operands go through LDS k-major (16 k a stage, two buffers, the next stage's loads in flight
// while this one is multiplied).  The MFMA's rows are W's (n) and its columns X's (m), so a lane
// holds 4 consecutive n of one m: 16-byte stores.  An output element is summed over k in
// ascending pairs whatever its row's place in the batch.
typedef float f32x16_t __attribute__((ext_vector_type(16)));

#define FM_T 128     // outputs of a block along m and along n
#define FM_K 16      // k a stage
#define FM_LD 130    // LDS row stride in floats (4 * FM_LD = 8 mod 32: the stores of a half-wave,
                     // 8 rows x 4 k-quads, fall into 32 different banks)

__global__ void __launch_bounds__(256)
gemm_f32_mfma_kernel(const float* __restrict__ X, const float* __restrict__ W, void* __restrict__ Y,
                     int y_dt, int M, int N, int K) {
    __shared__ float xs[2][FM_K][FM_LD];
    __shared__ float ws[2][FM_K][FM_LD];
    const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
    const int r = lane & 31, kh = lane >> 5;
    const int wm = wave & 1, wn = wave >> 1;
    const int m0 = blockIdx.y * FM_T, n0 = blockIdx.x * FM_T;

    // staging: thread t brings 4 k (quad t % 4) of rows t / 4 and t / 4 + 64 of both operands;
    // rows beyond the matrix read its last row (their outputs are not stored)
    const int s_row = tid >> 2, s_kq = tid & 3;
    const float* xsrc[2];
    const float* wsrc[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        xsrc[e] = X + (size_t)min(m0 + s_row + 64 * e, M - 1) * K + s_kq * 4;
        wsrc[e] = W + (size_t)min(n0 + s_row + 64 * e, N - 1) * K + s_kq * 4;
    }
    float4 xg[2], wg[2];
    auto fetch = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            xg[e] = *(const float4*)(xsrc[e] + k0);
            wg[e] = *(const float4*)(wsrc[e] + k0);
        }
    };
    auto stage = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int row = s_row + 64 * e;
            xs[buf][s_kq * 4 + 0][row] = xg[e].x; xs[buf][s_kq * 4 + 1][row] = xg[e].y;
            xs[buf][s_kq * 4 + 2][row] = xg[e].z; xs[buf][s_kq * 4 + 3][row] = xg[e].w;
            ws[buf][s_kq * 4 + 0][row] = wg[e].x; ws[buf][s_kq * 4 + 1][row] = wg[e].y;
            ws[buf][s_kq * 4 + 2][row] = wg[e].z; ws[buf][s_kq * 4 + 3][row] = wg[e].w;
        }
    };
    f32x16_t acc[2][2];                    // [n tile][m tile]
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    fetch(0);
    stage(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += FM_K, buf ^= 1) {
        const bool more = k0 + FM_K < K;
        if (more) fetch(k0 + FM_K);
#pragma unroll
        for (int s = 0; s < FM_K / 2; ++s) {
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = ws[buf][2 * s + kh][wn * 64 + 32 * i + r];
#pragma unroll
            for (int j = 0; j < 2; ++j) b[j] = xs[buf][2 * s + kh][wm * 64 + 32 * j + r];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (more) stage(buf ^ 1);          // (last read before the barrier that ended the stage before)
        __syncthreads();
    }
    // acc[i][j][v]: n = n0 + wn * 64 + 32 i + 8 (v / 4) + 4 kh + v % 4, m = m0 + wm * 64 + 32 j + r
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int m = m0 + wm * 64 + 32 * j + r;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * 64 + 32 * i + 8 * g + 4 * kh;
                const size_t at = (size_t)m * N + n;
                if (n + 3 < N && (N & 3) == 0 && y_dt == ILLM_F32) {
                    *(float4*)((float*)Y + at) = make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1],
                                                             acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (n + v < N) st_f(Y, y_dt, at + v, acc[i][j][4 * g + v]);
                }
            }
    }
}

// float32 X [M, K] and W [N, K], K % 16 == 0; Y float32 or bfloat16.  Else ILLM_ERR_ARG.
extern "C" int illm_gemm_f32_mfma(const float* X, const float* W, void* Y, int y_dt, int M, int N,
                                  int K, void* stream) {
    if (M <= 0 || N <= 0 || K <= 0 || (K % FM_K) || !illm_dtype_ok(y_dt) || !X || !W || !Y)
        return ILLM_ERR_ARG;
    const int gy = (M + FM_T - 1) / FM_T;
    if (gy > 65535) return ILLM_ERR_ARG;
    hipLaunchKernelGGL(gemm_f32_mfma_kernel, dim3((N + FM_T - 1) / FM_T, gy), dim3(256), 0,
                       (hipStream_t)stream, X, W, Y, y_dt, M, N, K);
    return illm_launch_status();
}


// ---------------------------------------------------------------- up to 128 rows, float32
// The same product for up to 128 float32 rows and K a multiple of 32, bound by reading W once:
// MFMA 16x16x4 float32 with operands straight from memory.  A block of 8 waves takes 16 rows of
// W; the waves take pieces of 32 k in turn (wave w pieces w, w + 8, ...: eight neighbouring
// 128-byte segments of a row at a time).  Lane l reads 16 bytes at k = 4 (l / 16) + 16 q of row
// l % 16, of W and of every 16 rows of X alike: element j of that load is the operand of an
// MFMA whose four k are 4 g + j + 16 q, the same four for both operands, so nothing is
// permuted.  The waves' sums are added through LDS in wave order: the order of a sum depends on
// K only, not on the row's place or on the number of rows.
typedef float f32x4v_t __attribute__((ext_vector_type(4)));

template <int RT, int CT>                      // tiles of 16 rows of X, tiles of 16 rows of W
__global__ void __launch_bounds__(512)
gemm_rows_f32_mfma_kernel(const float* __restrict__ X, const float* __restrict__ W, void* __restrict__ Y,
                          int y_dt, int M, int N, int K) {
    __shared__ f32x4v_t part[8][RT * CT][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
    const int r16 = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16 * CT;
    const float* wsrc[CT];
#pragma unroll
    for (int c = 0; c < CT; ++c) wsrc[c] = W + (size_t)min(n0 + 16 * c + r16, N - 1) * K + 4 * g;
    const float* xsrc[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) xsrc[t] = X + (size_t)min(16 * t + r16, M - 1) * K + 4 * g;
    f32x4v_t acc[RT][CT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int c = 0; c < CT; ++c) acc[t][c] = (f32x4v_t){0.f, 0.f, 0.f, 0.f};
    constexpr int U = RT * CT <= 2 ? 4 : (RT <= 4 ? 2 : 1);   // pieces asked for together
    const int pieces = K / 32;
    for (int p = wave; p < pieces; p += 8 * U) {
        f32x4v_t wr[U][CT][2], xr[U][RT][2];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k0 = 32 * min(p + 8 * u, pieces - 1);      // (past the end: a piece read again, not used)
#pragma unroll
            for (int q = 0; q < 2; ++q) {
#pragma unroll
                for (int c = 0; c < CT; ++c)
                    wr[u][c][q] = __builtin_nontemporal_load((const f32x4v_t*)(wsrc[c] + k0 + 16 * q));
#pragma unroll
                for (int t = 0; t < RT; ++t) xr[u][t][q] = *(const f32x4v_t*)(xsrc[t] + k0 + 16 * q);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (p + 8 * u < pieces) {
#pragma unroll
                for (int q = 0; q < 2; ++q)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int t = 0; t < RT; ++t)
#pragma unroll
                            for (int c = 0; c < CT; ++c)
                                acc[t][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(wr[u][c][q][j], xr[u][t][q][j],
                                                                                 acc[t][c], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int c = 0; c < CT; ++c) part[wave][t * CT + c][lane] = acc[t][c];
    __syncthreads();
    // acc[t][c][v]: n = n0 + 16 c + 4 g + v, m = 16 t + r16; a thread adds the eight waves' sums
    for (int e = tid; e < RT * CT * 64; e += 512) {
        const int tc = e >> 6, l = e & 63;
        f32x4v_t sum = part[0][tc][l];
#pragma unroll
        for (int w = 1; w < 8; ++w) sum += part[w][tc][l];
        const int m = 16 * (tc / CT) + (l & 15), n = n0 + 16 * (tc % CT) + 4 * (l >> 4);
        if (m >= M) continue;
        const size_t at = (size_t)m * N + n;
        if (n + 3 < N && (N & 3) == 0 && y_dt == ILLM_F32) {
            *(f32x4v_t*)((float*)Y + at) = sum;
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (n + v < N) st_f(Y, y_dt, at + v, sum[v]);
        }
    }
}

static int g_rows_f32_tiles = 0;     // tests: W tiles a block (1 or 2); 0: the library's choice
extern "C" void illm_set_rows_f32_tiles(int tiles) { g_rows_f32_tiles = tiles == 1 || tiles == 2 ? tiles : 0; }

// float32 X [M <= 128, K] and W [N, K], K % 32 == 0; Y float32 or bfloat16.  Else ILLM_ERR_ARG.
extern "C" int illm_gemm_rows_f32_mfma(const float* X, const float* W, void* Y, int y_dt, int M, int N,
                                       int K, void* stream) {
    if (M <= 0 || M > 128 || N <= 0 || K <= 0 || (K % 32) || !illm_dtype_ok(y_dt) || !X || !W || !Y)
        return ILLM_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    // two tiles of W a block halve what the blocks read of X together: from 17 rows on, where
    // that is most of the traffic, if there are still two blocks for every compute unit
    // (measured at 64 rows: 22016 x 4096 263 -> 204 us, 12288 x 4096 the same, 4096 x 4096 49 -> 65)
    const int rt = (M + 15) / 16;
    const int ct = g_rows_f32_tiles ? g_rows_f32_tiles : (rt >= 2 && N >= 32 * 512 ? 2 : 1);
    const dim3 grid((N + 16 * ct - 1) / (16 * ct)), block(512);
#define ILLM_ROWS_F32(RT)                                                                             \
    case RT:                                                                                          \
        if (ct == 2)                                                                                  \
            hipLaunchKernelGGL((gemm_rows_f32_mfma_kernel<RT, 2>), grid, block, 0, st, X, W, Y, y_dt, M, N, K); \
        else                                                                                          \
            hipLaunchKernelGGL((gemm_rows_f32_mfma_kernel<RT, 1>), grid, block, 0, st, X, W, Y, y_dt, M, N, K); \
        break;
    switch (rt) {
        ILLM_ROWS_F32(1) ILLM_ROWS_F32(2) ILLM_ROWS_F32(3) ILLM_ROWS_F32(4)
        ILLM_ROWS_F32(5) ILLM_ROWS_F32(6) ILLM_ROWS_F32(7) ILLM_ROWS_F32(8)
    }
#undef ILLM_ROWS_F32
    return illm_launch_status();
}


// ---------------------------------------------------------------- few rows, float32
// The same product for M <= 16 rows of float32 X and float32 W (decoding on the 32-bit path),
// bound by reading W once: a block of 4 waves takes R = 64 / MR rows of W (MR = M rounded up to
// 8 or 16), the waves split K in interleaved pieces of 256, a lane multiplies 4 consecutive k
// of every W row with every X row (plain multiply-adds, float32), and the R * MR sums of a wave
// are added over its lanes by a halving exchange that leaves sum number l in lane l.  The waves'
// sums are added in wave order.  The order of a sum depends on K only, not on the row's place.
template <int MR>
__global__ void __launch_bounds__(256)
gemv_rows_f32_kernel(const float* __restrict__ X, const float* __restrict__ W, void* __restrict__ Y,
                     int y_dt, int M, int N, int K) {
    constexpr int R = 64 / MR;
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, wave = wave_index();
    const int n0 = blockIdx.x * R;
    const float* wrow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wrow[r] = W + (size_t)min(n0 + r, N - 1) * K;
    float acc[R][MR];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[r][m] = 0.f;

    for (int k = (wave * 64 + lane) * 4; k < K; k += 4 * 256) {      // K is a multiple of 4
        f32x4v_t w[R];                                   // (W is used once: loads that do not stay in the caches)
#pragma unroll
        for (int r = 0; r < R; ++r) w[r] = __builtin_nontemporal_load((const f32x4v_t*)(wrow[r] + k));
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            const float4 x = *(const float4*)(X + (size_t)min(m, M - 1) * K + k);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float a = acc[r][m];
                a = fmaf(w[r].x, x.x, a);
                a = fmaf(w[r].y, x.y, a);
                a = fmaf(w[r].z, x.z, a);
                a = fmaf(w[r].w, x.w, a);
                acc[r][m] = a;
            }
        }
    }
    // 64 sums over 64 lanes: at the step that pairs lanes l and l ^ b a lane keeps the sums
    // whose number has l's bit b; sum number e = r * MR + m ends in lane e
    float v[64];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) v[r * MR + m] = acc[r][m];
#pragma unroll
    for (int b = 1, n = 32; b < 64; b <<= 1, n >>= 1) {
        const bool up = (lane & b) != 0;
#pragma unroll
        for (int i = 0; i < n; ++i) {
            const float keep = up ? v[2 * i + 1] : v[2 * i];
            const float send = up ? v[2 * i] : v[2 * i + 1];
            v[i] = keep + __shfl_xor(send, b, ILLM_WAVE);
        }
    }
    part[wave][lane] = v[0];
    __syncthreads();
    if (wave == 0) {
        const float t = ((part[0][lane] + part[1][lane]) + part[2][lane]) + part[3][lane];
        const int r = lane / MR, m = lane % MR;
        if (m < M && n0 + r < N) st_f(Y, y_dt, (size_t)m * N + n0 + r, t);
    }
}

// float32 X [M <= 16, K] and W [N, K], K % 4 == 0; Y float32 or bfloat16.  Else ILLM_ERR_ARG.
extern "C" int illm_gemv_rows_f32(const float* X, const float* W, void* Y, int y_dt, int M, int N,
                                  int K, void* stream) {
    if (M <= 0 || M > 16 || N <= 0 || K <= 0 || (K % 4) || !illm_dtype_ok(y_dt)) return ILLM_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    // (a block of 16 rows of W for up to 4 rows of X was slower than this one of 8 at three of
    // the four 7B shapes: 72 against 60 us for 22016 x 4096, 34 against 36 for 4096 x 11008)
    if (M <= 8)
        hipLaunchKernelGGL(gemv_rows_f32_kernel<8>, dim3((N + 7) / 8), dim3(256), 0, st, X, W, Y, y_dt, M, N, K);
    else
        hipLaunchKernelGGL(gemv_rows_f32_kernel<16>, dim3((N + 3) / 4), dim3(256), 0, st, X, W, Y, y_dt, M, N, K);
    return illm_launch_status();
}

// Y[M, N] = X[M, K] . W[N, K]^T for any sizes and any mix of float32 / bfloat16
// storage, accumulated in float32 with plain multiply-adds (no matrix cores, no
// reduced-precision mode).  Each output element is summed over k in ascending
// order, whatever its row's place in the batch, so a row gives the same bits
// whether it comes alone or among others.  This is the matrix product of the
// 32-bit path and the fallback for shapes the MFMA kernels do not take.
//
// The reference's float product is the same sum (src/kern/naive/naive.cpp:363-379);
// its GPU path calls cublasSgemm (src/kern/gpu/kernel_gpu.cu:420-435).
#include "api.h"
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


// ---------------------------------------------------------------- few rows, float32
// The same product for M <= 16 rows of float32 X and float32 W (decoding on the 32-bit path),
// bound by reading W once: a block of 4 waves takes R = 64 / MR rows of W (MR = M rounded up to
// 4, 8 or 16), the waves split K in interleaved pieces of 256, a lane multiplies 4 consecutive k
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
        float4 w[R];
#pragma unroll
        for (int r = 0; r < R; ++r) w[r] = *(const float4*)(wrow[r] + k);
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
    if (M <= 4)
        hipLaunchKernelGGL(gemv_rows_f32_kernel<4>, dim3((N + 15) / 16), dim3(256), 0, st, X, W, Y, y_dt, M, N, K);
    else if (M <= 8)
        hipLaunchKernelGGL(gemv_rows_f32_kernel<8>, dim3((N + 7) / 8), dim3(256), 0, st, X, W, Y, y_dt, M, N, K);
    else
        hipLaunchKernelGGL(gemv_rows_f32_kernel<16>, dim3((N + 3) / 4), dim3(256), 0, st, X, W, Y, y_dt, M, N, K);
    return illm_launch_status();
}

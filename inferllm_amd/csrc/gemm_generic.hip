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

// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wave (64 lanes) and block reductions, launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define ILLM_F32 0
#define ILLM_BF16 1

#define ILLM_OK 0
#define ILLM_ERR_ARG 1      // a size or dtype the kernel does not take
#define ILLM_ERR_LAUNCH 2   // the runtime refused the launch
#define ILLM_ERR_SCRATCH 3  // the call needs more of the library's own scratch memory than it has

#define ILLM_WAVE 64

typedef uint16_t bf16_t;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

typedef __bf16 illm_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float illm_f32x2_t __attribute__((ext_vector_type(2)));

// two floats to two bfloat16 (a in the low half), round to nearest even, by the
// hardware's packed conversion (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    const illm_f32x2_t v = {a, b};
    const illm_bf16x2_t r = __builtin_convertvector(v, illm_bf16x2_t);
    return *(const uint32_t*)&r;
}

__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    return (bf16_t)(pack_bf16x2(f, 0.f) & 0xffffu);
}

__device__ __forceinline__ float ld_f(const void* p, int dt, size_t i) {
    return dt == ILLM_BF16 ? bf16_to_f32(((const bf16_t*)p)[i]) : ((const float*)p)[i];
}

__device__ __forceinline__ void st_f(void* p, int dt, size_t i, float v) {
    if (dt == ILLM_BF16) ((bf16_t*)p)[i] = f32_to_bf16(v);
    else ((float*)p)[i] = v;
}

typedef uint32_t illm_u32x4_t __attribute__((ext_vector_type(4)));

// 16 bytes of data that is read once (weights, cache rows): a non-temporal load, which keeps
// the stream out of the way of lines that are used again.  Use it where an instruction reads
// whole 128-byte lines; a line read in halves by two such loads is fetched twice.
__device__ __forceinline__ uint4 ld16_stream(const void* p) {
    const illm_u32x4_t v = __builtin_nontemporal_load((const illm_u32x4_t*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// The wave's number within its block, as a value the compiler knows to be the same in all
// lanes: loops and branches on it run on the scalar unit instead of under lane masks.
__device__ __forceinline__ int wave_index() {
    return __builtin_amdgcn_readfirstlane((int)(threadIdx.x / ILLM_WAVE));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = ILLM_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, ILLM_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = ILLM_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, ILLM_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; `red` holds 16 floats of LDS.  Every
// thread gets the result; the order of the additions is fixed by the block size.
__device__ __forceinline__ float block_sum(float v, float* red) {
    const int lane = threadIdx.x & (ILLM_WAVE - 1), w = threadIdx.x / ILLM_WAVE;
    const int nw = (blockDim.x + ILLM_WAVE - 1) / ILLM_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}

__device__ __forceinline__ float block_max(float v, float* red) {
    const int lane = threadIdx.x & (ILLM_WAVE - 1), w = threadIdx.x / ILLM_WAVE;
    const int nw = (blockDim.x + ILLM_WAVE - 1) / ILLM_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
    return t;
}

static inline int illm_launch_status() {
    return hipGetLastError() == hipSuccess ? ILLM_OK : ILLM_ERR_LAUNCH;
}

static inline bool illm_dtype_ok(int dt) { return dt == ILLM_F32 || dt == ILLM_BF16; }

// Where position `pos` of the sequence in `slot` lies in a paged cache line laid
// out as [page][kv head][row in page][head_dim].  `ring` > 0: only the last
// `ring` logical pages of a sequence are kept (a window).
__device__ __forceinline__ size_t cache_row_offset(const int32_t* page_table, int table_stride,
                                                   int slot, int pos, int page_size, int ring,
                                                   int nkv, int kvh, int hd) {
    int lp = pos / page_size;
    if (ring > 0) lp %= ring;
    const int phys = page_table[(size_t)slot * table_stride + lp];
    return (((size_t)phys * nkv + kvh) * page_size + (pos % page_size)) * (size_t)hd;
}

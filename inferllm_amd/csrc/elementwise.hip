// Row-wise kernels: embedding rows, residual add + RMS norm, SiLU-multiply,
// rotation of q/k with the store of k/v into the paged cache.
//
// Formulas as the reference computes them: embedding row copy
// (src/kern/naive/naive.cpp:43-54), RMS norm = x * 1/sqrt(mean(x^2) + eps), then
// the weight (naive.cpp:186-207, src/core/op.cpp:37-47), silu(x) = x / (1 + exp(-x))
// (naive.cpp:80-89), rotation of pairs (i, i + hd/2) by pos * base^(-2i/rot)
// (naive.cpp:389-414) or of pairs (2i, 2i+1) (naive.cpp:415-440).  The reference
// runs each as a kernel of its own (src/kern/gpu/kernel_gpu.cu:127-148, :260-294,
// :183-258, :343-401); here the residual add is fused with the norm and the cache
// store with the rotation.
#include "api.h"
#include "common.h"

// ---------------------------------------------------------------- embedding
__global__ void embed_kernel(const int32_t* __restrict__ tokens, const void* __restrict__ table,
                             int table_dt, float* __restrict__ out, int E, int V) {
    const int t = blockIdx.x;
    int id = tokens[t];
    id = id < 0 ? 0 : (id >= V ? V - 1 : id);
    const size_t src = (size_t)id * E, dst = (size_t)t * E;
    for (int i = threadIdx.x; i < E; i += blockDim.x) out[dst + i] = ld_f(table, table_dt, src + i);
}

extern "C" int illm_embed(const int32_t* tokens, const void* table, int table_dt, float* out,
                          int T, int E, int V, void* stream) {
    if (T < 0 || E <= 0 || V <= 0 || !illm_dtype_ok(table_dt)) return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    hipLaunchKernelGGL(embed_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, tokens, table,
                       table_dt, out, E, V);
    return illm_launch_status();
}

// ---------------------------------------------------------------- add + rmsnorm
// One block per row.  The sum of squares is taken in float32 in an order that
// depends on E and the block size only, never on the row's place in the batch.
// `delta` may be `planes` arrays of the same shape, `plane_stride` elements apart (the sums of
// a product whose K was split): they are added in order.
__device__ __forceinline__ float ld_planes(const void* delta, int dt, size_t i, int planes,
                                           size_t plane_stride) {
    float d = ld_f(delta, dt, i);
    for (int s = 1; s < planes; ++s) d += ld_f(delta, dt, i + s * plane_stride);
    return d;
}

__global__ void add_rmsnorm_kernel(float* __restrict__ x, const void* __restrict__ delta,
                                   int delta_dt, int planes, size_t plane_stride,
                                   const void* __restrict__ w, int w_dt,
                                   void* __restrict__ out, int out_dt,
                                   const int32_t* __restrict__ row_idx, int E, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const int in_row = row_idx ? row_idx[r] : r;
    const size_t ib = (size_t)in_row * E, ob = (size_t)r * E;
    float ss = 0.f;
    for (int i = threadIdx.x; i < E; i += blockDim.x) {
        float v = x[ib + i];
        if (delta) {
            v += ld_planes(delta, delta_dt, ib + i, planes, plane_stride);
            if (!row_idx) x[ib + i] = v;
        }
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)E + eps);
    for (int i = threadIdx.x; i < E; i += blockDim.x) {
        float v = x[ib + i];
        if (delta && row_idx) v += ld_planes(delta, delta_dt, ib + i, planes, plane_stride);
        st_f(out, out_dt, ob + i, (v * scale) * ld_f(w, w_dt, i));
    }
}

// The same with every element of the row held in registers: each thread owns NV
// groups of 4 consecutive floats, all loads are issued before the first use, and x is
// read once.  Needs E % 4 == 0 and E <= 1024 * NV.
__device__ __forceinline__ float4 ld4_f(const void* p, int dt, size_t i4) {
    if (dt == ILLM_BF16) {
        const uint2 u = ((const uint2*)p)[i4];
        return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                           __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
    }
    return ((const float4*)p)[i4];
}

__device__ __forceinline__ void st4_f(void* p, int dt, size_t i4, float4 v) {
    if (dt == ILLM_BF16) {
        uint2 u;
        u.x = pack_bf16x2(v.x, v.y);
        u.y = pack_bf16x2(v.z, v.w);
        ((uint2*)p)[i4] = u;
    } else {
        ((float4*)p)[i4] = v;
    }
}

template <int NV, int TH>
__global__ void __launch_bounds__(TH)
add_rmsnorm_vec_kernel(float* __restrict__ x, const void* __restrict__ delta, int delta_dt,
                       int planes, size_t plane_stride4,
                       const void* __restrict__ w, int w_dt, void* __restrict__ out, int out_dt,
                       const int32_t* __restrict__ row_idx, int E, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const int in_row = row_idx ? row_idx[r] : r;
    const int E4 = E >> 2;
    const size_t ib = (size_t)in_row * E4, ob = (size_t)r * E4;
    float4 v[NV], wv[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = threadIdx.x + TH * j;
        v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        wv[j] = v[j];
        if (i < E4) {
            v[j] = ((const float4*)x)[ib + i];
            wv[j] = ld4_f(w, w_dt, i);
        }
    }
    if (delta) {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = threadIdx.x + TH * j;
            if (i < E4) {
                float4 d = ld4_f(delta, delta_dt, ib + i);
                // the planes of a split product, four loads at a time, added in order
                for (int s0 = 1; s0 < planes; s0 += 4) {
                    float4 e[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        e[t] = s0 + t < planes
                                   ? ld4_f(delta, delta_dt, ib + i + (size_t)(s0 + t) * plane_stride4)
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        d.x += e[t].x; d.y += e[t].y; d.z += e[t].z; d.w += e[t].w;
                    }
                }
                v[j].x += d.x; v[j].y += d.y; v[j].z += d.z; v[j].w += d.w;
                if (!row_idx) ((float4*)x)[ib + i] = v[j];
            }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j)
        ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)E + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = threadIdx.x + TH * j;
        if (i < E4)
            st4_f(out, out_dt, ob + i,
                  make_float4((v[j].x * scale) * wv[j].x, (v[j].y * scale) * wv[j].y,
                              (v[j].z * scale) * wv[j].z, (v[j].w * scale) * wv[j].w));
    }
}

extern "C" int illm_add_rmsnorm(float* x, const void* delta, int delta_dt, int planes,
                                size_t plane_stride, const void* w, int w_dt, void* out,
                                int out_dt, const int32_t* row_idx, int rows, int E, float eps,
                                void* stream) {
    if (rows < 0 || E <= 0 || !illm_dtype_ok(w_dt) || !illm_dtype_ok(out_dt) ||
        (delta && (!illm_dtype_ok(delta_dt) || planes < 1 ||
                   (planes > 1 && E % 4 == 0 && plane_stride % 4))))
        return ILLM_ERR_ARG;
    if (rows == 0) return ILLM_OK;
    hipStream_t st = (hipStream_t)stream;
#define VEC(NV_, TH_)                                                                         \
    hipLaunchKernelGGL((add_rmsnorm_vec_kernel<NV_, TH_>), dim3(rows), dim3(TH_), 0, st, x,   \
                       delta, delta_dt, planes, plane_stride / 4, w, w_dt, out, out_dt, row_idx, \
                       E, eps)
    // few rows (decoding): wide blocks, one group of 4 floats per thread, to shorten the row's
    // critical path; many rows: narrow blocks so that more rows are in flight per CU
    if (E % 4 == 0 && rows <= 128 && E > 1024 && E <= 4096) VEC(1, 1024);
    else if (E % 4 == 0 && rows <= 128 && E > 4096 && E <= 8192) VEC(2, 1024);
    else if (E % 4 == 0 && E <= 1024) VEC(1, 256);
    else if (E % 4 == 0 && E <= 2048) VEC(2, 256);
    else if (E % 4 == 0 && E <= 4096) VEC(4, 256);
    else if (E % 4 == 0 && E <= 8192) VEC(8, 256);
    else
        hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(rows), dim3(256), 0, st, x, delta, delta_dt,
                           planes, plane_stride, w, w_dt, out, out_dt, row_idx, E, eps);
#undef VEC
    return illm_launch_status();
}

// ---------------------------------------------------------------- silu * up
__global__ void silu_mul_kernel(const void* __restrict__ gu, void* __restrict__ out, int dt,
                                int F) {
    const size_t t = blockIdx.y;
    const int f = blockIdx.x * blockDim.x + threadIdx.x;
    if (f >= F) return;
    const float g = ld_f(gu, dt, t * 2 * F + f);
    const float u = ld_f(gu, dt, t * 2 * F + F + f);
    st_f(out, dt, t * F + f, (g / (1.0f + expf(-g))) * u);
}

// bfloat16 rows with F % 8 == 0: 8 values (16 bytes) of gate and of up per thread
__global__ void __launch_bounds__(256)
silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int F) {
    const size_t t = blockIdx.y;
    const int f = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (f >= F) return;
    const uint4 g = *(const uint4*)(gu + t * 2 * F + f);
    const uint4 u = *(const uint4*)(gu + t * 2 * F + F + f);
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t ow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
        const float r0 = (g0 / (1.0f + expf(-g0))) * u0, r1 = (g1 / (1.0f + expf(-g1))) * u1;
        ow[i] = pack_bf16x2(r0, r1);
    }
    *(uint4*)(out + t * F + f) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

extern "C" int illm_silu_mul(const void* gate_up, void* out, int dt, int T, int F, void* stream) {
    if (T < 0 || F <= 0 || !illm_dtype_ok(dt)) return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    if (dt == ILLM_BF16 && F % 8 == 0) {
        for (int t0 = 0; t0 < T; t0 += 65535) {
            const int rows = T - t0 < 65535 ? T - t0 : 65535;
            hipLaunchKernelGGL(silu_mul_bf16x8_kernel, dim3((F / 8 + 255) / 256, rows), dim3(256), 0,
                               (hipStream_t)stream, (const bf16_t*)gate_up + (size_t)t0 * 2 * F,
                               (bf16_t*)out + (size_t)t0 * F, F);
        }
        return illm_launch_status();
    }
    // gridDim.y is limited to 65535: rows beyond that go in further launches
    for (int t0 = 0; t0 < T; t0 += 65535) {
        const int rows = T - t0 < 65535 ? T - t0 : 65535;
        const size_t esz = dt == ILLM_BF16 ? 2 : 4;
        hipLaunchKernelGGL(silu_mul_kernel, dim3((F + 255) / 256, rows), dim3(256), 0,
                           (hipStream_t)stream,
                           (const void*)((const char*)gate_up + (size_t)t0 * 2 * F * esz),
                           (void*)((char*)out + (size_t)t0 * F * esz), dt, F);
    }
    return illm_launch_status();
}

// ---------------------------------------------------------------- rotation + cache store
// grid (T, nh + nkv): block (t, h) handles head h of row t; heads >= nh are k heads,
// whose block also stores the matching v head.  The angles come from a float32
// table that the host fills from double precision.
__global__ void rope_store_kernel(void* __restrict__ qkv, int dt,
                                  const float* __restrict__ cos_sin, int rot, int pairing,
                                  const int32_t* __restrict__ row_pos,
                                  const int32_t* __restrict__ row_slot,
                                  const int32_t* __restrict__ slot_len, void* __restrict__ kcache,
                                  void* __restrict__ vcache,
                                  const int32_t* __restrict__ page_table, int table_stride,
                                  int page_size, int ring, int nh, int nkv, int hd) {
    const int t = blockIdx.x, h = blockIdx.y;
    const int pos = row_pos[t];
    const size_t row = (size_t)t * (size_t)(nh + 2 * nkv) * hd;
    const size_t base = row + (size_t)h * hd;  // q heads, then k heads follow directly
    const int half = rot / 2;
    if (cos_sin) {
        const float* cs = cos_sin + (size_t)pos * rot;  // [rot/2][2]
        for (int i = threadIdx.x; i < half; i += blockDim.x) {
            const int a = pairing == 0 ? i : 2 * i;
            const int b = pairing == 0 ? i + hd / 2 : 2 * i + 1;  // partner at hd/2 (naive.cpp:393)
            const float c = cs[2 * i], s = cs[2 * i + 1];
            const float x0 = ld_f(qkv, dt, base + a), x1 = ld_f(qkv, dt, base + b);
            st_f(qkv, dt, base + a, x0 * c - x1 * s);
            st_f(qkv, dt, base + b, x0 * s + x1 * c);
        }
    }
    if (h < nh || kcache == nullptr) return;
    const int kvh = h - nh;
    const int slot = row_slot[t];
    if (ring > 0 && slot_len) {
        // a later row of this step lands on the same ring page: this one is already outside
        const int last_page = (slot_len[slot] - 1) / page_size;
        if (pos / page_size + ring <= last_page) return;
    }
    __syncthreads();  // the rotated k of this block is read back below
    const size_t dst = cache_row_offset(page_table, table_stride, slot, pos, page_size, ring, nkv,
                                        kvh, hd);
    const size_t vsrc = row + (size_t)(nh + nkv + kvh) * hd;
    const size_t esz = dt == ILLM_BF16 ? 2 : 4;
    if (esz == 2) {
        const bf16_t* ks = (const bf16_t*)qkv + base;
        const bf16_t* vs = (const bf16_t*)qkv + vsrc;
        bf16_t* kd = (bf16_t*)kcache + dst;
        bf16_t* vd = (bf16_t*)vcache + dst;
        for (int i = threadIdx.x; i < hd; i += blockDim.x) { kd[i] = ks[i]; vd[i] = vs[i]; }
    } else {
        const float* ks = (const float*)qkv + base;
        const float* vs = (const float*)qkv + vsrc;
        float* kd = (float*)kcache + dst;
        float* vd = (float*)vcache + dst;
        for (int i = threadIdx.x; i < hd; i += blockDim.x) { kd[i] = ks[i]; vd[i] = vs[i]; }
    }
}

// bfloat16, pairs (i, i + hd/2), all of the head rotated (rot == hd), hd % 16 == 0: one block
// per row; a thread rotates 8 pairs at a time with 16-byte loads, then the row's k and v
// heads are copied to the cache 16 bytes at a time.
__global__ void __launch_bounds__(256)
rope_store_bf16_kernel(bf16_t* __restrict__ qkv, const float* __restrict__ cos_sin,
                       const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_slot,
                       const int32_t* __restrict__ slot_len, bf16_t* __restrict__ kcache,
                       bf16_t* __restrict__ vcache, const int32_t* __restrict__ page_table,
                       int table_stride, int page_size, int ring, int nh, int nkv, int hd) {
    const int t = blockIdx.x;
    const int pos = row_pos[t];
    bf16_t* row = qkv + (size_t)t * (size_t)(nh + 2 * nkv) * hd;
    const int half = hd / 2, cpu8 = half / 8;             // chunks of 8 pairs per head
    if (cos_sin) {
        const float* cs = cos_sin + (size_t)pos * hd;     // [hd/2][2]
        for (int u = threadIdx.x; u < (nh + nkv) * cpu8; u += 256) {
            const int h = u / cpu8, i0 = (u - h * cpu8) * 8;
            bf16_t* p = row + (size_t)h * hd + i0;
            const uint4 a = *(const uint4*)p, b = *(const uint4*)(p + half);
            const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
            uint32_t ao[4], bo[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4 c = *(const float4*)(cs + 2 * (i0 + 2 * j));   // cos, sin, cos, sin
                const float x0 = __uint_as_float(aw[j] << 16), x1 = __uint_as_float(aw[j] & 0xffff0000u);
                const float y0 = __uint_as_float(bw[j] << 16), y1 = __uint_as_float(bw[j] & 0xffff0000u);
                ao[j] = pack_bf16x2(x0 * c.x - y0 * c.y, x1 * c.z - y1 * c.w);
                bo[j] = pack_bf16x2(x0 * c.y + y0 * c.x, x1 * c.w + y1 * c.z);
            }
            *(uint4*)p = make_uint4(ao[0], ao[1], ao[2], ao[3]);
            *(uint4*)(p + half) = make_uint4(bo[0], bo[1], bo[2], bo[3]);
        }
    }
    if (kcache == nullptr) return;
    const int slot = row_slot[t];
    if (ring > 0 && slot_len) {
        const int last_page = (slot_len[slot] - 1) / page_size;
        if (pos / page_size + ring <= last_page) return;
    }
    __syncthreads();
    const int c8 = hd / 8;
    for (int u = threadIdx.x; u < 2 * nkv * c8; u += 256) {
        const int which = u / (nkv * c8), r = u - which * nkv * c8;
        const int kvh = r / c8, off = (r - kvh * c8) * 8;
        const size_t dst = cache_row_offset(page_table, table_stride, slot, pos, page_size, ring, nkv,
                                            kvh, hd) + off;
        const bf16_t* src = row + (size_t)(nh + which * nkv + kvh) * hd + off;
        *(uint4*)((which ? vcache : kcache) + dst) = *(const uint4*)src;
    }
}

extern "C" int illm_rope_store(void* qkv, int dt, const float* cos_sin, int max_pos, int rot,
                               int pairing, const int32_t* row_pos, const int32_t* row_slot,
                               const int32_t* slot_len, void* kcache, void* vcache,
                               const int32_t* page_table, int table_stride, int page_size,
                               int ring, int T, int nh, int nkv, int hd, void* stream) {
    if (T < 0 || nh <= 0 || nkv < 0 || hd <= 0 || !illm_dtype_ok(dt)) return ILLM_ERR_ARG;
    if (cos_sin && (rot <= 0 || rot > hd || (rot & 1) || max_pos <= 0)) return ILLM_ERR_ARG;
    if (pairing != 0 && pairing != 1) return ILLM_ERR_ARG;
    if (kcache && (!vcache || !page_table || !row_slot || page_size <= 0 || table_stride <= 0))
        return ILLM_ERR_ARG;
    if (nh + nkv > 65535) return ILLM_ERR_ARG;
    if (T == 0) return ILLM_OK;
    if (dt == ILLM_BF16 && hd % 16 == 0 && (!cos_sin || (pairing == 0 && rot == hd))) {
        hipLaunchKernelGGL(rope_store_bf16_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream,
                           (bf16_t*)qkv, cos_sin, row_pos, row_slot, slot_len, (bf16_t*)kcache,
                           (bf16_t*)vcache, page_table, table_stride, page_size, ring, nh, nkv, hd);
        return illm_launch_status();
    }
    hipLaunchKernelGGL(rope_store_kernel, dim3(T, nh + nkv), dim3(64), 0, (hipStream_t)stream, qkv,
                       dt, cos_sin, rot, pairing, row_pos, row_slot, slot_len, kcache, vcache,
                       page_table, table_stride, page_size, ring, nh, nkv, hd);
    return illm_launch_status();
}

extern "C" int illm_version() { return 1; }

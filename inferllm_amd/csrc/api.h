// C entry points of the kernel library (the switches that tests and tuning runs flip are
// declared apart, in api_test.h: nothing of the product calls them).  Every function launches on `stream`
// and returns ILLM_OK, ILLM_ERR_ARG (sizes or dtypes it does not take; nothing
// was launched), ILLM_ERR_LAUNCH or, where said, ILLM_ERR_SCRATCH.  Pointers are device pointers.  dtype codes:
// 0 = float32, 1 = bfloat16.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int illm_version();

// out[t, :] = table[tokens[t], :] as float32.
int illm_embed(const int32_t* tokens, const void* table, int table_dt, float* out,
               int T, int E, int V, void* stream);

// Residual add and RMS norm.  in_row = row_idx ? row_idx[r] : r;
// v = x[in_row] (+ delta[in_row]); when delta is given and row_idx is not, v is
// written back to x.  out[r] = v * rsqrt(mean(v^2) + eps) * w.  delta may be `planes` >= 1
// arrays, plane_stride elements apart (the sums of a product whose K was split,
// illm_gemm_mid_bf16), which are added in order.
int illm_add_rmsnorm(float* x, const void* delta, int delta_dt, int planes, size_t plane_stride,
                     const void* w, int w_dt, void* out, int out_dt, const int32_t* row_idx,
                     int rows, int E, float eps, void* stream);

// out[t, f] = silu(gate_up[t, f]) * gate_up[t, F + f].
int illm_silu_mul(const void* gate_up, void* out, int dt, int T, int F, void* stream);

// Rotate q and k of packed rows [q (nh*hd) | k (nkv*hd) | v (nkv*hd)] in place by the
// angles of `cos_sin` ([max_pos][rot/2][2] float32; null: no rotation) at row_pos[t],
// pairing 0 = (i, i + hd/2), 1 = (2i, 2i+1), i < rot/2; then store k and v of each row in the
// paged cache of row_slot[t] (skipped when kcache is null).  With a ring of pages, slot_len
// (length of every slot after the step) lets rows that a later row of the same step would
// overwrite be skipped; it may be null when no sequence brings more than one row.
int illm_rope_store(void* qkv, int dt, const float* cos_sin, int max_pos, int rot, int pairing,
                    const int32_t* row_pos, const int32_t* row_slot, const int32_t* slot_len,
                    void* kcache, void* vcache, const int32_t* page_table, int table_stride,
                    int page_size, int ring, int T, int nh, int nkv, int hd, void* stream);

// Y[M, N] = X[M, K] . W[N, K]^T, float32 accumulation in a fixed order; any sizes.
int illm_gemm_generic(const void* X, int x_dt, const void* W, int w_dt, void* Y, int y_dt,
                      int M, int N, int K, void* stream);

// The same product for float32 X and W with K % 16 == 0 on the matrix cores' float32 instruction
// (float32 operands, products and sums), for many rows.
int illm_gemm_f32_mfma(const float* X, const float* W, void* Y, int y_dt, int M, int N, int K,
                       void* stream);

// The same product for M <= 128 rows of float32 X and W with K % 32 == 0, W read once, on the
// matrix cores' float32 instruction with operands straight from memory.
int illm_gemm_rows_f32_mfma(const float* X, const float* W, void* Y, int y_dt, int M, int N, int K,
                            void* stream);

// The same product for M <= 16 rows when X and W are float32 and K % 4 == 0: W is read once
// (decoding on the 32-bit path); plain float32 multiply-adds.
int illm_gemv_rows_f32(const float* X, const float* W, void* Y, int y_dt, int M, int N, int K,
                       void* stream);

// Causal attention over packed rows of whole prompts (keys and values of the step
// itself).  cu_seqlens[n_seqs + 1]; window <= 0: all earlier keys.
int illm_attn_prefill_generic(const void* qkv, void* out, int dt, const int32_t* cu_seqlens,
                              int n_seqs, int max_len, int nh, int nkv, int hd, float scale,
                              int window, void* stream);

// The same on the matrix cores for bfloat16 and head_dim % 16 == 0 (else ILLM_ERR_ARG).
int illm_attn_prefill_bf16(const void* qkv, void* out, const int32_t* cu_seqlens, int n_seqs,
                           int max_len, int nh, int nkv, int hd, float scale, int window,
                           void* stream);

// The two above for steps whose rows go on from tokens the cache already holds (a prompt cut into
// several steps): keys and values are read from the paged cache, which must hold the step's own
// rows too by then; row r of sequence b stands at position seq_start[b] + r and sees the keys
// 0 .. its position of the sequence in seq_slot[b].  The bfloat16 kernel needs pages of a multiple
// of 64 rows.
int illm_attn_prefill_paged_generic(const void* qkv, void* out, int dt, const int32_t* cu_seqlens,
                                    const int32_t* seq_slot, const int32_t* seq_start,
                                    const void* kcache, const void* vcache,
                                    const int32_t* page_table, int table_stride, int page_size,
                                    int ring, int n_seqs, int max_len, int nh, int nkv, int hd,
                                    float scale, int window, void* stream);
int illm_attn_prefill_paged_bf16(const void* qkv, void* out, const int32_t* cu_seqlens,
                                 const int32_t* seq_slot, const int32_t* seq_start,
                                 const void* kcache, const void* vcache, const int32_t* page_table,
                                 int table_stride, int page_size, int ring, int n_seqs, int max_len,
                                 int nh, int nkv, int hd, float scale, int window, void* stream);

// One query row per sequence over the paged cache.  partial: float32
// [B][nh][nsplit][hd + 2] scratch.  seq_len[b] = keys of sequence b, the new one included.
int illm_attn_decode_generic(const void* qkv, void* out, int dt, const void* kcache,
                             const void* vcache, const int32_t* page_table, int table_stride,
                             int page_size, int ring, const int32_t* seq_slot,
                             const int32_t* seq_len, float* partial, int nsplit, int B, int nh,
                             int nkv, int hd, float scale, int window, void* stream);

// The same for bfloat16 with head_dim % 8 == 0 and page_size % 64 == 0 (anything else:
// ILLM_ERR_ARG); nsplit == 1 needs no `partial`.  `waves`: waves per block that share a key
// range and combine through LDS (clamped to what the head group's registers and LDS allow).
int illm_attn_decode_bf16(const void* qkv, void* out, const void* kcache, const void* vcache,
                          const int32_t* page_table, int table_stride, int page_size, int ring,
                          const int32_t* seq_slot, const int32_t* seq_len, float* partial,
                          int nsplit, int waves, int B, int nh, int nkv, int hd, float scale,
                          int window, void* stream);

// illm_attn_decode_bf16 for callers that cannot allocate device memory (code under HIP graph
// capture, tight serving loops, harnesses that forbid it): it has no counterpart in the
// reference.  The split results go through an array that the library holds on every GPU it runs
// on (ILLM_DECODE_SCRATCH_BYTES, until the process ends) instead of a `partial` argument; the call
// allocates and frees nothing.  B * nh * nsplit * (hd + 2) * 4 bytes must fit the array, else
// ILLM_ERR_SCRATCH (3) and nothing is launched; nsplit == 1 uses no scratch.  All calls on one GPU
// share the array, so calls that overlap on one GPU (two streams) race: run them one after the
// other.  Nothing needs clearing between calls: every entry that is read was written by the same
// call before.
#define ILLM_DECODE_SCRATCH_BYTES (4u << 20)
int illm_attn_decode_bf16_static(const void* qkv, void* out, const void* kcache,
                                 const void* vcache, const int32_t* page_table, int table_stride,
                                 int page_size, int ring, const int32_t* seq_slot,
                                 const int32_t* seq_len, int nsplit, int waves, int B, int nh,
                                 int nkv, int hd, float scale, int window, void* stream);

// Y[M, N] = X[M, K] . W[N, K]^T for bfloat16 X and W, 1 <= M <= 64, K % 8 == 0, on the
// matrix cores with float32 accumulation; Y float32 or bfloat16.
// ssq != null (M <= 16 only): X is bfloat16(x * norm weight) of residual rows x whose sums of
// squares lie in ssq[M][parts] (left by illm_gemm_skinny_add), and row m of the result is scaled
// by 1 / sqrt(sum_p ssq[m][p] / K + eps): the product of the RMS norm of x.
// Wt (here and below, may be null): a copy of W laid out for these kernels,
// [tile][K / 32][16 rows][32 k] with tile t holding the 16 rows that block t works on (plain
// product: rows 16 t ..; gate|up: 8 gate rows 8 t .. and the same 8 up rows; q|k|v: 8 rows of a
// head and their 8 rotation partners, then 16 rows per tile for v), rows beyond the matrix zero.
// Used when M <= 16 and K % 32 == 0; W itself is then not read.
int illm_gemm_skinny_bf16(const void* X, const void* W, const void* Wt, void* Y, int y_dt, int M,
                          int N, int K, const float* ssq, int parts, float eps, int waves_wanted,
                          void* stream);

// Y[M, N] (float32 residual rows) += X . W^T for M <= 16 bfloat16 rows.  nw != null (the weight of
// the RMS norm that follows, bfloat16 or float32 [N]): also xb[M, N] = bfloat16(Y * nw) and
// ssq_out[M][ceil(N / 16)], partial sums of Y^2, for a product that takes `ssq`.
int illm_gemm_skinny_add(const void* X, const void* W, const void* Wt, float* Y, int M, int N,
                         int K, const void* nw, int nw_dt, void* xb, float* ssq_out,
                         int waves_wanted, void* stream);

// Y = X[M, K] . W[N, K]^T for M up to 128 from the tiled copy Wt of W, K a
// multiple of 32, X shared by a block's waves through LDS.  splits == 1: Y is [M, N] of y_dt;
// splits > 1: K is cut into that many ranges and Y is float32 [splits][M][N], the planes to be
// added by the caller (illm_add_rmsnorm takes them).  illm_gemm_mid_splits: the splits to use.
int illm_gemm_mid_bf16(const void* X, const void* Wt, void* Y, int y_dt, int M, int N, int K,
                       int splits, void* stream);
int illm_gemm_mid_splits(int N, int K);

// Products of 1 to 128 bfloat16 rows (meant for 9 and more) from the tiled copy
// Wt of W, K a multiple of 64, X shared by a block's waves through LDS, K cut inside the block
// (csrc/gemm_rows.hip).  illm_gemm_rows_bf16: Y[M, N] = X . W^T (plain tiles), float32 or bfloat16.
// illm_gemm_rows_gateup_silu: Y[M, F] = silu(X . Wg^T) * (X . Wu^T) from the gate|up tiles.
// illm_qkv_rope_store_rows: as illm_qkv_rope_store_skinny, from the q|k|v tiles.  ssq (M <= 16
// only): as for illm_gemm_skinny_bf16.
int illm_gemm_rows_bf16(const void* X, const void* Wt, void* Y, int y_dt, int M, int N, int K,
                        const float* ssq, int parts, float eps, void* stream);
int illm_gemm_rows_gateup_silu(const void* X, const void* Wt, void* Y, int y_dt, int M, int F,
                               int K, const float* ssq, int parts, float eps, void* stream);
int illm_qkv_rope_store_rows(const void* X, const void* Wt, void* Y, int M, int K,
                             const float* cos_sin, int max_pos, const int32_t* row_pos,
                             const int32_t* row_slot, void* kcache, void* vcache,
                             const int32_t* page_table, int table_stride, int page_size, int ring,
                             int nh, int nkv, int hd, const float* ssq, int parts, float eps,
                             void* stream);

// Y[M, F] = silu(X . Wg^T) * (X . Wu^T), W = [Wg | Wu] as [2F, K]; same limits as the skinny
// product, `ssq` included.  waves_wanted: waves per block (0: the default choice).
int illm_gemm_skinny_gateup_silu(const void* X, const void* W, const void* Wt, void* Y, int y_dt,
                                 int M, int F, int K, const float* ssq, int parts, float eps,
                                 int waves_wanted, void* stream);

// Few bfloat16 rows (M <= 16, hd % 16 == 0): the q|k|v product, the rotation of q and k (pairs
// (i, i + hd/2), all dims) at row_pos[m], q into Y[M, (nh + 2 nkv) hd] (k and v parts untouched),
// k and v into the paged cache of row_slot[m], all in one kernel.  ssq: as for
// illm_gemm_skinny_bf16.  waves_wanted: waves per block (0: the default choice).
int illm_qkv_rope_store_skinny(const void* X, const void* W, const void* Wt, void* Y, int M, int K,
                               const float* cos_sin, int max_pos, const int32_t* row_pos,
                               const int32_t* row_slot, void* kcache, void* vcache,
                               const int32_t* page_table, int table_stride, int page_size, int ring,
                               int nh, int nkv, int hd, const float* ssq, int parts, float eps,
                               int waves_wanted, void* stream);

// out[b] = index of the largest logit of row b (lowest index on ties).  A row is cut into
// `parts` (1 to 64) that blocks of their own take; scratch: 2 x B x parts 32-bit words (may be
// null when parts == 1).
int illm_argmax(const float* logits, int32_t* out, void* scratch, int B, int V, int parts,
                void* stream);

// Temperature / top-k / top-p / repeat-penalty sampling, one draw per row.
// scratch: float32 [2][B][V].  last_tokens: [B][n_last] (-1 = empty) or null.
// counters[b]: index of the draw in the request's stream; seeds[b]: the request's seed.
int illm_sample(const float* logits, float* scratch, int32_t* out, int B, int V, float temp,
                int top_k, float top_p, float repeat_penalty, const int32_t* last_tokens,
                int n_last, const uint64_t* seeds, const int32_t* counters, void* stream);

// The same without top_k for rows of 16,384 ids and more, several blocks a row and a kernel a
// pass (illm_sample walks such a row with one block).  rows: B x ILLM_SAMPLE_LONG_ROW_BYTES bytes
// of device memory, 8-byte aligned, that the passes hand their results on through; nothing in it
// needs clearing.  Shorter rows: ILLM_ERR_ARG.
#define ILLM_SAMPLE_LONG_ROW_BYTES 73728
int illm_sample_long_row_bytes(void);          // ILLM_SAMPLE_LONG_ROW_BYTES, for callers that cannot read this file
int illm_sample_long(const float* logits, float* scratch, void* rows, int32_t* out, int B, int V,
                     float temp, float top_p, float repeat_penalty, const int32_t* last_tokens,
                     int n_last, const uint64_t* seeds, const int32_t* counters, void* stream);

#ifdef __cplusplus
}
#endif

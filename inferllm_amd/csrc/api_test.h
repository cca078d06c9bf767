// Switches for tests and tuning runs: each forces one of several equivalent kernels or block
// shapes that the library otherwise chooses by itself, so that a test can compare them and a
// tuning run can time them.  They are process-wide and not part of the product's interface:
// nothing under inferllm_amd/ calls them, and a program that serves requests must not.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

// illm_gemm_rows_f32_mfma: tiles of 16 rows of W a block takes (1 or 2; 0: the library's choice).
// The sums are the same bits either way.
void illm_set_rows_f32_tiles(int tiles);

// Whether float32 prompts with head sizes 32, 64, 96 and 128 take the attention kernel on the
// matrix cores' float32 instruction (1, default) or the multiply-add kernel of every other size (0).
void illm_set_attn_f32_mfma(int on);

// Which bfloat16 prefill attention kernel head sizes up to 128 take: 0 the one with one LDS buffer
// (which larger head sizes use), 2 the one with two buffers and one barrier a tile (needs a
// positive scale), 1 (default) the second for head sizes 64 to 128 and sequences of 1,024 keys or
// more.
void illm_set_prefill_two_buffers(int on);

// illm_gemm_mid_bf16: tiles of W a wave takes, 1 or 2 (0, default: by the number of tiles).
void illm_set_mid_tiles_per_wave(int n);
// illm_gemm_mid_bf16: rows of X a launch takes, 64 or 128 (default); W is read once a launch.
void illm_set_mid_rows_a_launch(int rows);

// illm_gemm_skinny_add: 0 switches off the variant in which, for K up to 4096 and at most 512
// tiles, 8 waves each take their whole share of K at once (default 1).
void illm_set_skinny_one_shot(int on);

// illm_attn_decode_bf16: 0 sends grouped heads of head sizes up to 128 to the kernel with P.V on
// the vector units, which larger head sizes use, instead of the one with both products on the
// matrix cores (default 1).
void illm_set_gqa_pv_on_matrix_cores(int on);

// csrc/gemm_rows.hip: tiles a block of its products takes (2 to 8) and parts of K (1, 2, 4; four
// tiles and more: 1, 2); 0: the library's own choice.
void illm_set_rows_shape(int tb, int kp);
// csrc/gemm_rows.hip: rows of X a launch of its products takes, 64 or 128 (default).
void illm_set_rows_a_launch(int rows);

#ifdef __cplusplus
}
#endif

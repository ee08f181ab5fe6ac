/*
 * TEST INFRASTRUCTURE ONLY -- the parity checker for the HIP path and the CPU-baseline leg of
 * bench.py.  Nothing in the product (powerinfer_amd/) may include, link or call this.
 *
 * Plain-C restatement of the CPU arithmetic of PowerInfer's sparse decode token loop
 * (reference: ggml.c, ggml-quants.c, llama.cpp; every function in pi_oracle.c cites the lines
 * it follows).  Shapes use ggml's convention: ne0 is the contiguous dimension.
 */
#ifndef PI_ORACLE_H
#define PI_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PIO_API __attribute__((visibility("default")))

/* tensor element types: numeric values of enum ggml_type (ggml.h:333-355) */
enum { PIO_F32 = 0, PIO_F16 = 1, PIO_Q4_0 = 2, PIO_I32 = 18 };

/* ---- scalar / row codecs --------------------------------------------------------------- */
PIO_API uint16_t pio_f32_to_f16(float x);
PIO_API float    pio_f16_to_f32(uint16_t h);
PIO_API void     pio_f32_to_f16_row(const float * x, uint16_t * y, int64_t n);
PIO_API void     pio_f16_to_f32_row(const uint16_t * x, float * y, int64_t n);
PIO_API void     pio_quantize_row_q4_0(const float * x, void * y, int64_t n);   /* 18 B per 32 */
PIO_API void     pio_dequantize_row_q4_0(const void * x, float * y, int64_t n);
PIO_API void     pio_quantize_row_q8_0(const float * x, void * y, int64_t n);   /* 34 B per 32 */
PIO_API size_t   pio_row_bytes(int type, int64_t n);

/* ---- dot products ---------------------------------------------------------------------- */
PIO_API float pio_vec_dot_f16(int64_t n, const uint16_t * x, const uint16_t * y);
PIO_API float pio_vec_dot_q4_0_q8_0(int64_t n, const void * x, const void * y);

/* ---- ops ------------------------------------------------------------------------------- */
/* out[rows, T] = W[cols, rows] . x[cols, T]; activations are first rounded to the weight
 * type's dot type (F16 -> fp16, Q4_0 -> Q8_0 blocks) as the reference executor does. */
PIO_API int pio_mul_mat(int wtype, const void * w, int64_t rows, int64_t cols,
                        const float * x, int T, float * out, int n_threads);

/* GGML_OP_MUL_MAT_SPARSE on the CPU: row skipped (0 written) iff gpu_idx[row] == 1 or
 * idx[t][row] < threshold. */
PIO_API int pio_mul_mat_sparse(int wtype, const void * w, int64_t rows, int64_t cols,
                               const float * x, int T, const float * idx, const int32_t * gpu_idx,
                               float threshold, float * out, int n_threads);

/* GGML_OP_AXPY on the CPU: out[cols, T] = sum over rows of h[t][row] * Wt[row, :]; rows skipped
 * iff h == 0 (after rounding to the dot type), gpu_idx[row] == 1, or idx[t][row] < threshold. */
PIO_API int pio_axpy(int wtype, const void * wt, int64_t rows, int64_t cols,
                     const float * h, int T, const float * idx, const int32_t * gpu_idx,
                     float threshold, float * out, int n_threads);

PIO_API void pio_rms_norm(const float * x, int64_t n, int T, float eps, float * out);
PIO_API void pio_norm(const float * x, int64_t n, int T, float eps, float * out);
/* x [n_embd_head, n_head, T]; mode 0 = adjacent pairs (LLaMA), 2 = NeoX halves (Falcon) */
PIO_API void pio_rope(const float * x, int n_embd_head, int n_head, int T, const int32_t * pos,
                      int n_dims, int mode, float freq_base, float freq_scale, float * out);
/* the same with linear and YaRN scaling (ggml_rope_custom's operands; ext_factor 0 and attn_factor 1 give pio_rope) */
PIO_API void pio_rope_ext(const float * x, int n_embd_head, int n_head, int T, const int32_t * pos, int n_dims, int mode, int n_orig_ctx,
                          float freq_base, float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow, float * out);
PIO_API void pio_soft_max(const float * x, int64_t n, int64_t rows, float * out);

/* ascending indices of idx[i] >= threshold; returns the count */
PIO_API int pio_active_list(const float * idx, int64_t n, float threshold, int32_t * list);

/* the whole sparse FFN block for T tokens (llm_build_ffn_sparse on a CPU-only build) */
PIO_API int pio_ffn_sparse(int d, int ff, int r, int T, int wtype, int has_gate,
                           const void * up_w, const void * gate_w, const void * down_t,
                           const uint16_t * fc1, const uint16_t * fc2,
                           const float * x_ffn, const float * x_pred, const int32_t * gpu_idx,
                           float threshold, int n_threads,
                           float * logits, float * up_out, float * gate_out, float * h_out, float * out);

/* attention core for T new tokens; see pi_oracle.c */
PIO_API int pio_attention(int n_embd_head, int n_head, int n_head_kv, int n_ctx, int n_kv, int T,
                          const int32_t * kv_slot, const float * kq_mask,
                          const float * q, const float * k_cur, const float * v_cur,
                          uint16_t * k_cache, uint16_t * v_cache, float * out);

/* ---- whole model ----------------------------------------------------------------------- */
enum { PIO_ARCH_LLAMA = 0, PIO_ARCH_FALCON = 1 };

typedef struct pio_hparams {
    int32_t arch;
    int32_t n_embd, n_ff, n_head, n_head_kv, n_layer, n_vocab, n_ctx;
    float   norm_eps, rope_freq_base, sparse_threshold;
    float   rope_freq_scale;            /* linear RoPE scaling (llama_cparams.rope_freq_scale, llama.cpp:9857); 0 is read as 1 */
} pio_hparams;

/* tensor kinds; layer = -1 for the three global tensors */
enum {
    PIO_T_TOK_EMBD = 0, PIO_T_OUTPUT_NORM, PIO_T_OUTPUT_NORM_B, PIO_T_OUTPUT,
    PIO_T_ATTN_NORM, PIO_T_ATTN_NORM_B, PIO_T_ATTN_NORM_2, PIO_T_ATTN_NORM_2_B,
    PIO_T_WQ, PIO_T_WK, PIO_T_WV, PIO_T_WQKV, PIO_T_WO,
    PIO_T_FFN_NORM, PIO_T_FFN_GATE, PIO_T_FFN_UP, PIO_T_FFN_DOWN_T,
    PIO_T_FC1, PIO_T_FC2, PIO_T_GPU_IDX,
    PIO_T_COUNT
};

typedef struct pio_model pio_model;

PIO_API pio_model * pio_model_new(const pio_hparams * hp);
PIO_API void        pio_model_free(pio_model * m);
/* borrows `data` (no copy); ne1 is the number of rows (needed for FC1/FC2 whose rank is free) */
PIO_API int         pio_model_set_tensor(pio_model * m, int layer, int kind, int type, const void * data, int64_t ne0, int64_t ne1);
PIO_API void        pio_model_kv_clear(pio_model * m);

/* optional per-layer captures, each may be NULL: ffn_out [n_layer][T][n_embd], pred_logits [n_layer][T][n_ff],
 * ffn_src [n_layer][T][n_embd] (the vector the FFN block reads, before its norm: LLaMA ffn_inp, Falcon the layer
 * input); they are filled by the next pio_model_eval call */
PIO_API void        pio_model_set_capture(pio_model * m, float * ffn_out, float * pred_logits, float * ffn_src);

/*
 * One llama_decode of T tokens: tokens[T], pos[T], kv_slot[T] (cache cell each token is written to),
 * n_kv cells attended, kq_mask [T][n_kv] (0 or -inf).  logits_out [T][n_vocab] if all_logits else
 * [n_vocab] of the last token.  Returns 0 on success.
 */
/* llm_build_k_shift: rotates every cached K row by delta[cell] positions (delta[n_ctx]; 0 leaves the cell's bits unchanged) */
PIO_API int         pio_model_k_shift(pio_model * m, const int32_t * delta);
PIO_API int         pio_model_eval(pio_model * m, const int32_t * tokens, const int32_t * pos, const int32_t * kv_slot,
                                   int T, int n_kv, const float * kq_mask, int all_logits, float * logits_out, int n_threads);

/* convenience: single sequence, causal mask, slot = position; returns greedy argmax of the last token */
PIO_API int         pio_model_eval_simple(pio_model * m, const int32_t * tokens, int T, int n_past, float * logits_out, int n_threads);

#ifdef __cplusplus
}
#endif
#endif

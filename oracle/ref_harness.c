/*
 * TEST INFRASTRUCTURE ONLY -- never linked into, imported by, or called from the product.
 *
 * Thin driver around the reference's own CPU implementation.  It is compiled together with the
 * reference sources where they lie (ggml.c, ggml-quants.c, ggml-alloc.c, ggml-backend.c) into
 * oracle/_ref/libpi_ref.so by oracle/Makefile, only in a container that has the reference tree.
 * It builds the same op sequence that llm_build_ffn_sparse emits on a CPU-only build
 * (llama.cpp:4652-4757 with llm_build_sparse_mul_mat :4546 and llm_build_sparse_axpy :4599)
 * and runs it through the reference executor (ggml_graph_compute, ggml.c:17380), plus a few
 * single-op probes (dense mul_mat, norms, RoPE, softmax, Q4_0/Q8_0 codecs).
 *
 * Everything here is the reference's arithmetic; nothing is restated.  The fixtures under
 * tests/golden/ were produced by calling these functions with n_threads = 1 (the reference's
 * CPU AXPY merges per-thread partial sums without a lock, ggml.c:14433-14458).
 */
#include "ggml.h"

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#define REF_API __attribute__((visibility("default")))

static size_t tensor_bytes(enum ggml_type t, int64_t ne0, int64_t ne1) {
    return (size_t)(ne0 / ggml_blck_size(t)) * ggml_type_size(t) * (size_t)ne1;
}

static struct ggml_context * new_ctx(size_t payload) {
    struct ggml_init_params ip = { payload + (64u << 20), NULL, false };
    return ggml_init(ip);
}

static struct ggml_tensor * put2d(struct ggml_context * ctx, enum ggml_type t, int64_t ne0, int64_t ne1, const void * src) {
    struct ggml_tensor * x = ggml_new_tensor_2d(ctx, t, ne0, ne1);
    if (src) memcpy(x->data, src, ggml_nbytes(x));
    return x;
}

REF_API void ref_set_threshold(float thr) { sparse_pred_threshold = thr; }

/* ref_set_repeat(n > 1): the next ref_ffn_sparse calls run their graph n more times and keep the mean time of one run */
static int g_repeat = 1;
static double g_last_ms = 0.0;
REF_API void ref_set_repeat(int n) { g_repeat = n; }
REF_API double ref_last_compute_ms(void) { return g_last_ms; }

/*
 * One sparse FFN block exactly as a CPU-only build of llama.cpp assembles it:
 *   idx  = mul_mat(fc2, relu(mul_mat(fc1, x_pred)))
 *   up   = mul_mat_idx(up_w,   x_ffn, idx, gpu_idx)
 *   gate = mul_mat_idx(gate_w, x_ffn, idx, gpu_idx)        (omitted when has_gate == 0)
 *   h    = relu(gate) * up            |  relu(up)
 *   out  = axpy(down_t, h, idx, gpu_idx)
 * wtype: 1 = F16, 2 = Q4_0 (applies to up/gate/down_t; fc1/fc2 are always F16).
 * gpu_idx: int32[ff], 1 = "lives on the GPU, skip on the CPU".  All zero = everything computed.
 * Any output pointer may be NULL.  Returns 0 on success.
 */
REF_API int ref_ffn_sparse(int d, int ff, int r, int T, int wtype, int has_gate,
                           const void * up_w, const void * gate_w, const void * down_t,
                           const uint16_t * fc1, const uint16_t * fc2,
                           const float * x_ffn, const float * x_pred, const int32_t * gpu_idx,
                           float threshold, int n_threads,
                           float * logits, float * up_out, float * gate_out, float * h_out, float * out) {
    enum ggml_type wt = (enum ggml_type) wtype;
    size_t payload = 3 * tensor_bytes(wt, d, ff) + 2u * ((size_t)d * r + (size_t)r * ff)
                   + (size_t)T * (2u * d + 8u * ff + 2u * r) * sizeof(float) + (size_t)ff * 4
                   + (size_t)n_threads * d * 64 + (8u << 20);
    struct ggml_context * ctx = new_ctx(payload);
    if (!ctx) return 1;
    sparse_pred_threshold = threshold;

    struct ggml_tensor * t_up   = put2d(ctx, wt, d, ff, up_w);
    struct ggml_tensor * t_gate = has_gate ? put2d(ctx, wt, d, ff, gate_w) : NULL;
    struct ggml_tensor * t_down = put2d(ctx, wt, d, ff, down_t);
    struct ggml_tensor * t_fc1  = put2d(ctx, GGML_TYPE_F16, d, r, fc1);
    struct ggml_tensor * t_fc2  = put2d(ctx, GGML_TYPE_F16, r, ff, fc2);
    struct ggml_tensor * t_x    = put2d(ctx, GGML_TYPE_F32, d, T, x_ffn);
    struct ggml_tensor * t_xp   = put2d(ctx, GGML_TYPE_F32, d, T, x_pred);
    struct ggml_tensor * t_gid  = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, ff);
    memcpy(t_gid->data, gpu_idx, (size_t)ff * 4);

    struct ggml_tensor * idx = ggml_mul_mat(ctx, t_fc1, t_xp);
    idx = ggml_relu(ctx, idx);
    idx = ggml_mul_mat(ctx, t_fc2, idx);

    struct ggml_tensor * upo = ggml_mul_mat_idx(ctx, t_up, t_x, idx, t_gid);
    struct ggml_tensor * gto = NULL;
    struct ggml_tensor * cur;
    if (has_gate) {
        gto = ggml_mul_mat_idx(ctx, t_gate, t_x, idx, t_gid);
        cur = ggml_mul(ctx, ggml_relu(ctx, gto), upo);
    } else {
        cur = ggml_relu(ctx, upo);
    }
    struct ggml_tensor * res = ggml_axpy(ctx, t_down, cur, idx, t_gid);

    struct ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, res);
    if (g_repeat <= 1) {
        ggml_graph_compute_with_ctx(ctx, gf, n_threads);
    } else {                                         /* timing: the graph alone, set-up and copies excluded */
        struct ggml_cplan plan = ggml_graph_plan(gf, n_threads);
        plan.work_data = plan.work_size ? malloc(plan.work_size) : NULL;
        ggml_graph_compute(gf, &plan);
        struct timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        for (int i = 0; i < g_repeat; ++i) ggml_graph_compute(gf, &plan);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        g_last_ms = ((t1.tv_sec - t0.tv_sec) * 1e3 + (t1.tv_nsec - t0.tv_nsec) * 1e-6) / g_repeat;
        free(plan.work_data);
    }

    if (logits)          memcpy(logits,   idx->data, (size_t)ff * T * 4);
    if (up_out)          memcpy(up_out,   upo->data, (size_t)ff * T * 4);
    if (gate_out && gto) memcpy(gate_out, gto->data, (size_t)ff * T * 4);
    if (h_out)           memcpy(h_out,    cur->data, (size_t)ff * T * 4);
    if (out)             memcpy(out,      res->data, (size_t)d * T * 4);
    ggml_free(ctx);
    return 0;
}

/* dense ggml_mul_mat: W [cols, rows] of wtype (F32=0, F16=1, Q4_0=2), x F32 [cols, T] -> out F32 [rows, T] */
REF_API int ref_mul_mat(int wtype, const void * w, int rows, int cols, const float * x, int T, int n_threads, float * out) {
    enum ggml_type wt = (enum ggml_type) wtype;
    struct ggml_context * ctx = new_ctx(tensor_bytes(wt, cols, rows) + (size_t)T * (cols + rows) * 8 + (4u << 20));
    if (!ctx) return 1;
    struct ggml_tensor * tw = put2d(ctx, wt, cols, rows, w);
    struct ggml_tensor * tx = put2d(ctx, GGML_TYPE_F32, cols, T, x);
    struct ggml_tensor * r  = ggml_mul_mat(ctx, tw, tx);
    struct ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, r);
    ggml_graph_compute_with_ctx(ctx, gf, n_threads);
    memcpy(out, r->data, (size_t)rows * T * 4);
    ggml_free(ctx);
    return 0;
}

/* kind 0 = rms_norm, 1 = norm (LayerNorm without affine); x [n, T] */
REF_API int ref_norm(int kind, const float * x, int n, int T, float eps, float * out) {
    struct ggml_context * ctx = new_ctx((size_t)n * T * 16 + (1u << 20));
    if (!ctx) return 1;
    struct ggml_tensor * tx = put2d(ctx, GGML_TYPE_F32, n, T, x);
    struct ggml_tensor * r  = kind == 0 ? ggml_rms_norm(ctx, tx, eps) : ggml_norm(ctx, tx, eps);
    struct ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, r);
    ggml_graph_compute_with_ctx(ctx, gf, 1);
    memcpy(out, r->data, (size_t)n * T * 4);
    ggml_free(ctx);
    return 0;
}

/* ggml_rope_custom on x [n_embd_head, n_head, T] with positions pos[T]; mode 0 (LLaMA pairs) or 2 (NeoX) */
REF_API int ref_rope(const float * x, int n_embd_head, int n_head, int T, const int32_t * pos, int n_dims, int mode,
                     float freq_base, float freq_scale, float * out) {
    size_t n = (size_t)n_embd_head * n_head * T;
    struct ggml_context * ctx = new_ctx(n * 16 + (1u << 20));
    if (!ctx) return 1;
    struct ggml_tensor * tx = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, n_embd_head, n_head, T);
    memcpy(tx->data, x, n * 4);
    struct ggml_tensor * tp = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, T);
    memcpy(tp->data, pos, (size_t)T * 4);
    struct ggml_tensor * r = ggml_rope_custom(ctx, tx, tp, n_dims, mode, 0, 0, freq_base, freq_scale, 0.0f, 1.0f, 32.0f, 1.0f);
    struct ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, r);
    ggml_graph_compute_with_ctx(ctx, gf, 1);
    memcpy(out, r->data, n * 4);
    ggml_free(ctx);
    return 0;
}

/* the same with the scaling operands of ggml_rope_custom: linear (freq_scale) and YaRN (n_orig_ctx, ext_factor, attn_factor, beta_fast, beta_slow) */
REF_API int ref_rope_ext(const float * x, int n_embd_head, int n_head, int T, const int32_t * pos, int n_dims, int mode, int n_orig_ctx,
                         float freq_base, float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow, float * out) {
    size_t n = (size_t)n_embd_head * n_head * T;
    struct ggml_context * ctx = new_ctx(n * 16 + (1u << 20));
    if (!ctx) return 1;
    struct ggml_tensor * tx = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, n_embd_head, n_head, T);
    memcpy(tx->data, x, n * 4);
    struct ggml_tensor * tp = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, T);
    memcpy(tp->data, pos, (size_t)T * 4);
    struct ggml_tensor * r = ggml_rope_custom(ctx, tx, tp, n_dims, mode, 0, n_orig_ctx, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
    struct ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, r);
    ggml_graph_compute_with_ctx(ctx, gf, 1);
    memcpy(out, r->data, n * 4);
    ggml_free(ctx);
    return 0;
}

/* ggml_soft_max over rows of x [n, rows] */
REF_API int ref_soft_max(const float * x, int n, int rows, float * out) {
    struct ggml_context * ctx = new_ctx((size_t)n * rows * 16 + (1u << 20));
    if (!ctx) return 1;
    struct ggml_tensor * tx = put2d(ctx, GGML_TYPE_F32, n, rows, x);
    struct ggml_tensor * r  = ggml_soft_max(ctx, tx);
    struct ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, r);
    ggml_graph_compute_with_ctx(ctx, gf, 1);
    memcpy(out, r->data, (size_t)n * rows * 4);
    ggml_free(ctx);
    return 0;
}

/*
 * Single-token-batch attention core as llm_build_kqv assembles it (llama.cpp:4764-4850) after
 * llm_build_kv_store (llama.cpp:4383-4418): K cache F16 [n_ctx][n_embd_gqa], V cache F16 transposed
 * [n_embd_gqa][n_ctx]; the caller passes caches that already contain positions [0, n_past) and
 * this call stores k_cur/v_cur for T new tokens at n_past, then attends with a causal mask.
 * q [n_embd_head, n_head, T] and k_cur [n_embd_head, n_head_kv, T] are post-RoPE; v_cur [n_embd_gqa, T].
 * out: [n_embd, T] (kqv_merged_cont, before wo).  The caches are updated in place.
 */
REF_API int ref_attention(int n_embd_head, int n_head, int n_head_kv, int n_ctx, int n_past, int T,
                          const float * q, const float * k_cur, const float * v_cur,
                          uint16_t * k_cache, uint16_t * v_cache, float * out) {
    const int n_embd = n_embd_head * n_head, n_embd_gqa = n_embd_head * n_head_kv;
    const int n_kv = n_past + T;
    size_t payload = (size_t)n_ctx * n_embd_gqa * 4 + (size_t)T * (n_embd * 8 + n_embd_gqa * 8)
                   + (size_t)n_kv * T * (n_head * 12 + 4) + (size_t)n_embd * T * 16 + (8u << 20);
    struct ggml_context * ctx = new_ctx(payload);
    if (!ctx) return 1;
    struct ggml_tensor * kc = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, (int64_t)n_ctx * n_embd_gqa);
    struct ggml_tensor * vc = ggml_new_tensor_1d(ctx, GGML_TYPE_F16, (int64_t)n_ctx * n_embd_gqa);
    memcpy(kc->data, k_cache, ggml_nbytes(kc));
    memcpy(vc->data, v_cache, ggml_nbytes(vc));
    struct ggml_tensor * tq = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, n_embd_head, n_head, T);
    struct ggml_tensor * tk = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, n_embd_head, n_head_kv, T);
    struct ggml_tensor * tv = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, n_embd_gqa, T);
    memcpy(tq->data, q, ggml_nbytes(tq));
    memcpy(tk->data, k_cur, ggml_nbytes(tk));
    memcpy(tv->data, v_cur, ggml_nbytes(tv));
    struct ggml_tensor * scale = ggml_new_tensor_1d(ctx, GGML_TYPE_F32, 1);
    ((float *)scale->data)[0] = 1.0f / sqrtf((float)n_embd_head);
    struct ggml_tensor * mask = ggml_new_tensor_3d(ctx, GGML_TYPE_F32, n_kv, T, 1);
    for (int j = 0; j < T; ++j)
        for (int i = 0; i < n_kv; ++i)
            ((float *)mask->data)[(size_t)j * n_kv + i] = (i > n_past + j) ? -INFINITY : 0.0f;

    struct ggml_cgraph * gf = ggml_new_graph(ctx);
    const size_t es = ggml_element_size(kc);
    struct ggml_tensor * v_cur_t = ggml_transpose(ctx, ggml_reshape_2d(ctx, tv, n_embd_gqa, T));
    struct ggml_tensor * k_view  = ggml_view_1d(ctx, kc, (int64_t)T * n_embd_gqa, es * n_embd_gqa * n_past);
    struct ggml_tensor * v_view  = ggml_view_2d(ctx, vc, T, n_embd_gqa, n_ctx * es, n_past * es);
    ggml_build_forward_expand(gf, ggml_cpy(ctx, tk, k_view));
    ggml_build_forward_expand(gf, ggml_cpy(ctx, v_cur_t, v_view));

    struct ggml_tensor * qp = ggml_permute(ctx, tq, 0, 2, 1, 3);
    struct ggml_tensor * k  = ggml_view_3d(ctx, kc, n_embd_head, n_kv, n_head_kv, es * n_embd_gqa, es * n_embd_head, 0);
    struct ggml_tensor * kq = ggml_mul_mat(ctx, k, qp);
    kq = ggml_scale(ctx, kq, scale);
    kq = ggml_add(ctx, kq, mask);
    kq = ggml_soft_max(ctx, kq);
    struct ggml_tensor * v   = ggml_view_3d(ctx, vc, n_kv, n_embd_head, n_head_kv, es * n_ctx, es * n_ctx * n_embd_head, 0);
    struct ggml_tensor * kqv = ggml_mul_mat(ctx, v, kq);
    struct ggml_tensor * mrg = ggml_permute(ctx, kqv, 0, 2, 1, 3);
    struct ggml_tensor * cur = ggml_cont_2d(ctx, mrg, n_embd, T);
    ggml_build_forward_expand(gf, cur);
    ggml_graph_compute_with_ctx(ctx, gf, 1);

    memcpy(out, cur->data, (size_t)n_embd * T * 4);
    memcpy(k_cache, kc->data, ggml_nbytes(kc));
    memcpy(v_cache, vc->data, ggml_nbytes(vc));
    ggml_free(ctx);
    return 0;
}

/* codecs, through the type-traits table the executor itself uses (ggml.c:429-455) */
REF_API void ref_quantize_row(int type, const float * x, void * y, int n) {
    ggml_internal_get_type_traits((enum ggml_type) type).from_float_reference(x, y, n);
}
REF_API void ref_quantize_row_fast(int type, const float * x, void * y, int n) {
    ggml_internal_get_type_traits((enum ggml_type) type).from_float(x, y, n);
}
REF_API void ref_dequantize_row(int type, const void * x, float * y, int n) {
    ggml_internal_get_type_traits((enum ggml_type) type).to_float(x, y, n);
}
REF_API void ref_fp32_to_fp16_row(const float * x, uint16_t * y, int n) { ggml_fp32_to_fp16_row(x, y, n); }
REF_API void ref_fp16_to_fp32_row(const uint16_t * x, float * y, int n) { ggml_fp16_to_fp32_row(x, y, n); }

REF_API void ref_init(void) {
    struct ggml_init_params ip = { 1u << 20, NULL, false };
    struct ggml_context * ctx = ggml_init(ip);   /* fills the fp16 / exp lookup tables */
    ggml_free(ctx);
}

#ifdef GGML_USE_CUBLAS
/*
 * The same FFN block, but with the reference compiled with -DGGML_USE_CUBLAS and linked against THIS repository's
 * backend library in place of ggml-cuda.cu: the reference's own op constructors, graph and executor
 * (ggml_graph_compute, two threads, as the hybrid ops require: ggml.c:16714-16720) drive the HIP kernels through
 * ggml_cuda_compute_forward.  Graph as llm_build_ffn_sparse builds it under GGML_USE_CUBLAS (llama.cpp:4546-4757):
 *   n_bucket == 0 : full-GPU fast path, every FFN tensor and node on the GPU (src[3] == NULL);
 *   n_bucket  > 0 : hybrid, CPU part (full matrices, gpu_idx) + GPU part (bucket rows, gpu_bucket) + ggml_add.
 */
#include "ggml-cuda.h"

static struct ggml_tensor * to_gpu(struct ggml_tensor * t) {
    t->backend = GGML_BACKEND_GPU;
    ggml_cuda_transform_tensor(t->data, t);
    return t;
}
/* nodes placed on the device outside the scratch buffer own their memory (ggml-cuda.cu:9102-9109); released after the run */
static struct ggml_tensor * g_gpu_nodes[64];
static int g_n_gpu_nodes = 0;
static struct ggml_tensor * node_gpu(struct ggml_tensor * t) {
    ggml_cuda_assign_buffers_no_scratch(t);
    if (g_n_gpu_nodes < 64) g_gpu_nodes[g_n_gpu_nodes++] = t;
    return t;
}

static struct ggml_tensor * sparse_mm(struct ggml_context * ctx, struct ggml_tensor * w, struct ggml_tensor * w_gpu, struct ggml_tensor * x,
                                      struct ggml_tensor * idx, struct ggml_tensor * gid, struct ggml_tensor * bkt, int full_gpu) {
    if (full_gpu) return node_gpu(ggml_mul_mat_idx(ctx, w_gpu, x, idx, NULL));
    struct ggml_tensor * out = ggml_mul_mat_idx(ctx, w, x, idx, gid);
    struct ggml_tensor * out_gpu = node_gpu(ggml_mul_mat_idx_upscale(ctx, w_gpu, x, idx, bkt, out->ne[0]));
    return ggml_add(ctx, out, out_gpu);
}

static void * gather_rows(const void * w, size_t rb, const int32_t * bucket, int n) {
    char * p = (char *)malloc(rb * (size_t)(n ? n : 1));
    for (int i = 0; i < n; ++i) memcpy(p + rb * i, (const char *)w + rb * (size_t)bucket[i], rb);
    return p;
}

REF_API int ref_ffn_sparse_gpu_parts(int d, int ff, int r, int T, int wtype, int has_gate,
                                     const void * up_w, const void * gate_w, const void * down_t,
                                     const uint16_t * fc1, const uint16_t * fc2,
                                     const float * x_ffn, const float * x_pred,
                                     const int32_t * gpu_idx, const int32_t * gpu_bucket, int n_bucket,
                                     float threshold, float * logits, float * out,
                                     float * h_out, float * out_cpu_part, float * out_gpu_part);

REF_API int ref_ffn_sparse_gpu(int d, int ff, int r, int T, int wtype, int has_gate,
                               const void * up_w, const void * gate_w, const void * down_t,
                               const uint16_t * fc1, const uint16_t * fc2,
                               const float * x_ffn, const float * x_pred,
                               const int32_t * gpu_idx, const int32_t * gpu_bucket, int n_bucket,
                               float threshold, float * logits, float * out) {
    return ref_ffn_sparse_gpu_parts(d, ff, r, T, wtype, has_gate, up_w, gate_w, down_t, fc1, fc2, x_ffn, x_pred, gpu_idx, gpu_bucket, n_bucket,
                                    threshold, logits, out, NULL, NULL, NULL);
}

/* the same graph; a hybrid run also hands back the merged h ("ffn_gate_par", [T][ff]) and the two operands of the final ggml_add:
 * the host node's share ("ffn_down_sparse", [T][d], computed by the reference's own CPU axpy on two threads) and the backend
 * node's share ("ffn_down_sparse_gpu", [T][d]); each may be NULL */
REF_API int ref_ffn_sparse_gpu_parts(int d, int ff, int r, int T, int wtype, int has_gate,
                                     const void * up_w, const void * gate_w, const void * down_t,
                                     const uint16_t * fc1, const uint16_t * fc2,
                                     const float * x_ffn, const float * x_pred,
                                     const int32_t * gpu_idx, const int32_t * gpu_bucket, int n_bucket,
                                     float threshold, float * logits, float * out,
                                     float * h_out, float * out_cpu_part, float * out_gpu_part) {
    enum ggml_type wt = (enum ggml_type) wtype;
    const int full_gpu = n_bucket == 0;
    const size_t rb = tensor_bytes(wt, d, 1);
    size_t payload = 6 * tensor_bytes(wt, d, ff) + 2u * ((size_t)d * r + (size_t)r * ff)
                   + (size_t)T * (2u * d + 16u * ff + 2u * r) * sizeof(float) + (size_t)ff * 8 + (size_t)d * 256 + (16u << 20);
    struct ggml_context * ctx = new_ctx(payload);
    if (!ctx) return 1;
    sparse_pred_threshold = threshold;
    ggml_cuda_set_device_constants(threshold);

    struct ggml_tensor * t_fc1 = to_gpu(put2d(ctx, GGML_TYPE_F16, d, r, fc1));
    struct ggml_tensor * t_fc2 = to_gpu(put2d(ctx, GGML_TYPE_F16, r, ff, fc2));
    struct ggml_tensor * t_x   = put2d(ctx, GGML_TYPE_F32, d, T, x_ffn);
    struct ggml_tensor * t_xp  = put2d(ctx, GGML_TYPE_F32, d, T, x_pred);
    struct ggml_tensor *up = NULL, *gate = NULL, *down = NULL, *up_g, *gate_g = NULL, *down_g, *gid = NULL, *bkt = NULL;
    void * tmp[3] = {NULL, NULL, NULL};
    if (full_gpu) {
        up_g = to_gpu(put2d(ctx, wt, d, ff, up_w));
        if (has_gate) gate_g = to_gpu(put2d(ctx, wt, d, ff, gate_w));
        down_g = to_gpu(put2d(ctx, wt, d, ff, down_t));
    } else {
        up = put2d(ctx, wt, d, ff, up_w); down = put2d(ctx, wt, d, ff, down_t);
        if (has_gate) gate = put2d(ctx, wt, d, ff, gate_w);
        tmp[0] = gather_rows(up_w, rb, gpu_bucket, n_bucket);   up_g   = to_gpu(put2d(ctx, wt, d, n_bucket, tmp[0]));
        tmp[1] = gather_rows(down_t, rb, gpu_bucket, n_bucket); down_g = to_gpu(put2d(ctx, wt, d, n_bucket, tmp[1]));
        if (has_gate) { tmp[2] = gather_rows(gate_w, rb, gpu_bucket, n_bucket); gate_g = to_gpu(put2d(ctx, wt, d, n_bucket, tmp[2])); }
        gid = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, ff);       memcpy(gid->data, gpu_idx, (size_t)ff * 4);
        bkt = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, n_bucket); memcpy(bkt->data, gpu_bucket, (size_t)n_bucket * 4);
    }

    struct ggml_tensor * idx = node_gpu(ggml_mul_mat(ctx, t_fc1, t_xp));
    idx = node_gpu(ggml_relu(ctx, idx));
    idx = ggml_mul_mat(ctx, t_fc2, idx);
    if (full_gpu) node_gpu(idx);                                 /* hybrid: the sparsity index stays on the CPU (llama.cpp:4693-4695) */

    struct ggml_tensor * upo = sparse_mm(ctx, up, up_g, t_x, idx, gid, bkt, full_gpu);
    struct ggml_tensor * cur;
    if (has_gate) {
        struct ggml_tensor * gto = sparse_mm(ctx, gate, gate_g, t_x, idx, gid, bkt, full_gpu);
        struct ggml_tensor * act = ggml_relu(ctx, gto);
        cur = ggml_mul(ctx, act, upo);
        if (full_gpu) { node_gpu(act); node_gpu(cur); }
    } else {
        cur = ggml_relu(ctx, upo);
        if (full_gpu) node_gpu(cur);
    }
    struct ggml_tensor * res, * o_cpu = NULL, * o_gpu = NULL;
    if (full_gpu) {
        res = node_gpu(ggml_axpy(ctx, down_g, cur, idx, NULL));
    } else {
        o_cpu = ggml_axpy(ctx, down, cur, idx, gid);
        o_gpu = node_gpu(ggml_axpy(ctx, down_g, cur, idx, bkt));
        res = node_gpu(ggml_add(ctx, o_cpu, o_gpu));
    }

    struct ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, res);
    ggml_graph_compute_with_ctx(ctx, gf, 2);

    if (idx->backend == GGML_BACKEND_GPU) ggml_cuda_copy_to_host(idx);
    ggml_cuda_copy_to_host(res);
    if (logits) memcpy(logits, idx->data, (size_t)ff * T * 4);
    if (out)    memcpy(out, res->data, (size_t)d * T * 4);
    if (!full_gpu) {
        if (h_out) memcpy(h_out, cur->data, (size_t)ff * T * 4);
        if (out_cpu_part) memcpy(out_cpu_part, o_cpu->data, (size_t)d * T * 4);
        if (out_gpu_part) { ggml_cuda_copy_to_host(o_gpu); memcpy(out_gpu_part, o_gpu->data, (size_t)d * T * 4); }
    }

    struct ggml_tensor * owned[] = {t_fc1, t_fc2, up_g, gate_g, down_g};
    for (int i = 0; i < 5; ++i) if (owned[i]) ggml_cuda_free_data(owned[i]);
    for (int i = 0; i < g_n_gpu_nodes; ++i) ggml_cuda_free_data(g_gpu_nodes[i]);
    g_n_gpu_nodes = 0;
    ggml_cuda_free_scratch();
    for (int i = 0; i < 3; ++i) free(tmp[i]);
    ggml_free(ctx);
    return 0;
}
#endif

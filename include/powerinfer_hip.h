/*
 * C ABI of libpowerinfer_hip.so -- the MI355X (gfx950) implementation of PowerInfer's sparse decode
 * token loop.  Plain pointers and sizes only.  Three layers, each a drop-in for a slice of the
 * reference (citations are file:line into the reference tree):
 *
 *   1. pi_k_*      one launcher per hot operator (what ggml-cuda.cu's op functions launch)
 *   2. pi_model_*  the decode loop with resident weights (what llama_decode drives per token)
 *   3. ggml_cuda_* the reference's own backend entry points, same names and contracts
 *                  (declared in ggml_backend_abi.h)
 *
 * All device pointers are HIP device addresses on the current device.  Unless stated otherwise a
 * function returns 0 on success and a negative code on error; pi_last_error() then describes it.
 * Launchers are asynchronous on `stream` (a hipStream_t passed as void*, NULL = the default stream).
 */
#ifndef POWERINFER_HIP_H
#define POWERINFER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PI_API __attribute__((visibility("default")))

typedef void * pi_stream_t;

/* element types: numeric values of enum ggml_type (ggml.h:333-355) */
enum { PI_TYPE_F32 = 0, PI_TYPE_F16 = 1, PI_TYPE_Q4_0 = 2, PI_TYPE_I32 = 18 };

enum { PI_OK = 0, PI_E_ARG = -1, PI_E_HIP = -2, PI_E_UNSUPPORTED = -3, PI_E_STATE = -4 };

/* ---- runtime plumbing (ggml_init_cublas, ggml-cuda.cu:6463-6534; host/device copies :8005-8080) ---- */
PI_API int          pi_init(int device);
PI_API const char * pi_last_error(void);
PI_API int          pi_device_name(char * buf, size_t n);
PI_API void *       pi_malloc(size_t bytes);                 /* NULL on failure */
PI_API int          pi_free(void * dptr);
/* pinned host memory that kernels read and write directly over the host link (coherent: a kernel's stores are visible to the host once
 * the kernel has completed or has released them at system scope); for the logits / h / output-share operands of hybrid layers */
PI_API void *       pi_malloc_host(size_t bytes);            /* NULL on failure */
PI_API int          pi_free_host(void * hptr);
PI_API int          pi_memset(void * dptr, int byte, size_t bytes);
PI_API int          pi_memcpy_h2d(void * dptr, const void * host, size_t bytes);
PI_API int          pi_memcpy_d2h(void * host, const void * dptr, size_t bytes);
PI_API int          pi_memcpy_d2d(void * dst, const void * src, size_t bytes);
PI_API int          pi_sync(void);
/* deterministic N(0, std^2) fill rounded to fp16 (synthetic weights generated in HBM); row_bias, if
 * not NULL, holds one fp32 per row of `cols` elements that is added before rounding */
PI_API int          pi_fill_normal_f16(void * dptr, size_t n, uint64_t seed, float std, const float * row_bias, int cols, pi_stream_t stream);
/* the same values (rounded to fp16 first) quantised to Q4_0 blocks of 32 as quantize_row_q4_0_reference does
 * (ggml-quants.c:428-463); n_weights % 32 == 0, dptr receives n_weights / 32 * 18 bytes */
PI_API int          pi_fill_normal_q4_0(void * dptr, size_t n_weights, uint64_t seed, float std, pi_stream_t stream);
/* event timing on a stream: returns milliseconds between two recorded marks */
PI_API void *       pi_event_create(void);
PI_API int          pi_event_record(void * ev, pi_stream_t stream);
PI_API int          pi_event_elapsed_ms(void * start, void * stop, float * ms);   /* synchronises on stop */
PI_API int          pi_event_destroy(void * ev);

/* ---- operator launchers ---------------------------------------------------------------------------- */

/* optional normalisation applied to the activation vector before a mat-vec:
 * kind 0 none | 1 RMSNorm (rms_norm_f32, ggml-cuda.cu:667) | 2 LayerNorm (norm_f32, ggml-cuda.cu:621);
 * y = norm(x) * w (+ b).  w, b: device fp32 [cols] or NULL. */
typedef struct pi_norm {
    int32_t       kind;
    float         eps;
    const float * w;
    const float * b;
} pi_norm;

enum { PI_EPI_NONE = 0, PI_EPI_RELU = 1, PI_EPI_ADD = 2, PI_EPI_ADD2 = 3 };

/*
 * Dense mat-vec  y[rows] = epi(W[rows][cols] . act(x)),  batch 1.
 * Replaces dequantize_mul_mat_vec<1,1,convert_f16> (ggml-cuda.cu:4349, launcher :5629) and
 * mul_mat_vec_q<QK4_0,...> with quantize_q8_1 (ggml-cuda.cu:4311, 1624, launcher :5480) for
 * attention projections, predictor fc1 and lm-head.  Activations are rounded the way the CPU path
 * rounds them (fp16 for F16 weights, Q8_0 blocks for Q4_0 weights; ggml.c:9703-9716).
 * epilogue: NONE | RELU | ADD (y += add1) | ADD2 (y = (y + add1) + add2).
 */
PI_API int pi_k_gemv(int wtype, const void * W, int rows, int cols, const float * x, const pi_norm * norm,
                     int epilogue, const float * add1, const float * add2, float * y, pi_stream_t stream);
/* up to three F16 matrices of the same width against one vector in one launch: y[i][rows[i]] = W[i] . fp16(norm(x)).  For hosts that
 * keep the q, k and v projections as separate tensors (llama.cpp:4989-4995: three mul_mat nodes on the same normalised input); cols
 * 4096, 5120 or 8192.  Every product is the one pi_k_gemv computes for that matrix. */
PI_API int pi_k_gemv_multi_f16(const void * const * W, const int * rows, int n_mat, int cols, const float * x, const pi_norm * norm,
                               float * const * y, pi_stream_t stream);

/* scratch shared by the predictor / sparse kernels of one stream; sized for the largest ff and d used */
typedef struct pi_workspace pi_workspace;
PI_API pi_workspace * pi_workspace_create(int max_ff, int max_d);
PI_API int            pi_workspace_destroy(pi_workspace * ws);

/*
 * Predictor output layer fused with the activity test:
 *   logits[ff] = fc2[ff][r] . fp16(hidden[r]);  neuron j active iff !(logits[j] < threshold)
 * (mul_mat "mlp_pre_out", llama.cpp:4693; test ggml-cuda.cu:4695 / ggml.c:14256).  Each workgroup of 32
 * neurons emits one 32-bit activity word by wave ballot; the words stay in the workspace.
 * If active_rows/n_active are given, the ascending list of active rows and its length are produced as well
 * (second, single-workgroup launch: popcount prefix sums over the words).  With bucket == NULL rows are neuron
 * indices 0..ff-1.  With a gpu_bucket (sorted original indices of the GPU-resident neurons,
 * llama.cpp:2820-2870) the candidates are rows 0..n_bucket-1 of the compact GPU matrices and row i is active
 * iff neuron bucket[i] is.  With active_rows == NULL the list is left to pi_k_sparse_upgate(from_mask = 1),
 * which builds it on the fly.  The reference never materialises this list (it re-tests the mask in every kernel).
 * zero_fill (optional): fp32 [ff] cleared by the same launch (the dense h vector of the Q4_0 path).
 */
PI_API int pi_k_predictor_fc2(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                              const int32_t * bucket, int n_bucket, float * logits,
                              int32_t * active_rows, int32_t * n_active, float * zero_fill,
                              pi_workspace * ws, pi_stream_t stream);

/* the same test + compaction over logits that already exist (hybrid split: logits computed elsewhere) */
PI_API int pi_k_compact_active(const float * logits, int ff, float threshold, const int32_t * bucket, int n_bucket,
                               int32_t * active_rows, int32_t * n_active, pi_workspace * ws, pi_stream_t stream);

/*
 * Sparse up/gate mat-vec over the active rows only, fused with the activation:
 *   h[k] = relu(gate[row_k] . x) * (up[row_k] . x)      (gate != NULL, LLM_FFN_PAR)
 *   h[k] = relu(up[row_k] . x)                          (gate == NULL, Falcon)
 * Replaces dequantize_mul_mat_vec_sparse (ggml-cuda.cu:4685) / mul_mat_vec_q(lst, idx) (:5490) plus
 * relu_f32 and mul_f32.
 * from_mask != 0: the active set is taken from the mask words the last pi_k_predictor_fc2 on this workspace
 *   left; every workgroup derives rank -> row from a popcount prefix table, and active_rows[k] / *n_active are
 *   WRITTEN here (ascending list as a by-product).  bucket must be NULL.
 * from_mask == 0: active_rows / n_active are inputs (produced by pi_k_predictor_fc2 or pi_k_compact_active).
 * h_compact[k] is indexed like active_rows; if h_dense != NULL the value is also scattered to h_dense[neuron]
 * (neuron = bucket ? bucket[row] : row), which the caller has zeroed.  up_dense/gate_dense (optional, list
 * mode only) receive the raw dot products the same way (GGML_OP_MUL_MAT_SPARSE output).
 */
PI_API int pi_k_sparse_upgate(int wtype, const void * up, const void * gate, int cols, int ff, const float * x, const pi_norm * norm,
                              int from_mask, int32_t * active_rows, int32_t * n_active, const int32_t * bucket,
                              float * h_compact, float * h_dense, float * up_dense, float * gate_dense,
                              pi_workspace * ws, pi_stream_t stream);

/*
 * Sparse down projection (GGML_OP_AXPY):  out[cols] = epi( sum_k act(h_compact[k]) * down_t[row_k][:] ).
 * Replaces dequantize_mul_mat_axpy_sparse (ggml-cuda.cu:4541) and _sparse_pro (:4479) and their
 * per-row global atomics.  F16: a workgroup owns 128 output columns and all active rows, its 16 waves split
 * the rows and merge through LDS in a fixed order.  Q4_0: column tiles x row groups with a fixed-order second
 * stage.  Either way the result is deterministic.  Rows whose rounded h is zero are not read.
 * act(): fp16 rounding for F16 weights; for Q4_0 weights h is quantised to Q8_0 over blocks of 32
 * neurons as the CPU path does (ggml.c:14465-14618), which needs the dense neuron-indexed vector
 * h_dense (zeros at inactive neurons; may be NULL for F16) and the bucket that maps rows to neurons.
 * n_rows: number of candidate rows (capacity of h_compact / active_rows): ff, or the bucket size.
 * epilogue: NONE | ADD | ADD2 as for pi_k_gemv.
 */
PI_API int pi_k_sparse_axpy(int wtype, const void * down_t, int cols, int n_rows, const float * h_compact,
                            const float * h_dense, const int32_t * bucket,
                            const int32_t * active_rows, const int32_t * n_active,
                            int epilogue, const float * add1, const float * add2, float * out,
                            pi_workspace * ws, pi_stream_t stream);

/*
 * Full-GPU F16 fast route of the sparse FFN: predictor fc2, the activity test and the sparse up/gate mat-vec in
 * ONE launch, and the down projection straight from the dense h vector in a second one.  Replaces the
 * mul_mat(fc2) -> dequantize_mul_mat_vec_sparse x2 -> relu -> mul chain of llm_build_ffn_sparse
 * (llama.cpp:4688-4740; ggml-cuda.cu:4349, 4685) and dequantize_mul_mat_axpy_sparse (ggml-cuda.cu:4541).
 *   pi_k_pred_upgate: a workgroup owns 32 consecutive neurons: logits[n] = fc2[n] . fp16(hidden), active iff
 *     !(logit < threshold), h_dense[n] = relu(gate[n] . xn) * (up[n] . xn) for active n (relu(up[n] . xn) when
 *     gate == NULL) and 0 otherwise, xn = fp16(norm(x)).  Writes all ff entries of h_dense, the mask words of
 *     the workspace and, if logits != NULL, the ff predictor logits.  Shapes: see pi_k_pred_upgate_supported.
 *   pi_k_sparse_axpy_dense: out[cols] = epi( sum over n with fp16(h_dense[n]) != 0 of fp16(h_dense[n]) *
 *     down_t[n][:] ), ascending n within a fixed reduction tree; cols % 64 == 0.  If n_active != NULL it
 *     receives the number of set bits in the workspace's mask words (the predictor's active count).
 */
/*
 * The same block in its tightest form (what the F16 decode loop runs at cols == 4096): one launch computes fc2, the
 * activity test, gate/up, h and each workgroup's share of the down projection; a small second launch adds the
 * per-workgroup partial vectors in a fixed order plus the residual(s):
 *   out[cols] = epi( sum_n fp16(h[n]) * down_t[n][:] ),  h[n] as for pi_k_pred_upgate.
 * logits (fp32 [ff]), h_dense (fp32 [ff], every entry written) and n_active (predictor's active count) are
 * optional outputs for inspection.  Shapes: see pi_k_sparse_ffn_supported.
 */
/* Q4_0 weights, cols == 4096: predictor fc2 + mask + up/gate of the GPU-resident neurons in one launch, then the down
 * projection as per-workgroup partial vectors plus one reduction.  Replaces the GPU nodes of llm_build_ffn_sparse for Q4_0
 * (mul_mat_vec_sparse_q ggml-cuda.cu:7232, dequantize_axpy :7593) and follows the CPU arithmetic (Q8_0 input,
 * ggml-quants.c:2512-2650; Q8_0 h over 32-neuron blocks, ggml.c:14465-14618, ggml-quants.c:2426-2509).
 * hot_words[ff/32]: bit j of word g set iff neuron 32g+j is GPU-resident; hot_prefix[g]: GPU-resident neurons before group g
 * (= row of the compact matrices, llama.cpp:2820-2967); both NULL: every neuron resident, row = neuron.
 * h_dense[ff] gets h for active resident neurons and 0 elsewhere.  logits, h_dense and xq8_out (cols/32 blocks of
 * {fp16 d, int8 qs[32]}: the Q8_0 form of the normalised input, optional) may be pinned host memory, and so may `h` of the
 * partials call (the vector after the host share filled in its neurons) and add1/add2 of the reduction. */
PI_API int pi_k_pred_upgate_q4_supported(int ff, int r, int cols);
PI_API int pi_k_pred_upgate_q4(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                               const void * up_q4, const void * gate_q4, int cols, const float * x, const pi_norm * norm,
                               const uint32_t * hot_words, const int32_t * hot_prefix,
                               float * logits, float * h_dense, void * xq8_out, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_axpy_q4_partials(const void * down_t_q4, int cols, int ff, const float * h,
                                 const uint32_t * hot_words, const int32_t * hot_prefix, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_axpy_q4_reduce(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out,
                               int32_t * n_active, pi_workspace * ws, pi_stream_t stream);
/* The same two launches when the GPU computes the neurons outside the hot set as well, reading their rows where they lie: up_rest /
 * gate_rest / down_t_rest hold exactly the non-resident neurons' rows in ascending neuron order (row = neuron index minus the
 * resident neurons before it) and may be pinned host memory - only the rows of active neurons cross the host link.  The split
 * of llama.cpp:2820-2967 (hot rows in VRAM, the rest in host memory) is kept; what moves is who multiplies the cold rows
 * (the CPU half of llm_build_sparse_mul_mat / llm_build_sparse_axpy, llama.cpp:4581-4593, 4635-4646).  h_dense then holds h of
 * every active neuron.  *_rest == NULL: identical to the calls above. */
PI_API int pi_k_pred_upgate_q4_split(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                                     const void * up_q4, const void * gate_q4, const void * up_rest_q4, const void * gate_rest_q4,
                                     int cols, const float * x, const pi_norm * norm,
                                     const uint32_t * hot_words, const int32_t * hot_prefix,
                                     float * logits, float * h_dense, void * xq8_out, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_axpy_q4_partials_split(const void * down_t_q4, const void * down_t_rest_q4, int cols, int ff, const float * h,
                                       const uint32_t * hot_words, const int32_t * hot_prefix, pi_workspace * ws, pi_stream_t stream);
/* KV cache maintenance.  pi_k_k_shift replaces the graph of llm_build_k_shift (llama.cpp:4332-4381; the fp16 RoPE
 * ggml.c:11327-11478): cache [rows = layers x kv heads][n_ctx][hd] fp16, delta[n_cells] positions to rotate each cell by.
 * pi_k_kv_compact moves cell map[j] to cell j (map ascending) through `stage` ([rows][n_new][hd] fp16): this implementation keeps
 * the live cells contiguous instead of searching a ring for free slots (llama_kv_cache_find_slot, llama.cpp:1683-1736).
 * freq_scale: linear RoPE scaling as in pi_k_rope_kv_store. */
PI_API int pi_k_k_shift(void * k_cache, int rows, int n_ctx, int hd, int mode, float theta_scale, float freq_scale, const int32_t * delta, int n_cells, pi_stream_t stream);
PI_API int pi_k_kv_compact(void * cache, void * stage, int rows, int n_ctx, int hd, const int32_t * map, int n_new, pi_stream_t stream);
/* the K-shift on the reference's own cache layout, K cells [n_layer][n_cells][n_head_kv][hd] (the strided view llm_build_k_shift rotates,
 * llama.cpp:4366-4378): every cell's rows are rotated by delta[cell] positions, cells with delta 0 are left alone */
PI_API int pi_k_k_shift_cells(void * k_cache, int n_layer, int n_cells, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale,
                              const int32_t * delta, pi_stream_t stream);
/* Shapes of the fused block: cols 4096 or 8192 with a predictor of rank 512 or 1024 and ff % 32 == 0; cols 5120 with rank 1280 (the
 * 13B shape) where ff gives every compute unit 33..60 neurons, with a norm that carries its weights (or none).  Needs pi_init
 * (the answer depends on the device's compute units).  _hot_supported: the shapes of the hybrid forms below (the first group only). */
PI_API int pi_k_sparse_ffn_supported(int ff, int r, int cols);
PI_API int pi_k_sparse_ffn_hot_supported(int ff, int r, int cols);
/* Workgroups of the fused launch for a layer that is whole on the device (0: shape not covered).  Workgroup b computes neurons
 * [ff * b / n, ff * (b + 1) / n) and stores one partial output vector; a caller that arranges a layer's rows by firing rate deals
 * them out over these ranges (pi_model_finalize does, from PI_T_NEURON_RATE). */
PI_API int pi_k_sparse_ffn_workgroups(int ff, int r, int cols);
/* the two launches of pi_k_sparse_ffn on their own, for callers that overlap the block with an independent branch (Falcon's
 * attention reads the same layer input): _partials may run on another stream, _reduce needs it and the residual operands done */
PI_API int pi_k_sparse_ffn_partials(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                                    const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols,
                                    const float * x, const pi_norm * norm, float * logits, float * h_dense,
                                    pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_sparse_ffn_reduce(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out,
                                  int32_t * n_active, pi_workspace * ws, pi_stream_t stream);
/* the same two launches for a hot/cold split layer (F16): only the GPU-resident neurons are computed, from the compact matrices of
 * the bucket (hot_words / hot_prefix as for pi_k_pred_upgate_q4); logits and xn_f16_out (the fp16-rounded normalised input, cols
 * values, optional) may be pinned host memory for the host share; _reduce_hot counts the resident active neurons, and its add1 /
 * add2 may be pinned host memory (the host share's output).  GPU part of llm_build_sparse_mul_mat / _axpy, llama.cpp:4581-4646. */
PI_API int pi_k_sparse_ffn_partials_hot(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                                        const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols,
                                        const float * x, const pi_norm * norm, const uint32_t * hot_words, const int32_t * hot_prefix,
                                        float * logits, float * h_dense, void * xn_f16_out, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_sparse_ffn_reduce_hot(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out,
                                      int32_t * n_active, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_sparse_ffn(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                           const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols,
                           const float * x, const pi_norm * norm,
                           int epilogue, const float * add1, const float * add2, float * out,
                           float * logits, float * h_dense, int32_t * n_active,
                           pi_workspace * ws, pi_stream_t stream);
/*
 * pi_k_sparse_ffn for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as pi_k_sparse_ffn minus the workspace:
 * the per-workgroup partial vectors and the activity words live in a static device array of
 * pi_k_sparse_ffn_noalloc_scratch_bytes() (8 MiB + 32 KiB) that each GPU the library runs on holds until the process ends.  The call
 * allocates and frees nothing.  Shapes whose partial vectors exceed 8 MiB ((ff / 32) * cols floats at cols 4096, (ff / 128) * cols
 * at cols 8192 when ff / 128 >= 256) or with ff > 131072 are refused with PI_E_UNSUPPORTED (_supported tells beforehand).
 * All calls on one GPU share the array: calls that overlap on one GPU (different streams or threads) race; calls on one stream
 * are ordered.  Nothing in the array has to be cleared between calls (every word a call reads it has written itself).
 */
PI_API size_t pi_k_sparse_ffn_noalloc_scratch_bytes(void);
PI_API int pi_k_sparse_ffn_noalloc_supported(int ff, int r, int cols);
PI_API int pi_k_sparse_ffn_noalloc(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                                   const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols,
                                   const float * x, const pi_norm * norm,
                                   int epilogue, const float * add1, const float * add2, float * out,
                                   float * logits, float * h_dense, int32_t * n_active, pi_stream_t stream);
PI_API int pi_k_pred_upgate_supported(int ff, int r, int cols);      /* 1 if the fused kernel covers the shape */
PI_API int pi_k_pred_upgate(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                            const void * up_f16, const void * gate_f16, int cols, const float * x, const pi_norm * norm,
                            float * logits, float * h_dense, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_sparse_axpy_dense(const void * down_t_f16, int cols, int ff, const float * h_dense, int32_t * n_active,
                                  int epilogue, const float * add1, const float * add2, float * out,
                                  pi_workspace * ws, pi_stream_t stream);

/*
 * Batched decode step: T <= 16 tokens, one per sequence (examples/batched/batched.cpp:100-260 drives llama_decode with
 * n_tokens = n_parallel).  The weights are streamed once per step; the dense mat-muls and the sparse gate/up run on the
 * matrix cores (the batch >= 8 dense cross-over the reference takes through cuBLAS, ggml-cuda.cu:7717-7756, and its
 * mul_mat_batch_sparse kernels, :6994-7034).  Vectors of a step are token-major: x[T][cols], y[T][rows].
 *   pi_k_norm_round_f16: out_f16[t] = fp16(norm(x[t])) -- what the CPU path feeds every F16 dot (ggml.c:9703-9716);
 *     out_plain_f16 (optional) receives fp16(x[t]) from the same pass (the predictor reads the un-normalised vector).
 *   pi_k_gemm_f16:       y[t][row] = epi( W[row] . xn[t] ), cols % 128 == 0; add1/add2 are [T][rows]; y_f16 (optional) receives
 *     fp16(y) for the next mat-mul.
 *   pi_k_batch_predictor_fc2: logits[t][n] = fc2[n] . hidden_f16[t]; the epilogue also flags in the workspace every neuron with
 *     !(logit < threshold) for at least one token.
 *   pi_k_batch_sparse_ffn: logits [T][ff] and the workspace flags from pi_k_batch_predictor_fc2; union_rows/n_union receive the
 *     ascending list of neurons active for at least one token (each weight row is read once for the whole step);
 *     out[t] = epi( sum over union rows active for t of fp16(h[t][n]) * down_t[n][:] ), h as in pi_k_sparse_upgate;
 *     cols % 256 == 0.
 */
PI_API int pi_k_norm_round_f16(const float * x, int T, int cols, const pi_norm * norm, void * out_f16, void * out_plain_f16, pi_stream_t stream);
PI_API int pi_k_gemm_f16(const void * W_f16, int rows, int cols, const void * xn_f16, int T, int epilogue,
                         const float * add1, const float * add2, float * y, void * y_f16, pi_stream_t stream);
PI_API int pi_k_batch_predictor_fc2(const void * fc2_f16, int ff, int r, const void * hidden_f16, int T, float threshold, float * logits,
                                    pi_workspace * ws, pi_stream_t stream);
/* the union list and count alone, from the flags pi_k_batch_predictor_fc2 left in the workspace */
PI_API int pi_k_batch_union_count(int ff, int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_batch_sparse_ffn(const float * logits, int T, int ff, float threshold,
                                 const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols, const void * xn_f16,
                                 int epilogue, const float * add1, const float * add2, float * out,
                                 int32_t * union_rows, int32_t * n_union,
                                 pi_workspace * ws, pi_stream_t stream);
/*
 * The same four with the step's fp16 activations in the operand layout of the matrix cores instead of [T][cols]: 16 token slots
 * (whatever T is) laid out [cols / 8][16][8], element (t, c) at ((c / 8) * 16 + t) * 8 + c % 8, so that the fragment a wave loads
 * for a 32-column step is one contiguous kilobyte instead of 16 token rows x 64 bytes.  Same arithmetic, bit for bit; a buffer holds
 * 16 * cols fp16 values.  No counterpart in the reference (its batch kernels read ggml's row-major src1, ggml-cuda.cu:6994-7034): the
 * layout exists because the activation loads, not the weight loads, were what the vector L1 of a compute unit spent its cycles on.
 *   pi_k_norm_round_f16_ol: both outputs in the operand layout (cols % 8 == 0).
 *   pi_k_gemm_f16_ol: xn_ol read and y_ol (optional, rows % 8 == 0) written in it; y, add1, add2 stay [T][rows] fp32.
 *   pi_k_batch_predictor_fc2_ol: hidden_ol in it (the y_ol of the fc1 mat-mul).
 *   pi_k_batch_sparse_ffn_ol: xn_ol in it (cols % 256 == 0 and ff * cols < 2^31 required).
 */
PI_API int pi_k_norm_round_f16_ol(const float * x, int T, int cols, const pi_norm * norm, void * out_ol, void * out_plain_ol, pi_stream_t stream);
PI_API int pi_k_gemm_f16_ol(const void * W_f16, int rows, int cols, const void * xn_ol, int T, int epilogue,
                            const float * add1, const float * add2, float * y, void * y_ol, pi_stream_t stream);
PI_API int pi_k_batch_predictor_fc2_ol(const void * fc2_f16, int ff, int r, const void * hidden_ol, int T, float threshold, float * logits,
                                       pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_batch_sparse_ffn_ol(const float * logits, int T, int ff, float threshold,
                                    const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols, const void * xn_ol,
                                    int epilogue, const float * add1, const float * add2, float * out,
                                    int32_t * union_rows, int32_t * n_union,
                                    pi_workspace * ws, pi_stream_t stream);

/* Prompt chunks on this library's own mat-mul kernel (the prompt phase of llama_decode, where the reference goes through cuBLAS and
 * its batch kernels, ggml-cuda.cu:7662-7756, 6994-7034): pi_k_gemm_tile_f16 is pi_k_gemm_f16 for chunks of any length, both operands
 * tiled through LDS (64 columns per stage, two stages in LDS and two more in flight): cols % 64 == 0, operands 16-byte aligned.
 * tile = 0 lets the library choose the output tile from the number of workgroups it gives the device; 256128, 192128 (eight waves per
 * workgroup), 128128, 96128, 128064, 64128, 64064 (four waves; weight rows x 1000 + tokens) forces one, for tests and measurement.  pi_k_ffn_h_f16 forms h_f16[t][n] = fp16(relu(gate) * up)
 * where !(logits[t][n] < threshold) and 0 elsewhere from dense gate/up products (gate may be NULL: relu(up)); pi_k_transpose_f16 writes
 * out[cols][rows] of an fp16 matrix in[rows][cols] (the down projection of a chunk is a mat-mul over the neurons and wants them
 * contiguous). */
PI_API int pi_k_gemm_tile_f16(const void * W_f16, int rows, int cols, const void * xn_f16, int T, int epilogue,
                              const float * add1, const float * add2, float * y, void * y_f16, int tile, pi_stream_t stream);
/* Steps of up to 16 tokens on Q4_0 weights with the CPU path's arithmetic (ggml_vec_dot_q4_0_q8_0, ggml-quants.c:2512-2650; in the reference's
 * CUDA backend the mul_mat_q tiles and dequantize_mul_mat_batch_sparse, ggml-cuda.cu:3524-4308, 4757-4830): one integer matrix-core
 * instruction per pair of a Q4_0 weight block and a Q8_0 activation block gives the exact int32 sum, scaled by d_w * d_x in fp32.
 * pi_k_q4_split writes a Q4_0 matrix [rows][cols / 32] blocks as two arrays, quants (16 bytes per block, the dwords of four consecutive
 * blocks interleaved: [row][block / 4][dword][block % 4]) and scales [rows][cols / 32] fp16 (cols % 256 == 0); pi_k_norm_q8_blocks
 * normalises T <= 16 rows and quantises them as quantize_row_q8_0 does (ggml-quants.c:702-760) into q int8 [T][cols], d float
 * [cols / 32][16] and s8 = -8 * sum(q) int32 [cols / 32][16] (token innermost; cols <= 8192), and, if plain_f16 != NULL, also writes the
 * rows before the norm as fp16 (the predictor's input); pi_k_gemm_q4_t16 is y[t][row] = epilogue(W[row] . x[t]) on those forms; pi_k_batch_sparse_ffn_q4 is
 * pi_k_batch_sparse_ffn on them: the union list from the flags pi_k_batch_predictor_fc2 left in the workspace, up/gate dots of the
 * union rows, h [16][ff] under the predictor's mask, hq = the values h's Q8_0 blocks keep (blocks of 32 consecutive neurons, as the
 * CPU path's axpy reads them, ggml.c:14436-14470), and the down projection over the union rows on fp32 matrix cores.
 * h and hq are caller-provided scratch of 16 * ff floats each. */
PI_API int pi_k_q4_split(const void * W_q4, int rows, int cols, void * quants, void * scales, pi_stream_t stream);
PI_API int pi_k_norm_q8_blocks(const float * x, int T, int cols, const pi_norm * norm, void * q, float * d, int32_t * s8, void * plain_f16, pi_stream_t stream);
/* the same with the fp16 copy of the un-normalised rows in the operand layout of pi_k_gemm_f16_ol (16 token slots) */
PI_API int pi_k_norm_q8_blocks_ol(const float * x, int T, int cols, const pi_norm * norm, void * q, float * d, int32_t * s8, void * plain_ol, pi_stream_t stream);
PI_API int pi_k_gemm_q4_t16(const void * quants, const void * scales, int rows, int cols, const void * xq, const float * xd, const int32_t * xs8, int T,
                            int epilogue, const float * add1, const float * add2, float * y, pi_stream_t stream);
PI_API int pi_k_batch_sparse_ffn_q4(const float * logits, int T, int ff, float threshold, const void * up_quants, const void * up_scales,
                                    const void * gate_quants, const void * gate_scales, const void * down_quants, const void * down_scales, int cols,
                                    const void * xq, const float * xd, const int32_t * xs8, int epilogue, const float * add1, const float * add2, float * out,
                                    float * h, float * hq, int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_ffn_h_f16(const float * up, const float * gate, const float * logits, float threshold, int T, int ff, void * h_f16, pi_stream_t stream);
PI_API int pi_k_transpose_f16(const void * in_f16, int rows, int cols, void * out_f16, pi_stream_t stream);

/* Q4_0 models in prompt chunks.  The CPU path multiplies Q4_0 rows with the Q8_0 form of the activations (ggml_vec_dot_q4_0_q8_0,
 * ggml-quants.c:2512-2650; the down projection quantises h over blocks of 32 neurons, ggml.c:14465-14618).  The chunk path keeps
 * those values and only changes the container: pi_k_norm_q8_round_f16 is pi_k_norm_round_f16 with the normalised row passed through
 * Q8_0 blocks (value q * fp16(amax / 127)) before the fp16 rounding (cols % 32 == 0, cols <= 8192); pi_k_ffn_h_q8_f16 does the same
 * to h (n_ff % 64 == 0); pi_k_dequant_q4_f16 writes a Q4_0 matrix as fp16 ((q - 8) * d), optionally assembling it from the compact
 * matrix of the resident neurons and the matrix of the others (hot_words / hot_prefix as for pi_k_pred_upgate_q4_split).  The
 * products then differ from the CPU path's only by the fp16 rounding of the two factors. */
PI_API int pi_k_norm_q8_round_f16(const float * x, int T, int cols, const pi_norm * norm, void * out_f16, void * out_plain_f16, pi_stream_t stream);
PI_API int pi_k_ffn_h_q8_f16(const float * up, const float * gate, const float * logits, float threshold, int T, int ff, void * h_f16, pi_stream_t stream);
PI_API int pi_k_dequant_q4_f16(const void * W_q4, const void * W_rest_q4, const uint32_t * hot_words, const int32_t * hot_prefix, int rows, int cols,
                               void * out_f16, pi_stream_t stream);
/* the same assembly for an fp16 matrix of a hybrid layer (rows % 32 == 0, cols % 8 == 0), and the embedding rows of a chunk from a Q4_0 table */
PI_API int pi_k_assemble_rows_f16(const void * W_f16, const void * W_rest_f16, const uint32_t * hot_words, const int32_t * hot_prefix, int rows, int cols,
                                  void * out_f16, pi_stream_t stream);
PI_API int pi_k_embed_batch_q4(const void * table_q4, int cols, const int32_t * tokens, int T, float * x, pi_stream_t stream);

/* The whole Q4_0 sparse FFN behind fc1 as one launch plus the reduction, for layers whose active neurons are all computed on the device
 * (every neuron resident: no hot words, no second matrices; or the split of pi_k_pred_upgate_q4_split with the non-resident rows in
 * pinned host memory).  A workgroup's 32 neurons are one Q8_0 block of h, so the launch of pi_k_pred_upgate_q4 goes on with the down rows
 * of its own neurons (arithmetic of pi_k_axpy_q4_partials) and stores one partial output vector per workgroup;
 * pi_k_sparse_ffn_q4_reduce adds the ff / 32 vectors in order plus the residual(s) and counts the active neurons. */
PI_API int pi_k_sparse_ffn_q4_partials(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                                       const void * up_q4, const void * gate_q4, const void * down_t_q4,
                                       const void * up_rest_q4, const void * gate_rest_q4, const void * down_t_rest_q4,
                                       int cols, const float * x, const pi_norm * norm, const uint32_t * hot_words, const int32_t * hot_prefix,
                                       float * logits, float * h_dense, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_sparse_ffn_q4_reduce(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out, int32_t * n_active,
                                     pi_workspace * ws, pi_stream_t stream);
/* Hand-over points between the stream and host threads that compute the non-resident neurons of a hybrid layer (the CPU half of
 * llm_build_sparse_mul_mat / llm_build_sparse_axpy, llama.cpp:4581-4593, 4635-4646) without the host launching anything in between.
 * flags_pinned: 64 words of pinned host memory (words 0 and 8 written by the device, words 16 and 32 by the host, word 48 = the host's
 * stop word); seq: a device word counting the hand-overs; status_pinned: one device or pinned word, non-zero after a wait gave up.
 * pi_k_host_signal: flags[word] = *seq (after *seq += 1 when advance is set) once everything queued before it is complete.  pi_k_host_wait: holds the stream until
 * flags[slot] has reached *seq, for at most limit_seconds (then *status = 1 and every later wait returns at once).
 * pi_k_host_signal_wait: a signal without advance (signal_word 0 or 8; -1 = none) and a wait in one launch. */
PI_API int pi_k_host_signal(uint32_t * seq, uint32_t * flags_pinned, int word, int advance, pi_stream_t stream);
/* pi_k_pred_upgate_q4 cut in two for such a layer, so that the host threads start behind the predictor: pi_k_pred_q4_logits computes the
 * logits (to `logits`, optional, which may be pinned host memory, and to logits_dev), the mask words (bit j of word w = neuron 32 w + j is
 * active; also to words_out, optional, which may be pinned host memory) and the Q8_0 blocks of the normalised input;
 * pi_k_upgate_q4_hot_rows reads logits_dev and writes h (or 0) for the neurons of the hot words only - the other entries of h_dense
 * belong to the host.  With announce_seq / announce_flags (both or neither) the first lane of that launch does what
 * pi_k_host_signal(announce_seq, announce_flags, 0, 1) would have done right before it: the predictor's results are complete and
 * visible to the host at the boundary in front of the launch, so the hand-over needs no launch of its own. */
PI_API int pi_k_pred_q4_logits(const void * fc2_f16, int ff, int r, const float * hidden, float threshold, int cols, const float * x, const pi_norm * norm,
                               float * logits, float * logits_dev, void * xq8_out, uint32_t * words_out, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_upgate_q4_hot_rows(int ff, float threshold, const void * up_q4, const void * gate_q4, int cols, const float * x, const pi_norm * norm,
                                   const uint32_t * hot_words, const int32_t * hot_prefix, const float * logits_dev, float * h_dense,
                                   uint32_t * announce_seq, uint32_t * announce_flags, pi_workspace * ws, pi_stream_t stream);
/* The fused F16 launch of a hybrid layer (pi_k_sparse_ffn_partials_hot) cut in two in the same way (cols 4096): pi_k_sparse_ffn_logits_hot
 * computes the logits (to `logits`, optional, which may be pinned host memory, and to logits_dev), the mask words (also to words_out,
 * optional, as pi_k_pred_q4_logits) and the fp16 normalised input for
 * the host; pi_k_sparse_ffn_rows_hot reads logits_dev and computes the resident active neurons' gate / up / down rows into the partial
 * vectors that pi_k_sparse_ffn_reduce_hot adds; announce_seq / announce_flags as for pi_k_upgate_q4_hot_rows. */
PI_API int pi_k_sparse_ffn_two_phase_supported(int ff, int r, int cols);
PI_API int pi_k_sparse_ffn_logits_hot(const void * fc2_f16, int ff, int r, const float * hidden, float threshold, int cols, const float * x, const pi_norm * norm,
                                      const uint32_t * hot_words, const int32_t * hot_prefix, float * logits, float * logits_dev, void * xn_f16_out,
                                      uint32_t * words_out, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_sparse_ffn_rows_hot(int ff, float threshold, const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols, const float * x,
                                    const pi_norm * norm, const uint32_t * hot_words, const int32_t * hot_prefix, const float * logits_dev, float * h_dense,
                                    uint32_t * announce_seq, uint32_t * announce_flags, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_host_wait(const uint32_t * seq, const uint32_t * flags_pinned, int slot, uint32_t * status_pinned, double limit_seconds, pi_stream_t stream);
PI_API int pi_k_host_signal_wait(const uint32_t * seq, uint32_t * flags_pinned, int signal_word, int slot, uint32_t * status_pinned, double limit_seconds,
                                 pi_stream_t stream);

/* The same mat-mul for prompt chunks of any length through hipBLASLt (fp16 operands, fp32 accumulation and result), where the reference
 * calls cuBLAS (ggml_cuda_op_mul_mat_cublas, ggml-cuda.cu:7662-7756).  Arguments and epilogues as pi_k_gemm_f16; no limit on T or cols.
 * A pi_gemm_lib holds the library handle, its workspace and one plan per distinct (rows, cols, T) - at most 64 of them. */
typedef struct pi_gemm_lib pi_gemm_lib;
PI_API pi_gemm_lib * pi_gemm_lib_create(size_t workspace_bytes);
PI_API int           pi_gemm_lib_destroy(pi_gemm_lib * g);
PI_API int pi_gemm_lib_f16(pi_gemm_lib * g, const void * W_f16, int rows, int cols, const void * xn_f16, int T, int epilogue,
                           const float * add1, const float * add2, float * y, void * y_f16, pi_stream_t stream);

/* The two sparse operators of a step AS OPERATORS, for a host that runs the predictor itself and hands over its output idx [T][ff]
 * (the reference's mul_mat_batch_sparse and axpy at batch size > 1, ggml-cuda.cu:6994-7034, 8787-8814): T <= 16, F16 rows, cols % 256 == 0.
 *   pi_k_batch_sparse_mul_mat: y[t][n] = W[n] . xn_f16[t] where !(idx[t][n] < threshold), 0 elsewhere (y is [T][ff], fully written);
 *   pi_k_batch_sparse_axpy:    out[t] = sum over n with !(idx[t][n] < threshold) of fp16(h[t][n]) * down_t[n][:]   (h is [T][ff], out [T][cols]).
 * Each weight row is read once per step (rows active for at least one token); union_rows [ff] / n_union [1] are scratch the caller owns. */
PI_API int pi_k_batch_sparse_mul_mat(const void * W_f16, int ff, int cols, const void * xn_f16, int T, const float * idx, float threshold,
                                     float * y, int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream);
PI_API int pi_k_batch_sparse_axpy(const void * down_t_f16, int cols, int ff, const float * h, const float * idx, int T, float threshold,
                                  float * out, int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream);

/* pi_k_attn_fused with the cache cells of every head split over n_parts workgroups, for contexts whose K / V rows one workgroup per
 * head cannot pull fast enough (a compute unit sustains about 1/256 of the HBM rate) or whose scores do not fit one workgroup's LDS:
 * part s takes cells [n_kv * s / n_parts, n_kv * (s + 1) / n_parts), keeps (max, sum, weighted V sum) of its cells in `scratch`
 * (pi_k_attn_split_scratch_floats floats), and a second small launch merges the parts in order.  Each part rounds exp() to fp16
 * relative to its own maximum, as the CPU path does relative to the global one (ggml.c:10747-10759), so outputs differ from
 * pi_k_attn_fused in the last places of those roundings.  n_seq sequences as pi_k_attn_fused_batch (1 with strides 0 for one).
 * The reference runs K.q, scale, mask, soft-max and V.p as separate nodes (llm_build_kqv, llama.cpp:4764-4850). */
PI_API int    pi_k_attn_split_supported(int hd, int n_ctx, int n_parts);
PI_API size_t pi_k_attn_split_scratch_floats(int n_seq, int n_head, int hd, int n_parts);
PI_API int    pi_k_attn_split(const float * qkv, int qkv_stride, const void * rope_table, void * k_cache, void * v_cache, size_t cache_seq_stride,
                              int n_seq, int n_head, int n_head_kv, int hd, int mode, int n_ctx, int n_parts, const int32_t * pos, float * scratch,
                              float * out, int out_stride, void * out_f16, pi_stream_t stream);
/* pi_k_attn_chunk (below) for contexts beyond its kernels (pi_k_attn_chunk_supported tells): RoPE + KV store of the chunk's T tokens, then
 * each token's cells split as above (scratch: pi_k_attn_split_scratch_floats(T, ...)).  No K / V tile is shared between the tokens of the
 * chunk, so a long prompt costs T passes over the cache per chunk: it is the path that works at any context, not a fast one. */
PI_API int    pi_k_attn_chunk_supported(int hd, int n_ctx, int n_kv_max);
PI_API int    pi_k_attn_chunk_long(const float * qkv, int qkv_stride, int T, int n_head, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale,
                                   const int32_t * pos, int n_ctx, int n_parts, float * scratch, float * q_rot, void * k_cache, void * v_cache,
                                   float * out, void * out_f16, pi_stream_t stream);
/* the same for tokens whose K / V rows are in the cache already and whose q is rotated (a prompt chunk after pi_k_rope_kv_store):
 * q_rot fp32 [n_tok][n_head * hd], token t attends to cells [0, pos[t]] of the one cache */
PI_API int    pi_k_attn_split_cached(const float * q_rot, const void * k_cache, const void * v_cache, int n_tok, int n_head, int n_head_kv, int hd,
                                     int n_ctx, int n_parts, const int32_t * pos, float * scratch, float * out, pi_stream_t stream);

/* One token's attention on the reference's own cache layouts, for the ggml_cuda_* boundary: what llm_build_kv_store and llm_build_kqv
 * (llama.cpp:4383-4418, 4764-4850) build from two ROPE, two CPY, K.q, SCALE, ADD(mask), SOFT_MAX, V.p and CONT nodes, in one launch.
 * q [n_head * hd], k, v [n_head_kv * hd]: the token's projections before RoPE (fp32); pos: its position (device, one int32);
 * k_cache: the layer's cells [n_kv][n_head_kv * hd] fp16; v_cache: the layer's transposed values [n_head_kv * hd][n_ctx] fp16;
 * cell: where the token's rows are stored (< n_kv); kq_scale: one float; kq_mask: n_kv floats added to the scaled scores (-inf hides a
 * cell); out fp32 [n_head * hd].  mode 0 / 2 and theta_scale, freq_scale, mscale as the ROPE node carries them (no YaRN mixing). */
PI_API int pi_k_attn_ggml_supported(int hd, int n_ctx, int n_kv);
PI_API int pi_k_attn_ggml(const float * q, const float * k, const float * v, const int32_t * pos, int mode, float theta_scale, float freq_scale, float mscale,
                          void * k_cache, void * v_cache, int n_head, int n_head_kv, int hd, int n_ctx, int n_kv, int cell,
                          const float * kq_scale, const float * kq_mask, float * out, pi_stream_t stream);
/* the same for a step of T <= 16 tokens whose rows go to the consecutive cells cell0 .. cell0 + T - 1 (the run llama_kv_cache_find_slot
 * returns): token u's projections at qkv + u * qkv_stride ([q | k | v]), its position pos[u], its mask row at kq_mask + u * mask_stride,
 * its result at out + u * out_stride.  Every token sees the step's other new cells where its mask row allows, as if the whole batch
 * had been stored first (llm_build_kv_store runs ahead of llm_build_kqv, llama.cpp:4383-4418, 4764-4850). */
PI_API int pi_k_attn_ggml_step(const float * qkv, int qkv_stride, const int32_t * pos, int mode, float theta_scale, float freq_scale, float mscale,
                               void * k_cache, void * v_cache, int n_head, int n_head_kv, int hd, int n_ctx, int n_kv, int T, int cell0,
                               const float * kq_scale, const float * kq_mask, int mask_stride, float * out, int out_stride, pi_stream_t stream);

/* per-sequence pieces of a batched step: sequence t owns token t, position pos[t] and the cache at t * cache_seq_stride
 * (elements), out_f16 (optional) receives fp16(out); pi_k_argmax_batch picks each sequence's next token (first maximum wins), stores it in tokens[t], adds 1 to
 * positions[t] and records it at out_tokens[*step][t]; pi_k_step_advance then moves *step on. */
PI_API int pi_k_attn_fused_batch(const float * qkv, int qkv_stride, const void * rope_table, void * k_cache, void * v_cache,
                                 size_t cache_seq_stride, int n_seq, int n_head, int n_head_kv, int hd, int mode, int n_ctx,
                                 const int32_t * pos, float * out, int out_stride, void * out_f16, pi_stream_t stream);
/* the same for a Q4_0 output projection: instead of an fp16 copy, the output as the Q8_0 blocks pi_k_gemm_q4_t16 multiplies with (what
 * pi_k_norm_q8_blocks without a norm makes of `out`, bit for bit: blocks in the MFMA operand layout, scales and -8 * sums as [block][16]);
 * head size % 32 == 0 */
PI_API int pi_k_attn_fused_batch_q8(const float * qkv, int qkv_stride, const void * rope_table, void * k_cache, void * v_cache,
                                    size_t cache_seq_stride, int n_seq, int n_head, int n_head_kv, int hd, int mode, int n_ctx,
                                    const int32_t * pos, float * out, int out_stride, void * q8_quants, float * q8_scales, int32_t * q8_sums,
                                    pi_stream_t stream);
/* the same with the fp16 copy in the operand layout of pi_k_gemm_f16_ol (16 sequence slots of n_head * hd columns; out stays [n_seq][out_stride]) */
PI_API int pi_k_attn_fused_batch_ol(const float * qkv, int qkv_stride, const void * rope_table, void * k_cache, void * v_cache,
                                    size_t cache_seq_stride, int n_seq, int n_head, int n_head_kv, int hd, int mode, int n_ctx,
                                    const int32_t * pos, float * out, int out_stride, void * out_ol, pi_stream_t stream);
/* prompt chunk of ONE sequence: T <= 512 consecutive tokens at positions pos[t]; RoPE + KV store of the whole chunk first, then
 * every token attends to the cells up to its own position (the causal mask of llama.cpp:6506-6531).  q_rot: fp32 [T][n_head*hd].
 * n_kv_max: an upper bound of max(pos) + 1, the cells the chunk's furthest token attends (<= 0: n_ctx); positions beyond it are
 * clamped.  Head sizes 128 and 64 with 16 * n_kv_max floats of scores within 156 KB of LDS (about 1850 cells, whatever the cache's
 * n_ctx) take 16 tokens per workgroup on the matrix cores; other shapes one token per workgroup (n_ctx up to about 11 k).  Same
 * rounding points either way (llm_build_kqv on the CPU path: fp16 q and K, fp16 in and out of exp, fp16 probabilities). */
PI_API int pi_k_attn_chunk(const float * qkv, int qkv_stride, int T, int n_head, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale,
                           const int32_t * pos, int n_ctx, int n_kv_max, float * q_rot, void * k_cache, void * v_cache,
                           float * out, int out_stride, void * out_f16, pi_stream_t stream);
PI_API int pi_k_embed_batch(const void * table_f16, int cols, const int32_t * tokens, int T, float * x, pi_stream_t stream);
PI_API int pi_k_argmax_batch(const float * logits, int n, int T, int32_t * tokens, int32_t * positions, int32_t * step,
                             int32_t * out_tokens, int max_steps, pi_stream_t stream);
PI_API int pi_k_step_advance(int32_t * step, pi_stream_t stream);

/*
 * RoPE on q and k of one token plus the KV-cache store (rope / rope_neox ggml-cuda.cu:4999,5027 and
 * cpy_f32_f16 :4944 for llm_build_kv_store, llama.cpp:4383).  qkv: fp32 [n_head*hd + 2*n_head_kv*hd]
 * (q | k | v).  mode 0 = adjacent pairs, 2 = NeoX halves.  The position is read from *pos (device).
 * Cache layout (this library's own): K and V are fp16 [n_head_kv][n_ctx][hd].
 * theta_scale = freq_base^(-2/hd); freq_scale = linear RoPE scaling (llama_context_params.rope_freq_scale, 1 = none): the angle
 * of a pair is freq_scale * theta as rope_yarn forms it with ext_factor 0 (ggml.c:11124-11146), and mode 2 multiplies the
 * starting angle by freq_scale once more as the CPU path does (ggml.c:11292).
 */
PI_API int pi_k_rope_kv_store(const float * qkv, int n_head, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale,
                              const int32_t * pos, int n_ctx, float * q_rot, void * k_cache, void * v_cache, pi_stream_t stream);

/*
 * Single-token attention over cells [0, *pos] of the cache (KQ, scale, softmax, KQV; replaces the
 * batched hipBLAS GEMMs + soft_max_f32 the reference runs at batch 1, ggml-cuda.cu:8564-8712, 5135).
 * Probabilities go through the same fp16 exp rounding as the CPU path (ggml.c:10747-10759).
 * out: fp32 [n_head*hd].
 */
PI_API int pi_k_attn_decode(const float * q_rot, const void * k_cache, const void * v_cache, int n_head, int n_head_kv,
                            int hd, int n_ctx, const int32_t * pos, float * out, pi_stream_t stream);

/* cos/sin table for pi_k_attn_fused: float2 [n_ctx][hd/2], angles formed as the CPU path forms them
 * (theta advanced by repeated fp32 multiplication with theta_scale = base^(-2/hd), ggml.c:11196-11319; mode and freq_scale as in
 * pi_k_rope_kv_store).  A set-up call: the
 * values are computed on the host with the C library's cosf / sinf (what the CPU path calls) and copied with a blocking copy
 * after the stream has drained. */
PI_API int pi_k_rope_table(void * table, int n_ctx, int hd, int mode, float theta_scale, float freq_scale, pi_stream_t stream);

/* pi_k_rope_kv_store + pi_k_attn_decode in one launch (one workgroup per query head; the new cell is used
 * from LDS and stored by the first query head of each KV group).  Same arithmetic, same cache layout. */
PI_API int pi_k_attn_fused(const float * qkv, const void * rope_table, void * k_cache, void * v_cache, int n_head, int n_head_kv,
                           int hd, int mode, int n_ctx, const int32_t * pos, float * out, pi_stream_t stream);

/* 1 if the single-pass attention kernels cover the head size and context (they keep the scores of every cell in LDS: at head
 * size 128 pi_k_attn_fused reaches n_ctx 6784 and pi_k_attn_decode 13312).  pi_model_finalize picks the fused kernel where it
 * fits and the rope_kv_store + attn_decode pair otherwise; batched decoding needs the fused one. */
PI_API int pi_k_attn_fused_supported(int hd, int n_ctx);
PI_API int pi_k_attn_decode_supported(int hd, int n_ctx);

/* x[cols] = row *token of the embedding table (k_get_rows, ggml-cuda.cu:1664) */
PI_API int pi_k_embed(int wtype, const void * table, int cols, const int32_t * token, float * x, pi_stream_t stream);

/* greedy sampling: *token_out = index of the first maximum (llama_sample_token_greedy, llama.cpp:8617-8631) */
PI_API int pi_k_argmax(const float * logits, int n, int32_t * token_out, pi_stream_t stream);

/* ---- decode loop with resident weights ------------------------------------------------------------- */

enum { PI_ARCH_LLAMA = 0, PI_ARCH_FALCON = 1 };

/* the llama_hparams fields this path reads (llama.cpp:1207-1270) */
typedef struct pi_hparams {
    int32_t arch;
    int32_t n_embd, n_ff, n_head, n_head_kv, n_layer, n_vocab, n_ctx;
    float   norm_eps, rope_freq_base, sparse_threshold;
    float   rope_freq_scale;            /* linear RoPE scaling (llama_cparams.rope_freq_scale, llama.cpp:9857); 0 is read as 1 */
} pi_hparams;

/* tensor roles; names as llama.cpp:403-461 (blk.N.<role>.weight).  layer = -1 for the global ones. */
enum {
    PI_T_TOK_EMBD = 0, PI_T_OUTPUT_NORM, PI_T_OUTPUT_NORM_B, PI_T_OUTPUT,
    PI_T_ATTN_NORM, PI_T_ATTN_NORM_B, PI_T_ATTN_NORM_2, PI_T_ATTN_NORM_2_B,
    PI_T_WQ, PI_T_WK, PI_T_WV, PI_T_WQKV, PI_T_WO,
    PI_T_FFN_NORM, PI_T_FFN_GATE, PI_T_FFN_UP, PI_T_FFN_DOWN_T,
    PI_T_FC1, PI_T_FC2, PI_T_GPU_IDX, PI_T_GPU_BUCKET,
    PI_T_NEURON_RATE,
    PI_T_COUNT
};

/* The ggml_cuda_* boundary (include/ggml_backend_abi.h) keeps single-token nodes in a window until it knows whether they form a block
 * it computes in one launch: llm_build_ffn_sparse's sequence (llama.cpp:4652-4757), with every neuron on the device, becomes pi_k_gemv +
 * pi_k_sparse_ffn when its AXPY node arrives.  These two calls are not part of the reference's interface: the counters tell a test or
 * a profile what the window did, the switch turns it off at run time (GGML_CUDA_NO_FUSION=1 in the environment does so from the start). */
typedef struct pi_ggml_backend_stats { int64_t nodes_deferred, windows_flushed, ffn_blocks_fused, attn_blocks_fused; } pi_ggml_backend_stats;
PI_API void pi_ggml_backend_get_stats(pi_ggml_backend_stats * out);
PI_API void pi_ggml_backend_set_fusion(int enable);

typedef struct pi_model pi_model;

/* llama_load_model_from_file + llama_new_context_with_model (llama.cpp:9789, 9819) without the file
 * format: the caller hands over tensors one by one. */
PI_API pi_model * pi_model_create(const pi_hparams * hp);
PI_API void       pi_model_free(pi_model * m);

/*
 * Give the model one tensor.  `data` is a host pointer (copied to HBM) or, with on_device != 0, a device
 * pointer the model adopts without copying (the caller keeps ownership).  ne0 = contiguous dimension,
 * ne1 = rows.  wq/wk/wv are packed into one [n_embd + 2*n_embd_gqa][n_embd] matrix at finalize.
 * FFN matrices of a layer that has a PI_T_GPU_BUCKET are given FULL-SIZE on the host: the bucket's rows are
 * sliced into compact device matrices (slice_ffn_mat_to_gpu, llama.cpp:2898-2967) and the host copy is
 * kept (borrowed, must outlive the model) for the cold neurons that run on the CPU.
 * PI_T_NEURON_RATE (optional, host, F32 [n_ff], copied): each neuron's firing rate, the activation statistics the reference's offline
 * solver places neurons with (powerinfer-py/powerinfer/solver.py:8-100, export_split.py:24-52).  For an F16 layer that is whole on
 * the device and that the fused kernel covers, pi_model_finalize then deals the neurons out by rate over the 32-neuron groups of that
 * kernel (group g, slot j holds the neuron of rank j * n_ff / 32 + g; fc2 / gate / up / down_t rows are moved alike into storage the
 * model owns) so that every workgroup of that kernel carries the same expected number of active rows.  Results are those of the file
 * order up to the order of the fp32 sums over neurons; everything the model reports per neuron (pi_model_get_capture) stays in file
 * order.
 */
PI_API int pi_model_set_tensor(pi_model * m, int layer, int kind, int type, const void * data,
                               int64_t ne0, int64_t ne1, int on_device);
PI_API int pi_model_finalize(pi_model * m);
PI_API int pi_model_kv_clear(pi_model * m);                    /* llama_kv_cache_clear, llama.h:367 */
/*
 * llama_kv_cache_seq_rm / llama_kv_cache_seq_shift for the model's own sequence (llama.cpp:1757-1785, 1819-1848; p1 < 0 means
 * "to the end").  Removed cells are squeezed out at once and shifted cells get their K rows rotated at once (the reference marks
 * the cells and applies the rotation inside the next llama_decode, llama.cpp:5494-5500).  Decoding needs the cells' positions to
 * be 0 .. n-1 again (what the context shift of examples/main does: remove [keep, keep+discard), shift the rest by -discard);
 * pi_model_decode / pi_model_generate report PI_E_STATE while a gap is open.  After an edit that leaves contiguous positions the
 * next position is n (pi_model_generate continues there; pi_model_decode takes n_past = n).  Both return n or a negative error.
 */
PI_API int pi_model_kv_seq_rm(pi_model * m, int p0, int p1);
PI_API int pi_model_kv_seq_shift(pi_model * m, int p0, int p1, int delta);

/*
 * llama_decode (llama.cpp:10672) for one sequence: evaluates tokens[0..n_tokens) at positions
 * n_past..n_past+n_tokens-1, stores K/V, and leaves the logits of the last token on the device.
 * logits_out (optional, host, fp32 [n_vocab]) receives them (llama_get_logits).
 * Returns the greedy token of the last position (llama_sample_token_greedy) or a negative error.
 */
PI_API int pi_model_decode(pi_model * m, const int32_t * tokens, int n_tokens, int n_past, float * logits_out);

/*
 * The batch-1 greedy token loop of examples/main (main.cpp:462-623 with temp == 0): continues from the
 * state pi_model_decode left (next token = its greedy choice), generates n_steps tokens entirely on the
 * device (one captured HIP graph replayed per token) and writes them to out_tokens (host).
 * ms_out (optional) receives the device time of the loop measured with events on the model's stream.
 */
PI_API int pi_model_generate(pi_model * m, int n_steps, int32_t * out_tokens, float * ms_out);

/* parity hooks: when enabled, pi_model_decode also records, for its LAST token, each layer's FFN output
 * [n_layer][n_embd] (before the residual add), predictor logits [n_layer][n_ff], active-row count [n_layer]
 * and the vector the FFN block read [n_layer][n_embd] (LLaMA: ffn_inp; Falcon: the layer input; both before
 * the norm; it is also the predictor's input).  Any output pointer may be NULL. */
/*
 * Batched greedy decoding: n_seq <= 16 independent sequences advance one token per step (examples/batched/batched.cpp:100-260).
 * F16 models, or Q4_0 models with F16 predictors, with every neuron on the GPU (Q4_0: integer matrix-core kernels on the Q4_0 x Q8_0
 * blocks, pi_k_gemm_q4_t16 / pi_k_batch_sparse_ffn_q4, from a split copy of the quants made at pi_model_batch_init).
 * pi_model_batch_init allocates one KV cache per sequence and the step buffers;
 * pi_model_batch_decode feeds tokens[t] of sequence t at positions[t] and returns each sequence's greedy next token (and,
 * if logits_out != NULL, the [n_seq][n_vocab] logits); pi_model_batch_generate continues greedily from that state for
 * n_steps steps and returns out_tokens[n_steps][n_seq].
 */
PI_API int pi_model_batch_init(pi_model * m, int n_seq);
PI_API int pi_model_batch_decode(pi_model * m, const int32_t * tokens, const int32_t * positions, int32_t * next_tokens, float * logits_out);
PI_API int pi_model_batch_generate(pi_model * m, int n_steps, int32_t * out_tokens, float * ms_out);
/* llama_kv_cache_seq_rm / _seq_shift / _seq_cp (llama.cpp:1757-1848) for sequence `seq` of the batch, with the semantics of
 * pi_model_kv_seq_rm / _shift.  Sequences own their caches, so _cp copies cells [p0, p1) of src into dst, which must hold exactly
 * p0 cells (a prompt prefix evaluated once and handed to the other sequences); returns dst's cell count. */
PI_API int pi_model_batch_kv_seq_rm(pi_model * m, int seq, int p0, int p1);
PI_API int pi_model_batch_kv_seq_shift(pi_model * m, int seq, int p0, int p1, int delta);
PI_API int pi_model_batch_kv_seq_cp(pi_model * m, int src, int dst, int p0, int p1);
/* One KV cache whose cells are shared between sequences: llama_kv_cell / llama_kv_cache (llama.cpp:1381-1420), llama_kv_cache_find_slot (:1683-1730),
 * _seq_rm / _seq_cp / _seq_keep / _seq_shift / _clear (:1745-1848), the visibility mask of llama_decode (:6506-6531) and the cell range a step looks
 * at (:1735-1743, 6842).  A cell holds a position and a set of sequence ids (0..31, one bit each); a step of up to 16 tokens takes a run
 * of free cells found from the ring's head, every token attends the cells of its (first) sequence at positions not beyond its own;
 * _seq_cp makes the cells of src visible to dst without copying anything (a prompt evaluated once serves every continuation).
 * F16 models, or Q4_0 models with F16 predictors, with every neuron on the GPU; n_cells a multiple of 32.  _decode returns PI_E_STATE when no run of free cells is left (the reference's
 * llama_decode returns 1), each token's greedy next token and, if logits_out != NULL, its logits [n_tokens][n_vocab].
 * _state copies the cells' positions (-1: free) and sequence bit sets and the ring's head out (tests, monitoring); returns n_cells.
 * _seq_shift moves the positions of a sequence's cells in [p0, p1) by delta (llama_kv_cache_seq_shift, :1824-1848; a cell whose position
 * falls below 0 is freed); the K rows are rotated at the start of the next step (llm_build_k_shift, :4332-4381), after which the pending
 * deltas are cleared (:6925-6932). */
PI_API int pi_model_kv_cells_init(pi_model * m, int n_cells);
PI_API int pi_model_kv_cells_decode(pi_model * m, const int32_t * tokens, const int32_t * positions, const uint32_t * seq_masks, int n_tokens,
                                    int32_t * next_tokens, float * logits_out);
PI_API int pi_model_kv_cells_seq_rm(pi_model * m, int seq, int p0, int p1);
PI_API int pi_model_kv_cells_seq_cp(pi_model * m, int src, int dst, int p0, int p1);
PI_API int pi_model_kv_cells_seq_keep(pi_model * m, int seq);
PI_API int pi_model_kv_cells_seq_shift(pi_model * m, int seq, int p0, int p1, int delta);
PI_API int pi_model_kv_cells_clear(pi_model * m);
PI_API int pi_model_kv_cells_state(pi_model * m, int32_t * cell_pos, uint32_t * cell_seq, int32_t * head);
PI_API int pi_model_batch_union(pi_model * m, int32_t * n_union_per_layer);   /* union sizes of the last step, [n_layer] */
/* Dense cross-over of lockstep decoding (the reference leaves its batch-sparse kernels for a plain mat-mul when a step has many
 * tokens, ggml-cuda.cu:8787-8814, 7717-7756; here the switch is the union of the sequences' active rows): a layer whose union in the
 * last step exceeded fraction * n_ff computes its FFN in the next step as dense gate / up mat-muls, h with the predictor's mask, and a
 * dense down mat-mul (one more copy of that layer's down projection with the neurons contiguous, made on first use).  <= 0: always
 * dense, >= 1: never, which is the default: on the 13B shape with 16 sequences the union kernels are the faster ones at every union
 * fraction measured (5.59 against 7.61 ms per step at 0.41 of n_ff, 7.55 against 7.77 at 0.99).
 * pi_model_batch_dense_layers: how many layers the next step runs dense. */
PI_API int pi_model_batch_set_dense_above(pi_model * m, float fraction);
PI_API int pi_model_batch_dense_layers(pi_model * m);

/* Before pi_model_finalize: layers with a gpu_bucket keep their non-resident rows in pinned host memory and the GPU reads the
 * rows of active neurons from there itself (pi_k_pred_upgate_q4_split) instead of handing those neurons to host threads; the
 * token loop then needs no host step and replays as a HIP graph.  Q4_0 layers at n_embd 4096; the VRAM split is unchanged. */
PI_API int pi_model_set_rest_on_gpu(pi_model * m, int enable);
PI_API int pi_model_set_capture(pi_model * m, int enable);
PI_API int pi_model_get_capture(pi_model * m, float * ffn_out, float * pred_logits, int32_t * n_active, float * ffn_src);

/*
 * Event-timed replay of one section of the token loop on the model's stream, `rounds` passes over all layers,
 * on the activations the last token left behind (the per-node timers of GGML_PERF, ggml.c:16604-16619, are the
 * nearest thing in the reference).  section 0: the q|k|v projection mat-vec of every layer (the kernel that
 * moves the most bytes per token); 1: the sparse FFN block of every layer (fc1, fc2+compaction, up/gate, axpy);
 * 2: the lm-head mat-vec; 3: the fused predictor + gate/up/down kernel of every layer alone (F16 models the fused block
 * covers); 4: the reduction of its partial vectors alone.  ms_total: device milliseconds for everything issued; launches: number of
 * section instances issued (rounds * n_layer, or rounds for the lm-head).
 */
PI_API int pi_model_time_section(pi_model * m, int section, int rounds, float * ms_total, int * launches);

/* for each of the n_steps tokens of the most recent pi_model_generate: the sum over layers of the active-row
 * counts (feeds the touched-bytes accounting of the benchmark) */
PI_API int pi_model_step_active(pi_model * m, int32_t * per_step_total, int n_steps);

#ifdef __cplusplus
}
#endif
#endif

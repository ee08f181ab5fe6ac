// Batched greedy decoding on top of the single-sequence engine's weights: n_seq <= 16 independent sequences advance one
// token per step (what examples/batched/batched.cpp:100-260 drives through llama_decode with n_tokens = n_parallel).
// Per layer: activations are normalised + rounded to fp16 once per mat-mul input, dense mat-muls and the sparse gate/up
// run on the matrix cores, every weight row of the union of the sequences' active sets is read once per step.
#include "engine_internal.hpp"
#include "runtime.hpp"

#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <algorithm>
#include <unordered_map>
#include <string.h>

struct BatchState {
    int n_seq = 0, max_steps = 4096;
    int kv_hi = 0;                        // prompt chunks: cells the chunk's last token attends (its position + 1)
    // lockstep decoding: layers whose union of active rows was above dense_above * n_ff in the last step run their FFN dense
    // (>= 1: never, the default: the union kernels are the faster ones at every union fraction measured, see batch_layer)
    std::vector<char> dense_ffn, graph_dense;
    float dense_above = 1.0f;
    bool prefill = false;                 // prompt chunks of the model's own sequence: tokens share the model's KV cache
    float * q_rot = nullptr;
    size_t cache_seq_stride = 0;          // elements per sequence: n_layer * n_head_kv * n_ctx * hd
    __half *k_cache = nullptr, *v_cache = nullptr;
    float *x = nullptr, *x2 = nullptr, *qkv = nullptr, *att = nullptr, *attn_out = nullptr, *ffn_inp = nullptr, *hidden = nullptr;
    float *pred_logits = nullptr, *logits = nullptr;
    __half *xa16 = nullptr, *xf16 = nullptr, *xp16 = nullptr, *att16 = nullptr, *hid16 = nullptr;
    int32_t *d_tokens = nullptr, *d_pos = nullptr, *d_step = nullptr, *d_out_tokens = nullptr, *union_rows = nullptr, *n_union = nullptr;
    float *up_out = nullptr, *gate_out = nullptr;      // wide prompt chunks: dense gate/up products [T][n_ff]
    __half *h16 = nullptr;                             //                     and the FFN's hidden vector
    // One KV cache whose cells are shared between sequences (llama_kv_cache, llama.cpp:1683-1848): a cell holds a position and a set of
    // sequence ids; K cells [n_layer][n_cells][n_embd_gqa] and transposed values [n_layer][n_embd_gqa][n_cells] as the reference lays them
    // out.  Host side: the cells' positions (-1: free), sequence sets (bit s) and the ring's search start.
    bool unified = false;
    int n_cells = 0, head = 0, n_kv = 0;
    std::vector<int32_t> cell_pos;
    std::vector<uint32_t> cell_seq;
    std::vector<int32_t> cell_delta;                   // position shifts not yet applied to the K rows
    bool has_shift = false;
    int32_t * d_delta = nullptr;
    __half *cells_k = nullptr, *cells_v = nullptr;
    float *cells_mask = nullptr, *kq_scale = nullptr;  // device: [16][n_cells] mask rows of a step, 1 / sqrt(head size)
    int slot[16] = {0};                                // the cells the step's tokens were given
    // steps of a Q4_0 model on integer matrix cores: Q8_0 blocks of the attention-side and of the FFN-side mat-mul input (int8 quants
    // [16][n_embd], scales and 8 * sums [n_embd / 32][16]), h and the values its Q8_0 blocks keep [16][n_ff]
    void *qa = nullptr, *qf = nullptr; float *da = nullptr, *df = nullptr; int32_t *sa = nullptr, *sf = nullptr;
    float *h32 = nullptr, *hq32 = nullptr;
    __half *w16 = nullptr, *w16t = nullptr;            // wide prompt chunks of Q4_0 / hybrid layers: one matrix as fp16, and the down projection with the neurons contiguous
    // hybrid layers in wide prompt chunks: the non-resident rows of the next layer travel from pinned host memory into one of two device
    // staging buffers on a copy stream while this layer computes (up | gate | down, each n_rest rows)
    unsigned char * stage[2] = {nullptr, nullptr};
    size_t stage_rows = 0, stage_row_bytes = 0;
    hipStream_t copy_stream = nullptr;
    hipEvent_t ev_copied[2] = {nullptr, nullptr}, ev_free[2] = {nullptr, nullptr};
    bool free_recorded[2] = {false, false};
    int staged_layer[2] = {-1, -1};
    hipGraphExec_t graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    std::vector<std::vector<int32_t>> kv_pos;      // per sequence: cell positions while an edit left them non-contiguous
};

namespace {

#define PI_TRY(expr) do { int _rc = (expr); if (_rc != PI_OK) return _rc; } while (0)

pi_norm mk_norm(int kind, float eps, const Tensor & w, const Tensor * b) {
    pi_norm n{kind, eps, (const float *)w.dev, b ? (const float *)b->dev : nullptr};
    return n;
}

// attention of a prompt chunk of the model's own sequence: the chunk kernels where the context fits them, the split-over-cells path beyond
int chunk_attention(pi_model * m, BatchState * b, int T, size_t kv_off) {
    const pi_hparams & hp = m->hp;
    const int d = hp.n_embd, hd = m->hd, gqa = m->gqa, mode = hp.arch == PI_ARCH_FALCON ? 2 : 0;
    if (pi_k_attn_chunk_supported(hd, hp.n_ctx, b->kv_hi))
        return pi_k_attn_chunk(b->qkv, d + 2 * gqa, T, hp.n_head, hp.n_head_kv, hd, mode, m->theta_scale, m->freq_scale, b->d_pos, hp.n_ctx, b->kv_hi, b->q_rot,
                               m->k_cache + kv_off, m->v_cache + kv_off, b->att, d, b->att16, m->stream);
    const int parts = m->attn_parts > 1 ? m->attn_parts : 2;
    if (!m->attn_scratch_chunk) {
        m->attn_scratch_chunk = m->alloc<float>(pi_k_attn_split_scratch_floats(512, hp.n_head, hd, parts));
        if (!m->attn_scratch_chunk) return PI_E_HIP;
    }
    return pi_k_attn_chunk_long(b->qkv, d + 2 * gqa, T, hp.n_head, hp.n_head_kv, hd, mode, m->theta_scale, m->freq_scale, b->d_pos, hp.n_ctx, parts,
                                m->attn_scratch_chunk, b->q_rot, m->k_cache + kv_off, m->v_cache + kv_off, b->att, b->att16, m->stream);
}

// fp16 mat-mul input for a matrix of the given type: rounded to fp16, for a Q4_0 matrix through Q8_0 blocks first (the CPU path
// multiplies Q4_0 rows with the Q8_0 form of the activations)
int batch_input(int wtype, const float * x, int T, int cols, const pi_norm * norm, void * out16, void * plain16, hipStream_t st) {
    if (wtype == PI_TYPE_Q4_0) return pi_k_norm_q8_round_f16(x, T, cols, norm, out16, plain16, st);
    return pi_k_norm_round_f16(x, T, cols, norm, out16, plain16, st);
}

// attention of a step whose tokens live in the shared-cell cache: token t's K / V rows go to cell slot[0] + t, and it attends the cells
// its mask row leaves visible (same sequence, position not beyond its own: llama.cpp:6506-6531), the step's other new cells included
int cells_attention(pi_model * m, BatchState * b, int il, int T) {
    const pi_hparams & hp = m->hp;
    const int d = hp.n_embd, gqa = m->gqa;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    __half * k = b->cells_k + (size_t)il * b->n_cells * gqa;
    __half * v = b->cells_v + (size_t)il * gqa * b->n_cells;
    PI_TRY(pi_k_attn_ggml_step(b->qkv, d + 2 * gqa, b->d_pos, falcon ? 2 : 0, m->theta_scale, m->freq_scale, 1.0f, k, v, hp.n_head, hp.n_head_kv, m->hd,
                               b->n_cells, b->n_kv, T, b->slot[0], b->kq_scale, b->cells_mask, b->n_cells, b->att, d, m->stream));
    const pi_norm plain{0, 0.0f, nullptr, nullptr};
    return pi_k_norm_round_f16(b->att, T, d, &plain, b->att16, nullptr, m->stream);
}

// why the model's multi-token steps cannot run on the integer matrix-core kernels, or null
const char * q4_steps_unsupported(pi_model * m) {
    const pi_hparams & hp = m->hp;
    if (m->hybrid || m->capture) return "hybrid models and capture hooks follow single tokens";
    if (hp.n_embd % 512 || hp.n_embd > 8192 || hp.n_ff % 32 || (int)m->L(0, PI_T_FC1).ne1 % 128) return "n_embd % 512 == 0, n_embd <= 8192, n_ff % 32 == 0 and predictor rank % 128 == 0 required";
    for (int il = 0; il < hp.n_layer; ++il) {
        for (int k : {PI_T_WQKV, PI_T_WO, PI_T_FFN_UP, PI_T_FFN_GATE, PI_T_FFN_DOWN_T}) {
            if (k == PI_T_FFN_GATE && hp.arch == PI_ARCH_FALCON) continue;
            if (m->L(il, k).type != PI_TYPE_Q4_0) return "every attention and FFN matrix must be Q4_0";
        }
        if (m->L(il, PI_T_FC1).type != PI_TYPE_F16 || m->L(il, PI_T_FC2).type != PI_TYPE_F16) return "predictors must be F16";
    }
    const int te = m->glob[PI_T_TOK_EMBD].type, to = m->glob[PI_T_OUTPUT].type;
    if ((te != PI_TYPE_F16 && te != PI_TYPE_Q4_0) || (to != PI_TYPE_F16 && to != PI_TYPE_Q4_0)) return "embedding and output matrix must be F16 or Q4_0";
    return nullptr;
}

// the split form of every Q4_0 matrix the steps multiply with, made once
int ensure_q4_split(pi_model * m) {
    if (m->q4_steps) return PI_OK;
    auto split = [&](Tensor & t) -> int {
        if (t.type != PI_TYPE_Q4_0 || !t.dev || m->q4_split.count(&t)) return PI_OK;
        const size_t nb = (size_t)t.ne1 * (t.ne0 / 32);
        unsigned char * q = m->alloc<unsigned char>(nb * 16);
        __half * d = m->alloc<__half>(nb);
        if (!q || !d) return PI_E_HIP;
        PI_TRY(pi_k_q4_split(t.dev, (int)t.ne1, (int)t.ne0, q, d, m->stream));
        m->q4_split[&t] = pi_model::Q4Split{q, d};
        return PI_OK;
    };
    PI_TRY(split(m->glob[PI_T_OUTPUT]));
    for (int il = 0; il < m->hp.n_layer; ++il)
        for (int k : {PI_T_WQKV, PI_T_WO, PI_T_FFN_UP, PI_T_FFN_GATE, PI_T_FFN_DOWN_T}) PI_TRY(split(m->L(il, k)));
    m->q4_steps = true;
    return PI_OK;
}

int chunk_attention(pi_model * m, BatchState * b, int T, size_t kv_off);

// One layer of a step of up to 16 tokens of a Q4_0 model: the mat-muls of the Q4_0 matrices on integer matrix cores against the
// Q8_0 blocks of their inputs (the CPU path's arithmetic), the F16 predictor as in an F16 model.
int batch_layer_q4(pi_model * m, BatchState * b, int il) {
    const pi_hparams & hp = m->hp;
    const int T = b->n_seq, d = hp.n_embd, ff = hp.n_ff, hd = m->hd, gqa = m->gqa;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    hipStream_t st = m->stream;
    auto W = [&](int kind) { return m->q4_split.at(&m->L(il, kind)); };
    Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
    const int r = (int)fc1.ne1;
    const size_t kv_off = (size_t)il * hp.n_head_kv * hp.n_ctx * hd;
    float * x = b->x;
    const pi_norm plain{0, 0.0f, nullptr, nullptr};
    pi_norm an;
    if (!falcon) an = mk_norm(1, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), nullptr);
    else if (m->L(il, PI_T_ATTN_NORM_2).dev) an = mk_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM_2), &m->L(il, PI_T_ATTN_NORM_2_B));
    else an = mk_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B));
    // (the predictor's fp16 inputs, xp16 and hid16, are kept in the operand layout of the 16-token fp16 mat-muls)
    PI_TRY(pi_k_norm_q8_blocks_ol(x, T, d, &an, b->qa, b->da, b->sa, falcon ? b->xp16 : nullptr, st));   // Falcon: the predictor reads the layer input as plain fp16
    if (falcon) {
        // the FFN branch reads the layer input too, under its own norm (with a single norm: the attention's)
        pi_norm fn = mk_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B));
        PI_TRY(pi_k_norm_q8_blocks(x, T, d, m->L(il, PI_T_ATTN_NORM_2).dev ? &fn : &an, b->qf, b->df, b->sf, nullptr, st));
    }
    const auto wqkv = W(PI_T_WQKV), wo = W(PI_T_WO);
    PI_TRY(pi_k_gemm_q4_t16(wqkv.quants, wqkv.scales, d + 2 * gqa, d, b->qa, b->da, b->sa, T, PI_EPI_NONE, nullptr, nullptr, b->qkv, st));
    if (b->unified)
        PI_TRY(cells_attention(m, b, il, T));
    else if (b->prefill)
        PI_TRY(chunk_attention(m, b, T, kv_off));
    else if (hd % 32 == 0)                                         // lockstep: the attention writes the Q8_0 blocks of its output itself
        PI_TRY(pi_k_attn_fused_batch_q8(b->qkv, d + 2 * gqa, m->rope_table, b->k_cache + kv_off, b->v_cache + kv_off, b->cache_seq_stride, T,
                                        hp.n_head, hp.n_head_kv, hd, falcon ? 2 : 0, hp.n_ctx, b->d_pos, b->att, d, b->qa, b->da, b->sa, st));
    else
        PI_TRY(pi_k_attn_fused_batch(b->qkv, d + 2 * gqa, m->rope_table, b->k_cache + kv_off, b->v_cache + kv_off, b->cache_seq_stride, T,
                                     hp.n_head, hp.n_head_kv, hd, falcon ? 2 : 0, hp.n_ctx, b->d_pos, b->att, d, b->att16, st));
    if (b->unified || b->prefill || hd % 32 != 0) PI_TRY(pi_k_norm_q8_blocks(b->att, T, d, &plain, b->qa, b->da, b->sa, nullptr, st));
    if (!falcon) {
        PI_TRY(pi_k_gemm_q4_t16(wo.quants, wo.scales, d, d, b->qa, b->da, b->sa, T, PI_EPI_ADD, x, nullptr, b->ffn_inp, st));       // ffn_inp = wo.att + x
        pi_norm fn = mk_norm(1, hp.norm_eps, m->L(il, PI_T_FFN_NORM), nullptr);
        PI_TRY(pi_k_norm_q8_blocks_ol(b->ffn_inp, T, d, &fn, b->qf, b->df, b->sf, b->xp16, st));                                     // the predictor reads the rows before the norm
    } else {
        PI_TRY(pi_k_gemm_q4_t16(wo.quants, wo.scales, d, d, b->qa, b->da, b->sa, T, PI_EPI_NONE, nullptr, nullptr, b->attn_out, st));
    }
    PI_TRY(pi_k_gemm_f16_ol(fc1.dev, r, d, b->xp16, T, PI_EPI_RELU, nullptr, nullptr, b->hidden, b->hid16, st));
    PI_TRY(pi_k_batch_predictor_fc2_ol(fc2.dev, ff, r, b->hid16, T, hp.sparse_threshold, b->pred_logits, m->ws, st));
    const auto up = W(PI_T_FFN_UP), down = W(PI_T_FFN_DOWN_T);
    if (!falcon) {
        const auto gate = W(PI_T_FFN_GATE);
        PI_TRY(pi_k_batch_sparse_ffn_q4(b->pred_logits, T, ff, hp.sparse_threshold, up.quants, up.scales, gate.quants, gate.scales, down.quants, down.scales, d,
                                        b->qf, b->df, b->sf, PI_EPI_ADD, b->ffn_inp, nullptr, b->x2, b->h32, b->hq32, b->union_rows, b->n_union + il, m->ws, st));
    } else {
        PI_TRY(pi_k_batch_sparse_ffn_q4(b->pred_logits, T, ff, hp.sparse_threshold, up.quants, up.scales, nullptr, nullptr, down.quants, down.scales, d,
                                        b->qf, b->df, b->sf, PI_EPI_ADD2, b->attn_out, x, b->x2, b->h32, b->hq32, b->union_rows, b->n_union + il, m->ws, st));
    }
    std::swap(b->x, b->x2);
    return PI_OK;
}

// the down projection of layer il with the neurons contiguous ([n_embd][n_ff] fp16), made on first use: a dense mat-mul over the
// neurons wants them along the rows' contiguous dimension (the decode kernels keep the row-per-neuron layout)
int ensure_down_rows(pi_model * m, int il) {
    const pi_hparams & hp = m->hp;
    if ((int)m->down_rows.size() != hp.n_layer) m->down_rows.assign(hp.n_layer, nullptr);
    if (m->down_rows[il]) return PI_OK;
    m->down_rows[il] = m->alloc<__half>((size_t)hp.n_embd * hp.n_ff);
    if (!m->down_rows[il]) return PI_E_HIP;
    return pi_k_transpose_f16(m->L(il, PI_T_FFN_DOWN_T).dev, hp.n_ff, hp.n_embd, m->down_rows[il], m->stream);
}

int batch_layer(pi_model * m, BatchState * b, int il) {
    if (m->q4_steps) return batch_layer_q4(m, b, il);
    const pi_hparams & hp = m->hp;
    const int T = b->n_seq, d = hp.n_embd, ff = hp.n_ff, hd = m->hd, gqa = m->gqa;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    hipStream_t st = m->stream;
    Tensor & wqkv = m->L(il, PI_T_WQKV); Tensor & wo = m->L(il, PI_T_WO);
    Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    const int r = (int)fc1.ne1;
    const size_t kv_off = (size_t)il * hp.n_head_kv * hp.n_ctx * hd;
    float * x = b->x;

    // attention
    pi_norm an;
    if (!falcon) an = mk_norm(1, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), nullptr);
    else if (m->L(il, PI_T_ATTN_NORM_2).dev) an = mk_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM_2), &m->L(il, PI_T_ATTN_NORM_2_B));
    else an = mk_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B));
    // the fp16 inputs of the step's mat-muls (xa16, xf16, xp16, hid16, and att16 of a lockstep step) are kept in the matrix cores'
    // operand layout; the attention of a prompt chunk and of the shared-cell cache write att16 token-major
    PI_TRY(pi_k_norm_round_f16_ol(x, T, d, &an, b->xa16, falcon ? b->xp16 : nullptr, st));    // Falcon: the predictor reads the raw layer input
    PI_TRY(pi_k_gemm_f16_ol(wqkv.dev, d + 2 * gqa, d, b->xa16, T, PI_EPI_NONE, nullptr, nullptr, b->qkv, nullptr, st));
    if (b->unified)
        PI_TRY(cells_attention(m, b, il, T));
    else if (b->prefill)
        PI_TRY(chunk_attention(m, b, T, kv_off));
    else
        PI_TRY(pi_k_attn_fused_batch_ol(b->qkv, d + 2 * gqa, m->rope_table, b->k_cache + kv_off, b->v_cache + kv_off, b->cache_seq_stride, T,
                                        hp.n_head, hp.n_head_kv, hd, falcon ? 2 : 0, hp.n_ctx, b->d_pos, b->att, d, b->att16, st));
    const bool att_ol = !b->unified && !b->prefill;               // the lockstep attention writes its fp16 copy in the operand layout
    auto wo_gemm = att_ol ? pi_k_gemm_f16_ol : pi_k_gemm_f16;

    pi_norm fn;
    if (!falcon) {
        PI_TRY(wo_gemm(wo.dev, d, d, b->att16, T, PI_EPI_ADD, x, nullptr, b->ffn_inp, nullptr, st));             // ffn_inp = wo.att + x
        fn = mk_norm(1, hp.norm_eps, m->L(il, PI_T_FFN_NORM), nullptr);
        PI_TRY(pi_k_norm_round_f16_ol(b->ffn_inp, T, d, &fn, b->xf16, b->xp16, st));                             // FFN input and predictor input in one pass
    } else {
        PI_TRY(wo_gemm(wo.dev, d, d, b->att16, T, PI_EPI_NONE, nullptr, nullptr, b->attn_out, nullptr, st));
        fn = mk_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B));
        if (m->L(il, PI_T_ATTN_NORM_2).dev) PI_TRY(pi_k_norm_round_f16_ol(x, T, d, &fn, b->xf16, nullptr, st));  // two norms: the FFN has its own
    }
    const __half * ffn_x = (falcon && !m->L(il, PI_T_ATTN_NORM_2).dev) ? b->xa16 : b->xf16;                        // single-norm Falcon: attention and FFN share it
    // predictor
    PI_TRY(pi_k_gemm_f16_ol(fc1.dev, r, d, b->xp16, T, PI_EPI_RELU, nullptr, nullptr, b->hidden, b->hid16, st));
    PI_TRY(pi_k_batch_predictor_fc2_ol(fc2.dev, ff, r, b->hid16, T, hp.sparse_threshold, b->pred_logits, m->ws, st));
    // Dense cross-over (the reference's switch from its batch-sparse kernels to a plain mat-mul, ggml-cuda.cu:8787-8814, 7717-7756):
    // when the sequences' active sets together cover nearly all of the layer, gathering rows costs more than streaming all of them.
    // Measured on the 13B shape, 40 layers, 16 sequences, 128-token prompts (ms per step, union kernels / dense): union 0.41 of n_ff
    // 5.59 / 7.61, 0.61 7.03 / 7.66, 0.75 7.26 / 7.68, 0.92 7.44 / 7.74, 0.99 7.55 / 7.77 - the union kernels win everywhere (they lost
    // beyond 0.9, 9.60 / 9.38 at 0.99, before the union rows were dealt evenly to the units and the down projection stopped going
    // through LDS), so the switch is off unless the caller sets a fraction (pi_model_batch_set_dense_above).  The choice is made from
    // the union the previous step measured (the count below keeps that statistic alive while the layer runs dense).
    if (!b->prefill && !b->unified && il < (int)b->dense_ffn.size() && b->dense_ffn[il]) {
        PI_TRY(pi_k_batch_union_count(ff, b->union_rows, b->n_union + il, m->ws, st));
        PI_TRY(pi_k_gemm_f16_ol(up.dev, ff, d, ffn_x, T, PI_EPI_NONE, nullptr, nullptr, b->up_out, nullptr, st));
        if (!falcon) PI_TRY(pi_k_gemm_f16_ol(gate.dev, ff, d, ffn_x, T, PI_EPI_NONE, nullptr, nullptr, b->gate_out, nullptr, st));
        PI_TRY(pi_k_ffn_h_f16(b->up_out, falcon ? nullptr : b->gate_out, b->pred_logits, hp.sparse_threshold, T, ff, b->h16, st));
        if (!falcon) PI_TRY(pi_k_gemm_f16(m->down_rows[il], d, ff, b->h16, T, PI_EPI_ADD, b->ffn_inp, nullptr, b->x2, nullptr, st));
        else         PI_TRY(pi_k_gemm_f16(m->down_rows[il], d, ff, b->h16, T, PI_EPI_ADD2, b->attn_out, x, b->x2, nullptr, st));
        std::swap(b->x, b->x2);
        return PI_OK;
    }
    // sparse FFN over the union of the sequences' active sets
    if (!falcon)
        PI_TRY(pi_k_batch_sparse_ffn_ol(b->pred_logits, T, ff, hp.sparse_threshold, up.dev, gate.dev, down.dev, d, ffn_x, PI_EPI_ADD, b->ffn_inp, nullptr,
                                     b->x2, b->union_rows, b->n_union + il, m->ws, st));
    else
        PI_TRY(pi_k_batch_sparse_ffn_ol(b->pred_logits, T, ff, hp.sparse_threshold, up.dev, nullptr, down.dev, d, ffn_x, PI_EPI_ADD2, b->attn_out, x,
                                     b->x2, b->union_rows, b->n_union + il, m->ws, st));
    std::swap(b->x, b->x2);
    return PI_OK;
}

int batch_step(pi_model * m, BatchState * b) {
    const pi_hparams & hp = m->hp;
    const int T = b->n_seq, d = hp.n_embd;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    hipStream_t st = m->stream;
    if (m->glob[PI_T_TOK_EMBD].type == PI_TYPE_Q4_0) PI_TRY(pi_k_embed_batch_q4(m->glob[PI_T_TOK_EMBD].dev, d, b->d_tokens, T, b->x, st));
    else PI_TRY(pi_k_embed_batch(m->glob[PI_T_TOK_EMBD].dev, d, b->d_tokens, T, b->x, st));
    for (int il = 0; il < hp.n_layer; ++il) PI_TRY(batch_layer(m, b, il));
    pi_norm on = mk_norm(falcon ? 2 : 1, hp.norm_eps, m->glob[PI_T_OUTPUT_NORM], falcon ? &m->glob[PI_T_OUTPUT_NORM_B] : nullptr);
    if (m->q4_steps && m->glob[PI_T_OUTPUT].type == PI_TYPE_Q4_0) {
        const auto wout = m->q4_split.at(&m->glob[PI_T_OUTPUT]);
        PI_TRY(pi_k_norm_q8_blocks(b->x, T, d, &on, b->qa, b->da, b->sa, nullptr, st));
        PI_TRY(pi_k_gemm_q4_t16(wout.quants, wout.scales, hp.n_vocab, d, b->qa, b->da, b->sa, T, PI_EPI_NONE, nullptr, nullptr, b->logits, st));
    } else {
        PI_TRY(pi_k_norm_round_f16_ol(b->x, T, d, &on, b->xa16, nullptr, st));
        PI_TRY(pi_k_gemm_f16_ol(m->glob[PI_T_OUTPUT].dev, hp.n_vocab, d, b->xa16, T, PI_EPI_NONE, nullptr, nullptr, b->logits, nullptr, st));
    }
    PI_TRY(pi_k_argmax_batch(b->logits, hp.n_vocab, T, b->d_tokens, b->d_pos, b->d_step, b->d_out_tokens, b->max_steps, st));
    PI_TRY(pi_k_step_advance(b->d_step, st));
    return PI_OK;
}

}  // namespace

namespace {

// why the model cannot take multi-token steps on the F16 kernels, or null
const char * batch_unsupported(pi_model * m) {
    const pi_hparams & hp = m->hp;
    if (m->hybrid) return "hybrid models decode one token at a time";
    for (int il = 0; il < hp.n_layer; ++il)
        for (int k : {PI_T_WQKV, PI_T_WO, PI_T_FC1, PI_T_FC2, PI_T_FFN_UP, PI_T_FFN_DOWN_T})
            if (m->L(il, k).type != PI_TYPE_F16) return "multi-token steps need F16 weights, or Q4_0 matrices with F16 predictors";
    if (m->glob[PI_T_TOK_EMBD].type != PI_TYPE_F16 || m->glob[PI_T_OUTPUT].type != PI_TYPE_F16) return "multi-token steps need F16 weights, or Q4_0 matrices with F16 predictors";
    if (hp.n_embd % 512 || (int)m->L(0, PI_T_FC1).ne1 % 128) return "n_embd % 512 == 0 and predictor rank % 128 == 0 required";
    return nullptr;
}

// step buffers for up to T tokens; caches only for independent sequences
BatchState * batch_alloc(pi_model * m, int T, bool with_caches) {
    const pi_hparams & hp = m->hp;
    const int d = hp.n_embd, ff = hp.n_ff, r = (int)m->L(0, PI_T_FC1).ne1;
    BatchState * b = new BatchState();
    b->n_seq = T;
    b->cache_seq_stride = (size_t)hp.n_layer * hp.n_head_kv * hp.n_ctx * m->hd;
    const size_t n = T;
    bool ok = true;
    if (with_caches) {
        b->k_cache = m->alloc<__half>(b->cache_seq_stride * n); b->v_cache = m->alloc<__half>(b->cache_seq_stride * n);
        ok = b->k_cache && b->v_cache;
    } else {
        b->q_rot = m->alloc<float>(n * d);
        ok = b->q_rot != nullptr;
    }
    b->x = m->alloc<float>(n * d); b->x2 = m->alloc<float>(n * d); b->qkv = m->alloc<float>(n * (d + 2 * m->gqa));
    b->att = m->alloc<float>(n * d); b->attn_out = m->alloc<float>(n * d); b->ffn_inp = m->alloc<float>(n * d);
    b->hidden = m->alloc<float>(n * r); b->pred_logits = m->alloc<float>(n * ff); b->logits = m->alloc<float>(n * hp.n_vocab);
    const size_t n16 = n < 16 ? 16 : n;                            // steps of up to 16 tokens keep these in the operand layout: 16 token slots
    b->xa16 = m->alloc<__half>(n16 * d); b->xf16 = m->alloc<__half>(n16 * d); b->xp16 = m->alloc<__half>(n16 * d);
    b->att16 = m->alloc<__half>(n16 * d); b->hid16 = m->alloc<__half>(n16 * r);
    b->d_tokens = m->alloc<int32_t>(n); b->d_pos = m->alloc<int32_t>(n); b->d_step = m->alloc<int32_t>(1);
    b->d_out_tokens = m->alloc<int32_t>((size_t)b->max_steps * n); b->union_rows = m->alloc<int32_t>(ff); b->n_union = m->alloc<int32_t>(hp.n_layer);
    if (m->L(0, PI_T_WQKV).type == PI_TYPE_Q4_0 && d % 32 == 0) {          // steps of a Q4_0 model on integer matrix cores
        b->qa = m->alloc<unsigned char>((size_t)16 * d); b->qf = m->alloc<unsigned char>((size_t)16 * d);
        b->da = m->alloc<float>((size_t)d / 32 * 16); b->df = m->alloc<float>((size_t)d / 32 * 16);
        b->sa = m->alloc<int32_t>((size_t)d / 32 * 16); b->sf = m->alloc<int32_t>((size_t)d / 32 * 16);
        b->h32 = m->alloc<float>((size_t)16 * ff); b->hq32 = m->alloc<float>((size_t)16 * ff);
        ok = ok && b->qa && b->qf && b->da && b->df && b->sa && b->sf && b->h32 && b->hq32;
        if (ok) ok = hipMemsetAsync(b->qa, 0, (size_t)16 * d, m->stream) == hipSuccess && hipMemsetAsync(b->qf, 0, (size_t)16 * d, m->stream) == hipSuccess &&
                     hipMemsetAsync(b->hq32, 0, sizeof(float) * 16 * ff, m->stream) == hipSuccess && hipMemsetAsync(b->h32, 0, sizeof(float) * 16 * ff, m->stream) == hipSuccess;
    }
    if (with_caches) {                                 // the dense form of a step's FFN (dense_ffn)
        b->up_out = m->alloc<float>(n * ff); b->gate_out = m->alloc<float>(n * ff); b->h16 = m->alloc<__half>(n * ff);
        ok = ok && b->up_out && b->gate_out && b->h16;
        b->dense_ffn.assign(hp.n_layer, 0);
    }
    if (!ok || !b->x || !b->x2 || !b->qkv || !b->att || !b->attn_out || !b->ffn_inp || !b->hidden || !b->pred_logits || !b->logits ||
        !b->xa16 || !b->xf16 || !b->xp16 || !b->att16 || !b->hid16 || !b->d_tokens || !b->d_pos || !b->d_step || !b->d_out_tokens || !b->union_rows || !b->n_union) {
        delete b;
        return nullptr;
    }
    return b;
}

}  // namespace

namespace {
// one layer of a wide prompt chunk (16 < T <= 128): every mat-mul reads its matrix once for the chunk; with that many tokens the union
// of the active sets is nearly every neuron, so gate/up run dense and the predictor's mask turns into exact zeros of h (what the
// sparse operators compute, term by term: an inactive neuron contributes nothing to the down projection)
// one dense mat-mul of a chunk: the library's plan for long chunks, this library's own kernel otherwise
int chunk_gemm(pi_model * m, const void * W, int rows, int cols, const void * xn, int T, int epi, const float * add1, const float * add2,
               float * y, void * y16) {
    if (m->gemm_lib) return pi_gemm_lib_f16(m->gemm_lib, W, rows, cols, xn, T, epi, add1, add2, y, y16, m->stream);
    return pi_k_gemm_tile_f16(W, rows, cols, xn, T, epi, add1, add2, y, y16, 0, m->stream);
}

// a matrix of layer il as fp16 rows for a chunk's mat-mul: an F16 matrix that is whole on the device as stored; a Q4_0 one expanded into
// the chunk's scratch (values (q - 8) * d rounded to fp16); an FFN matrix of a hybrid layer assembled there from the compact matrix of the
// resident neurons and the non-resident rows in pinned host memory, which the kernel reads over the host link once per chunk
int chunk_weight(pi_model * m, BatchState * b, int il, int kind, int rows, int cols, const void ** out) {
    Tensor & t = m->L(il, kind);
    const bool ffn = kind == PI_T_FFN_UP || kind == PI_T_FFN_GATE || kind == PI_T_FFN_DOWN_T;
    const bool split = ffn && m->L(il, PI_T_GPU_BUCKET).dev != nullptr;
    const void * rest = !split ? nullptr : kind == PI_T_FFN_UP ? m->rest_up[il] : kind == PI_T_FFN_GATE ? m->rest_gate[il] : m->rest_down[il];
    if (split && b->staged_layer[il & 1] == il) {      // the copy stream has brought this layer's rows into device memory
        const int which = kind == PI_T_FFN_UP ? 0 : kind == PI_T_FFN_GATE ? 1 : 2;
        rest = b->stage[il & 1] + (size_t)which * b->stage_rows * b->stage_row_bytes;
    }
    const uint32_t * hw = split ? m->hot_words[il] : nullptr;
    const int32_t * hpx = split ? m->hot_prefix[il] : nullptr;
    if (t.type == PI_TYPE_Q4_0) {
        PI_TRY(pi_k_dequant_q4_f16(t.dev, rest, hw, hpx, rows, cols, b->w16, m->stream));
        *out = b->w16;
    } else if (split) {
        PI_TRY(pi_k_assemble_rows_f16(t.dev, rest, hw, hpx, rows, cols, b->w16, m->stream));
        *out = b->w16;
    } else {
        *out = t.dev;
    }
    return PI_OK;
}

int wide_layer(pi_model * m, BatchState * b, int il) {
    const pi_hparams & hp = m->hp;
    const int T = b->n_seq, d = hp.n_embd, ff = hp.n_ff, hd = m->hd, gqa = m->gqa;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    hipStream_t st = m->stream;
    Tensor & wqkv = m->L(il, PI_T_WQKV); Tensor & wo = m->L(il, PI_T_WO);
    Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    const int r = (int)fc1.ne1;
    const size_t kv_off = (size_t)il * hp.n_head_kv * hp.n_ctx * hd;
    float * x = b->x;
    const void * W = nullptr;
    const pi_norm plain{0, 0.0f, nullptr, nullptr};
    pi_norm an;
    if (!falcon) an = mk_norm(1, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), nullptr);
    else if (m->L(il, PI_T_ATTN_NORM_2).dev) an = mk_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM_2), &m->L(il, PI_T_ATTN_NORM_2_B));
    else an = mk_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B));
    PI_TRY(batch_input(wqkv.type, x, T, d, &an, b->xa16, falcon ? b->xp16 : nullptr, st));
    PI_TRY(chunk_weight(m, b, il, PI_T_WQKV, d + 2 * gqa, d, &W));
    PI_TRY(chunk_gemm(m, W, d + 2 * gqa, d, b->xa16, T, PI_EPI_NONE, nullptr, nullptr, b->qkv, nullptr));
    PI_TRY(chunk_attention(m, b, T, kv_off));
    if (wo.type == PI_TYPE_Q4_0) PI_TRY(pi_k_norm_q8_round_f16(b->att, T, d, &plain, b->att16, nullptr, st));
    PI_TRY(chunk_weight(m, b, il, PI_T_WO, d, d, &W));
    pi_norm fn;
    const __half * ffn_x = b->xf16;
    if (!falcon) {
        PI_TRY(chunk_gemm(m, W, d, d, b->att16, T, PI_EPI_ADD, x, nullptr, b->ffn_inp, nullptr));
        fn = mk_norm(1, hp.norm_eps, m->L(il, PI_T_FFN_NORM), nullptr);
        PI_TRY(batch_input(up.type, b->ffn_inp, T, d, &fn, b->xf16, b->xp16, st));
    } else {
        PI_TRY(chunk_gemm(m, W, d, d, b->att16, T, PI_EPI_NONE, nullptr, nullptr, b->attn_out, nullptr));
        fn = mk_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B));
        // the FFN branch reads the layer input under its own norm; with a single norm it shares the attention branch's rows unless
        // the two matrices want different containers (fp16 against Q8_0 blocks)
        if (m->L(il, PI_T_ATTN_NORM_2).dev || up.type != wqkv.type) PI_TRY(batch_input(up.type, x, T, d, &fn, b->xf16, nullptr, st));
        else ffn_x = b->xa16;
    }
    PI_TRY(chunk_gemm(m, fc1.dev, r, d, b->xp16, T, PI_EPI_RELU, nullptr, nullptr, b->hidden, b->hid16));
    PI_TRY(chunk_gemm(m, fc2.dev, ff, r, b->hid16, T, PI_EPI_NONE, nullptr, nullptr, b->pred_logits, nullptr));
    PI_TRY(chunk_weight(m, b, il, PI_T_FFN_UP, ff, d, &W));
    PI_TRY(chunk_gemm(m, W, ff, d, ffn_x, T, PI_EPI_NONE, nullptr, nullptr, b->up_out, nullptr));
    if (!falcon) {
        PI_TRY(chunk_weight(m, b, il, PI_T_FFN_GATE, ff, d, &W));
        PI_TRY(chunk_gemm(m, W, ff, d, ffn_x, T, PI_EPI_NONE, nullptr, nullptr, b->gate_out, nullptr));
    }
    if (down.type == PI_TYPE_Q4_0) PI_TRY(pi_k_ffn_h_q8_f16(b->up_out, falcon ? nullptr : b->gate_out, b->pred_logits, hp.sparse_threshold, T, ff, b->h16, st));
    else                           PI_TRY(pi_k_ffn_h_f16(b->up_out, falcon ? nullptr : b->gate_out, b->pred_logits, hp.sparse_threshold, T, ff, b->h16, st));
    const void * Wd = m->down_rows[il];
    if (!Wd) {
        PI_TRY(chunk_weight(m, b, il, PI_T_FFN_DOWN_T, ff, d, &W));
        PI_TRY(pi_k_transpose_f16(W, ff, d, b->w16t, st));
        Wd = b->w16t;
    }
    if (!falcon) PI_TRY(chunk_gemm(m, Wd, d, ff, b->h16, T, PI_EPI_ADD, b->ffn_inp, nullptr, b->x2, nullptr));
    else         PI_TRY(chunk_gemm(m, Wd, d, ff, b->h16, T, PI_EPI_ADD2, b->attn_out, x, b->x2, nullptr));
    std::swap(b->x, b->x2);
    return PI_OK;
}

// why the model's prompts cannot go through wide chunks, or null
const char * wide_unsupported(pi_model * m) {
    const pi_hparams & hp = m->hp;
    if (m->capture) return "capture hooks follow single tokens";
    if (hp.n_embd % 256 || hp.n_ff % 256 || (int)m->L(0, PI_T_FC1).ne1 % 256) return "n_embd, n_ff and the predictor rank must be multiples of 256";
    const int te = m->glob[PI_T_TOK_EMBD].type;
    if (te != PI_TYPE_F16 && te != PI_TYPE_Q4_0) return "embedding table must be F16 or Q4_0";
    for (int il = 0; il < hp.n_layer; ++il) {
        for (int k : {PI_T_WQKV, PI_T_WO, PI_T_FFN_UP, PI_T_FFN_GATE, PI_T_FFN_DOWN_T}) {
            if (k == PI_T_FFN_GATE && hp.arch == PI_ARCH_FALCON) continue;
            const int ty = m->L(il, k).type;
            if (ty != PI_TYPE_F16 && ty != PI_TYPE_Q4_0) return "matrices must be F16 or Q4_0";
        }
        if (m->L(il, PI_T_FC1).type != PI_TYPE_F16 || m->L(il, PI_T_FC2).type != PI_TYPE_F16 || (int)m->L(il, PI_T_FC1).ne1 != (int)m->L(0, PI_T_FC1).ne1)
            return "predictors must be F16 and of one rank";
        if (hp.arch != PI_ARCH_FALCON && m->L(il, PI_T_FFN_GATE).type != m->L(il, PI_T_FFN_UP).type) return "gate and up must share a type";
        if (m->L(il, PI_T_GPU_BUCKET).dev) {
            if (!m->hot_words[il]) return "hybrid layers need n_ff % 32 == 0";
            for (int k : {PI_T_FFN_UP, PI_T_FFN_GATE, PI_T_FFN_DOWN_T})
                if (!(k == PI_T_FFN_GATE && hp.arch == PI_ARCH_FALCON) && !m->L(il, k).host && !m->rest_up[il]) return "hybrid layers need the host copy of the FFN matrices";
        }
    }
    return nullptr;
}
}  // namespace

namespace {
// queues the copies of layer il's non-resident rows into its staging buffer on the copy stream (after the layer that used the
// buffer last has finished with it) and marks the buffer; layers that are whole on the device need nothing
int stage_rest_rows(pi_model * m, BatchState * b, int il) {
    if (il >= m->hp.n_layer || !b->copy_stream || !m->L(il, PI_T_GPU_BUCKET).dev) return PI_OK;
    const int s = il & 1;
    const size_t n_rest = (size_t)m->hp.n_ff - (size_t)m->L(il, PI_T_GPU_BUCKET).ne0;
    const size_t rb = m->L(il, PI_T_FFN_UP).type == PI_TYPE_Q4_0 ? (size_t)(m->hp.n_embd / 32) * 18 : (size_t)m->hp.n_embd * 2;
    if (n_rest > b->stage_rows || rb > b->stage_row_bytes) return pi::fail(PI_E_STATE, "stage_rest_rows: staging buffer too small");
    if (b->free_recorded[s]) PI_HIP_TRY(hipStreamWaitEvent(b->copy_stream, b->ev_free[s], 0));
    const void * src[3] = {m->rest_up[il], m->hp.arch == PI_ARCH_FALCON ? nullptr : m->rest_gate[il], m->rest_down[il]};
    for (int k = 0; k < 3; ++k)
        if (src[k] && n_rest) PI_HIP_TRY(hipMemcpyAsync(b->stage[s] + (size_t)k * b->stage_rows * b->stage_row_bytes, src[k], n_rest * rb, hipMemcpyHostToDevice, b->copy_stream));
    PI_HIP_TRY(hipEventRecord(b->ev_copied[s], b->copy_stream));
    b->staged_layer[s] = il;
    return PI_OK;
}
}  // namespace

namespace pi {
bool prefill_wide_supported(pi_model * m) {
    const char * off = getenv("PI_NO_PREFILL_WIDE");          // the comparison side of the chunk tests: prompts in steps of 16 tokens
    return !(off && off[0] == '1') && wide_unsupported(m) == nullptr;
}

int prefill_wide_max(pi_model * m) { (void)m; return 512; }      // the longest chunk of the attention, embedding and elementwise kernels

// PI_PREFILL_GEMM=own: the dense mat-muls of prompt chunks run on this library's LDS-tiled MFMA kernel instead of hipBLASLt plans
static bool prefill_own_gemm() {
    const char * own = getenv("PI_PREFILL_GEMM");
    return own && !strcmp(own, "own");
}

int prefill_wide_chunk(pi_model * m, const int32_t * tokens, int T, int n_past) {
    const int kMaxT = prefill_wide_max(m);
    if (T <= 16 || T > kMaxT) return pi::fail(PI_E_ARG, "prefill_wide_chunk: chunk length outside 17 .. prefill_wide_max");
    const pi_hparams & hp = m->hp;
    if (!m->prefill_wide) {
        if (!prefill_own_gemm() && !m->gemm_lib) {
            m->gemm_lib = pi_gemm_lib_create((size_t)64 << 20);
            if (!m->gemm_lib) return PI_E_HIP;
        }
        BatchState * b = batch_alloc(m, kMaxT, false);
        if (!b) return PI_E_HIP;
        // until the state is complete every early return undoes what was created here (the device buffers stay with the model's
        // allocation list; the mat-mul library is kept for the next attempt)
        struct SetupGuard {
            pi_model * m; BatchState * b; bool armed = true;
            ~SetupGuard() {
                if (!armed) return;
                if (b->copy_stream) (void)hipStreamDestroy(b->copy_stream);
                for (int i = 0; i < 2; ++i) { if (b->ev_copied[i]) (void)hipEventDestroy(b->ev_copied[i]); if (b->ev_free[i]) (void)hipEventDestroy(b->ev_free[i]); }
                delete b;
                m->down_rows.clear();
            }
        } guard{m, b};
        b->prefill = true;
        b->up_out = m->alloc<float>((size_t)kMaxT * hp.n_ff);
        b->gate_out = hp.arch == PI_ARCH_FALCON ? nullptr : m->alloc<float>((size_t)kMaxT * hp.n_ff);
        b->h16 = m->alloc<__half>((size_t)kMaxT * hp.n_ff);
        if (!b->up_out || (hp.arch != PI_ARCH_FALCON && !b->gate_out) || !b->h16) return PI_E_HIP;
        // the down projection of a chunk is a mat-mul whose reduction runs over the neurons.  An F16 layer that is whole on the device
        // gets one more copy of it with the neurons contiguous (n_embd x n_ff fp16; the decode loop keeps the row-per-neuron layout);
        // Q4_0 and hybrid layers expand one matrix at a time into scratch instead, so that prompts leave the model's footprint as
        // the quantisation and the VRAM split made it
        size_t w16 = 0;
        bool scratch = false;
        if ((int)m->down_rows.size() != hp.n_layer) m->down_rows.assign(hp.n_layer, nullptr);
        for (int il = 0; il < hp.n_layer; ++il) {
            const bool split = m->L(il, PI_T_GPU_BUCKET).dev != nullptr;
            if (split) PI_TRY(gather_rest_rows(m, il));
            if (m->L(il, PI_T_WQKV).type == PI_TYPE_Q4_0) w16 = std::max(w16, (size_t)(hp.n_embd + 2 * m->gqa) * hp.n_embd);
            if (m->L(il, PI_T_WO).type == PI_TYPE_Q4_0) w16 = std::max(w16, (size_t)hp.n_embd * hp.n_embd);
            if (split || m->L(il, PI_T_FFN_UP).type == PI_TYPE_Q4_0 || m->L(il, PI_T_FFN_DOWN_T).type == PI_TYPE_Q4_0) w16 = std::max(w16, (size_t)hp.n_ff * hp.n_embd);
            if (split || m->L(il, PI_T_FFN_DOWN_T).type == PI_TYPE_Q4_0) { scratch = true; continue; }
            PI_TRY(ensure_down_rows(m, il));
        }
        if (w16) b->w16 = m->alloc<__half>(w16);
        if (scratch) b->w16t = m->alloc<__half>((size_t)hp.n_embd * hp.n_ff);
        if ((w16 && !b->w16) || (scratch && !b->w16t)) return PI_E_HIP;
        // two staging buffers for the non-resident rows of hybrid layers (the largest such layer decides their size)
        for (int il = 0; il < hp.n_layer; ++il) {
            if (!m->L(il, PI_T_GPU_BUCKET).dev) continue;
            b->stage_rows = std::max(b->stage_rows, (size_t)hp.n_ff - (size_t)m->L(il, PI_T_GPU_BUCKET).ne0);
            b->stage_row_bytes = std::max(b->stage_row_bytes, m->L(il, PI_T_FFN_UP).type == PI_TYPE_Q4_0 ? (size_t)(hp.n_embd / 32) * 18 : (size_t)hp.n_embd * 2);
        }
        if (b->stage_rows) {
            for (int i = 0; i < 2; ++i) {
                b->stage[i] = m->alloc<unsigned char>(3 * b->stage_rows * b->stage_row_bytes);
                if (!b->stage[i]) return PI_E_HIP;
                PI_HIP_TRY(hipEventCreateWithFlags(&b->ev_copied[i], hipEventDisableTiming));
                PI_HIP_TRY(hipEventCreateWithFlags(&b->ev_free[i], hipEventDisableTiming));
            }
            PI_HIP_TRY(hipStreamCreateWithFlags(&b->copy_stream, hipStreamNonBlocking));
        }
        guard.armed = false;
        m->prefill_wide = b;
    }
    BatchState * b = m->prefill_wide;
    b->n_seq = T;
    b->kv_hi = n_past + T;
    int32_t pos[512];
    for (int t = 0; t < T; ++t) pos[t] = n_past + t;
    PI_HIP_TRY(hipMemcpyAsync(b->d_tokens, tokens, sizeof(int32_t) * T, hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipMemcpyAsync(b->d_pos, pos, sizeof(int32_t) * T, hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    if (m->glob[PI_T_TOK_EMBD].type == PI_TYPE_Q4_0) PI_TRY(pi_k_embed_batch_q4(m->glob[PI_T_TOK_EMBD].dev, hp.n_embd, b->d_tokens, T, b->x, m->stream));
    else PI_TRY(pi_k_embed_batch(m->glob[PI_T_TOK_EMBD].dev, hp.n_embd, b->d_tokens, T, b->x, m->stream));
    b->staged_layer[0] = b->staged_layer[1] = -1;
    PI_TRY(stage_rest_rows(m, b, 0));
    for (int il = 0; il < hp.n_layer; ++il) {
        PI_TRY(stage_rest_rows(m, b, il + 1));                   // the next layer's rows cross the host link under this layer's mat-muls
        const bool staged = b->staged_layer[il & 1] == il;
        if (staged) PI_HIP_TRY(hipStreamWaitEvent(m->stream, b->ev_copied[il & 1], 0));
        PI_TRY(wide_layer(m, b, il));
        if (staged) { PI_HIP_TRY(hipEventRecord(b->ev_free[il & 1], m->stream)); b->free_recorded[il & 1] = true; }
    }
    return PI_OK;
}

bool prefill_supported(pi_model * m) {
    return !m->capture && (batch_unsupported(m) == nullptr || q4_steps_unsupported(m) == nullptr);
}

// T <= 16 consecutive prompt tokens of the model's own sequence in one step: the weights are read once for the chunk
// (the prompt-phase counterpart of llama_decode with n_tokens > 1; the reference's batch kernels, ggml-cuda.cu:6994-7034)
int prefill_chunk(pi_model * m, const int32_t * tokens, int T, int n_past) {
    if (T < 1 || T > 16) return pi::fail(PI_E_ARG, "prefill_chunk: 1 <= T <= 16");
    if (batch_unsupported(m) != nullptr) PI_TRY(ensure_q4_split(m));          // a Q4_0 model: the integer matrix-core route
    if (!m->prefill) {
        m->prefill = batch_alloc(m, 16, false);
        if (!m->prefill) return PI_E_HIP;
        m->prefill->prefill = true;
    }
    BatchState * b = m->prefill;
    b->n_seq = T;
    b->kv_hi = n_past + T;
    int32_t pos[16];
    for (int t = 0; t < T; ++t) pos[t] = n_past + t;
    PI_HIP_TRY(hipMemcpyAsync(b->d_tokens, tokens, sizeof(int32_t) * T, hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipMemcpyAsync(b->d_pos, pos, sizeof(int32_t) * T, hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    if (m->glob[PI_T_TOK_EMBD].type == PI_TYPE_Q4_0) PI_TRY(pi_k_embed_batch_q4(m->glob[PI_T_TOK_EMBD].dev, m->hp.n_embd, b->d_tokens, T, b->x, m->stream));
    else PI_TRY(pi_k_embed_batch(m->glob[PI_T_TOK_EMBD].dev, m->hp.n_embd, b->d_tokens, T, b->x, m->stream));
    for (int il = 0; il < m->hp.n_layer; ++il) PI_TRY(batch_layer(m, b, il));
    return PI_OK;
}

void batch_destroy(pi_model * m) {
    if (m->prefill) { delete m->prefill; m->prefill = nullptr; }
    if (m->prefill_wide) {
        BatchState * b = m->prefill_wide;
        if (b->copy_stream) { (void)hipStreamSynchronize(b->copy_stream); (void)hipStreamDestroy(b->copy_stream); }
        for (int i = 0; i < 2; ++i) { if (b->ev_copied[i]) (void)hipEventDestroy(b->ev_copied[i]); if (b->ev_free[i]) (void)hipEventDestroy(b->ev_free[i]); }
        delete b;
        m->prefill_wide = nullptr;
    }
    if (m->gemm_lib) { (void)pi_gemm_lib_destroy(m->gemm_lib); m->gemm_lib = nullptr; }
    if (m->cells) { delete m->cells; m->cells = nullptr; }
    if (!m->batch) return;
    if (m->batch->graph_exec) (void)hipGraphExecDestroy(m->batch->graph_exec);
    if (m->batch->graph) (void)hipGraphDestroy(m->batch->graph);
    delete m->batch;                      // device buffers are owned by the model's allocation list
    m->batch = nullptr;
}
}  // namespace pi

namespace {
// after a step has completed: which layers run their FFN dense in the next one
int choose_dense_layers(pi_model * m, BatchState * b) {
    const pi_hparams & hp = m->hp;
    if (hp.n_ff % 128 || hp.n_embd % 128 || m->q4_steps) return PI_OK;            // the dense mat-muls' shapes; the integer route has no dense form
    std::vector<int32_t> u(hp.n_layer);
    PI_TRY(pi_memcpy_d2h(u.data(), b->n_union, sizeof(int32_t) * hp.n_layer));
    for (int il = 0; il < hp.n_layer; ++il) {
        const bool dense = b->dense_above <= 0.0f || (b->dense_above < 1.0f && (float)u[il] > b->dense_above * (float)hp.n_ff);
        if (dense) PI_TRY(ensure_down_rows(m, il));
        b->dense_ffn[il] = dense ? 1 : 0;
    }
    return PI_OK;
}
}  // namespace

extern "C" {

int pi_model_batch_set_dense_above(pi_model * m, float fraction) {
    if (!m || !m->batch) return pi::fail(PI_E_STATE, "pi_model_batch_set_dense_above: pi_model_batch_init first");
    m->batch->dense_above = fraction;
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    return choose_dense_layers(m, m->batch);
}

int pi_model_batch_dense_layers(pi_model * m) {
    if (!m || !m->batch) return pi::fail(PI_E_STATE, "pi_model_batch_dense_layers: pi_model_batch_init first");
    int n = 0;
    for (char c : m->batch->dense_ffn) n += c ? 1 : 0;
    return n;
}

int pi_model_batch_init(pi_model * m, int n_seq) {
    if (!m || !m->finalized) return pi::fail(PI_E_STATE, "pi_model_batch_init: model not finalized");
    if (n_seq < 1 || n_seq > 16) return pi::fail(PI_E_ARG, "pi_model_batch_init: 1 <= n_seq <= 16");
    if (m->batch) return pi::fail(PI_E_STATE, "pi_model_batch_init: already initialised");
    if (!m->rope_table || !pi_k_attn_fused_supported(m->hd, m->hp.n_ctx)) return pi::fail(PI_E_UNSUPPORTED, "pi_model_batch_init: head size or context outside the fused attention kernel (pi_k_attn_fused_supported)");
    const bool q4_route = q4_steps_unsupported(m) == nullptr;
    if (!q4_route) if (const char * why = batch_unsupported(m)) { pi::set_error(why); return PI_E_UNSUPPORTED; }
    if (q4_route) PI_TRY(ensure_q4_split(m));
    BatchState * b = batch_alloc(m, n_seq, true);
    if (!b) return PI_E_HIP;
    const size_t T = n_seq;
    PI_HIP_TRY(hipMemsetAsync(b->k_cache, 0, sizeof(__half) * b->cache_seq_stride * T, m->stream));
    PI_HIP_TRY(hipMemsetAsync(b->v_cache, 0, sizeof(__half) * b->cache_seq_stride * T, m->stream));
    PI_HIP_TRY(hipMemsetAsync(b->n_union, 0, sizeof(int32_t) * m->hp.n_layer, m->stream));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    m->batch = b;
    return PI_OK;
}

int pi_model_batch_decode(pi_model * m, const int32_t * tokens, const int32_t * positions, int32_t * next_tokens, float * logits_out) {
    if (!m || !m->batch) return pi::fail(PI_E_STATE, "pi_model_batch_decode: pi_model_batch_init first");
    if (!tokens || !positions) return pi::fail(PI_E_ARG, "pi_model_batch_decode: null pointer");
    BatchState * b = m->batch;
    for (auto & v : b->kv_pos) if (!v.empty()) return pi::fail(PI_E_STATE, "pi_model_batch_decode: a sequence's KV cells are not at contiguous positions");
    for (int t = 0; t < b->n_seq; ++t) {
        if (tokens[t] < 0 || tokens[t] >= m->hp.n_vocab) return pi::fail(PI_E_ARG, "pi_model_batch_decode: token id out of range");
        if (positions[t] < 0 || positions[t] >= m->hp.n_ctx) return pi::fail(PI_E_ARG, "pi_model_batch_decode: position outside the context");
    }
    PI_HIP_TRY(hipMemcpyAsync(b->d_tokens, tokens, sizeof(int32_t) * b->n_seq, hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipMemcpyAsync(b->d_pos, positions, sizeof(int32_t) * b->n_seq, hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipMemsetAsync(b->d_step, 0, 4, m->stream));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));          // the host arrays may be pageable: finish the copies before returning control
    PI_TRY(batch_step(m, m->batch));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    PI_TRY(choose_dense_layers(m, b));
    if (next_tokens) PI_TRY(pi_memcpy_d2h(next_tokens, b->d_tokens, sizeof(int32_t) * b->n_seq));
    if (logits_out) PI_TRY(pi_memcpy_d2h(logits_out, b->logits, sizeof(float) * (size_t)b->n_seq * m->hp.n_vocab));
    return PI_OK;
}

int pi_model_batch_generate(pi_model * m, int n_steps, int32_t * out_tokens, float * ms_out) {
    if (!m || !m->batch) return pi::fail(PI_E_STATE, "pi_model_batch_generate: pi_model_batch_init first");
    BatchState * b = m->batch;
    if (n_steps <= 0 || n_steps > b->max_steps || !out_tokens) return pi::fail(PI_E_ARG, "pi_model_batch_generate: bad step count");
    for (auto & v : b->kv_pos) if (!v.empty()) return pi::fail(PI_E_STATE, "pi_model_batch_generate: a sequence's KV cells are not at contiguous positions");
    std::vector<int32_t> pos(b->n_seq);
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    PI_TRY(pi_memcpy_d2h(pos.data(), b->d_pos, sizeof(int32_t) * b->n_seq));
    for (int t = 0; t < b->n_seq; ++t)
        if (pos[t] + n_steps > m->hp.n_ctx) return pi::fail(PI_E_ARG, "pi_model_batch_generate: would run past the context");
    PI_HIP_TRY(hipMemsetAsync(b->d_step, 0, 4, m->stream));
    const char * no_graph = getenv("PI_NO_GRAPH");
    const bool use_graph = !(no_graph && no_graph[0] == '1');
    if (b->graph_exec && b->graph_dense != b->dense_ffn) {          // the captured step runs other layers dense than the next one should
        (void)hipGraphExecDestroy(b->graph_exec); b->graph_exec = nullptr;
        if (b->graph) { (void)hipGraphDestroy(b->graph); b->graph = nullptr; }
    }
    if (use_graph && !b->graph_exec) {
        b->graph_dense = b->dense_ffn;
        PI_HIP_TRY(hipStreamBeginCapture(m->stream, hipStreamCaptureModeThreadLocal));
        const int rc = batch_step(m, m->batch);
        hipGraph_t g = nullptr;
        const hipError_t e = hipStreamEndCapture(m->stream, &g);
        if (rc != PI_OK) { if (g) (void)hipGraphDestroy(g); return rc; }
        if (e != hipSuccess) return pi::hip_fail(e, "hipStreamEndCapture");
        b->graph = g;
        PI_HIP_TRY(hipGraphInstantiate(&b->graph_exec, g, nullptr, nullptr, 0));
    }
    PI_HIP_TRY(hipEventRecord(m->ev0, m->stream));
    for (int s = 0; s < n_steps; ++s) {
        if (use_graph) PI_HIP_TRY(hipGraphLaunch(b->graph_exec, m->stream));
        else PI_TRY(batch_step(m, m->batch));
    }
    PI_HIP_TRY(hipEventRecord(m->ev1, m->stream));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    if (ms_out) PI_HIP_TRY(hipEventElapsedTime(ms_out, m->ev0, m->ev1));
    PI_TRY(pi_memcpy_d2h(out_tokens, b->d_out_tokens, sizeof(int32_t) * (size_t)n_steps * b->n_seq));
    return choose_dense_layers(m, b);
}

// llama_kv_cache_seq_rm / _seq_shift / _seq_cp for one sequence of the batch (llama.cpp:1757-1848).  Every sequence owns a cache,
// so "copy" really copies: cells [p0, p1) of src become the same cells of dst, which must hold exactly p0 cells (a shared prompt
// prefix is evaluated once and handed to the other sequences).
int pi_model_batch_kv_seq_rm(pi_model * m, int seq, int p0, int p1) {
    if (!m || !m->batch || seq < 0 || seq >= m->batch->n_seq) return pi::fail(PI_E_ARG, "pi_model_batch_kv_seq_rm: bad sequence");
    BatchState * b = m->batch;
    if ((int)b->kv_pos.size() != b->n_seq) b->kv_pos.resize(b->n_seq);
    return pi::kv_edit(m, b->k_cache + (size_t)seq * b->cache_seq_stride, b->v_cache + (size_t)seq * b->cache_seq_stride, b->d_pos + seq, b->kv_pos[seq], p0, p1, 0, false);
}

int pi_model_batch_kv_seq_shift(pi_model * m, int seq, int p0, int p1, int delta) {
    if (!m || !m->batch || seq < 0 || seq >= m->batch->n_seq) return pi::fail(PI_E_ARG, "pi_model_batch_kv_seq_shift: bad sequence");
    BatchState * b = m->batch;
    if ((int)b->kv_pos.size() != b->n_seq) b->kv_pos.resize(b->n_seq);
    return pi::kv_edit(m, b->k_cache + (size_t)seq * b->cache_seq_stride, b->v_cache + (size_t)seq * b->cache_seq_stride, b->d_pos + seq, b->kv_pos[seq], p0, p1, delta, true);
}

int pi_model_batch_kv_seq_cp(pi_model * m, int src, int dst, int p0, int p1) {
    if (!m || !m->batch || src < 0 || dst < 0 || src >= m->batch->n_seq || dst >= m->batch->n_seq || src == dst)
        return pi::fail(PI_E_ARG, "pi_model_batch_kv_seq_cp: bad sequences");
    BatchState * b = m->batch;
    if ((int)b->kv_pos.size() == b->n_seq && (!b->kv_pos[src].empty() || !b->kv_pos[dst].empty()))
        return pi::fail(PI_E_STATE, "pi_model_batch_kv_seq_cp: a sequence has non-contiguous cell positions");
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    std::vector<int32_t> pos(b->n_seq);
    PI_TRY(pi_memcpy_d2h(pos.data(), b->d_pos, sizeof(int32_t) * b->n_seq));
    if (p0 < 0) p0 = 0;
    if (p1 < 0 || p1 > pos[src]) p1 = pos[src];
    if (p1 < p0) return pi::fail(PI_E_ARG, "pi_model_batch_kv_seq_cp: empty range");
    if (pos[dst] != p0) return pi::fail(PI_E_UNSUPPORTED, "pi_model_batch_kv_seq_cp: the destination must hold exactly p0 cells");
    const int rows = m->hp.n_layer * m->hp.n_head_kv;
    const size_t pitch = (size_t)m->hp.n_ctx * m->hd * sizeof(__half), width = (size_t)(p1 - p0) * m->hd * sizeof(__half);
    if (width) {
        for (__half * base : {b->k_cache, b->v_cache})
            PI_HIP_TRY(hipMemcpy2DAsync(base + (size_t)dst * b->cache_seq_stride + (size_t)p0 * m->hd, pitch,
                                        base + (size_t)src * b->cache_seq_stride + (size_t)p0 * m->hd, pitch, width, rows, hipMemcpyDeviceToDevice, m->stream));
        PI_HIP_TRY(hipStreamSynchronize(m->stream));
    }
    const int32_t n = p1;
    PI_TRY(pi_memcpy_h2d(b->d_pos + dst, &n, 4));
    return p1;
}

// ---- one KV cache with cells shared between sequences ----------------------------------------------------------------------------
int pi_model_kv_cells_init(pi_model * m, int n_cells) {
    if (!m || !m->finalized) return pi::fail(PI_E_STATE, "pi_model_kv_cells_init: model not finalized");
    if (m->cells) return pi::fail(PI_E_STATE, "pi_model_kv_cells_init: already initialised");
    if (n_cells < 32 || n_cells % 32) return pi::fail(PI_E_ARG, "pi_model_kv_cells_init: n_cells must be a multiple of 32, at least 32");
    const bool q4_route = q4_steps_unsupported(m) == nullptr;
    if (!q4_route) if (const char * why = batch_unsupported(m)) { pi::set_error(why); return PI_E_UNSUPPORTED; }
    if (!pi_k_attn_ggml_supported(m->hd, n_cells, n_cells)) return pi::fail(PI_E_UNSUPPORTED, "pi_model_kv_cells_init: head size or cell count outside pi_k_attn_ggml");
    if (q4_route) PI_TRY(ensure_q4_split(m));
    BatchState * b = batch_alloc(m, 16, false);
    if (!b) return PI_E_HIP;
    b->unified = true;
    b->n_cells = n_cells;
    b->cell_pos.assign(n_cells, -1);
    b->cell_seq.assign(n_cells, 0u);
    b->cell_delta.assign(n_cells, 0);
    const size_t per_layer = (size_t)n_cells * m->gqa;
    b->cells_k = m->alloc<__half>(per_layer * m->hp.n_layer); b->cells_v = m->alloc<__half>(per_layer * m->hp.n_layer);
    b->cells_mask = m->alloc<float>((size_t)16 * n_cells); b->kq_scale = m->alloc<float>(1); b->d_delta = m->alloc<int32_t>(n_cells);
    if (!b->cells_k || !b->cells_v || !b->cells_mask || !b->kq_scale || !b->d_delta) { delete b; return PI_E_HIP; }
    const float scale = 1.0f / sqrtf((float)m->hd);
    PI_HIP_TRY(hipMemsetAsync(b->cells_k, 0, sizeof(__half) * per_layer * m->hp.n_layer, m->stream));
    PI_HIP_TRY(hipMemsetAsync(b->cells_v, 0, sizeof(__half) * per_layer * m->hp.n_layer, m->stream));
    PI_HIP_TRY(hipMemcpyAsync(b->kq_scale, &scale, 4, hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    m->cells = b;
    return PI_OK;
}

// llama_kv_cache_find_slot (llama.cpp:1683-1730): n contiguous free cells, searched from the ring's head, wrapping once
static bool cells_find_slot(BatchState * b, int n) {
    const int n_ctx = b->n_cells;
    if (n > n_ctx) return false;
    int n_tested = 0;
    while (true) {
        if (b->head + n > n_ctx) { n_tested += n_ctx - b->head; b->head = 0; continue; }
        bool found = true;
        for (int i = 0; i < n; ++i)
            if (b->cell_pos[b->head + i] >= 0) { found = false; b->head += i + 1; n_tested += i + 1; break; }
        if (found) return true;
        if (n_tested >= n_ctx) return false;
    }
}

int pi_model_kv_cells_decode(pi_model * m, const int32_t * tokens, const int32_t * positions, const uint32_t * seq_masks, int n_tokens,
                             int32_t * next_tokens, float * logits_out) {
    if (!m || !m->cells) return pi::fail(PI_E_STATE, "pi_model_kv_cells_decode: pi_model_kv_cells_init first");
    if (!tokens || !positions || !seq_masks || n_tokens < 1 || n_tokens > 16) return pi::fail(PI_E_ARG, "pi_model_kv_cells_decode: 1 <= n_tokens <= 16");
    BatchState * b = m->cells;
    for (int t = 0; t < n_tokens; ++t) {
        if (tokens[t] < 0 || tokens[t] >= m->hp.n_vocab) return pi::fail(PI_E_ARG, "pi_model_kv_cells_decode: token id out of range");
        if (positions[t] < 0 || seq_masks[t] == 0) return pi::fail(PI_E_ARG, "pi_model_kv_cells_decode: a token needs a position and at least one sequence");
    }
    if (!cells_find_slot(b, n_tokens)) return pi::fail(PI_E_STATE, "pi_model_kv_cells_decode: no run of free cells for the step (llama_kv_cache_find_slot failed)");
    for (int t = 0; t < n_tokens; ++t) {
        b->slot[t] = b->head + t;
        b->cell_pos[b->head + t] = positions[t];
        b->cell_seq[b->head + t] |= seq_masks[t];
    }
    // the cells a step looks at: up to the last one in use, at least 32 (llama_kv_cache_cell_max, llama.cpp:1735-1743, 6842)
    int cell_max = 0;
    for (int i = b->n_cells - 1; i > 0; --i) if (b->cell_pos[i] >= 0 && b->cell_seq[i]) { cell_max = i + 1; break; }
    b->n_kv = std::min(b->n_cells, std::max(32, cell_max));
    // mask rows (llama.cpp:6506-6531): a cell is hidden from token t unless it belongs to t's sequence and its position is not beyond t's
    std::vector<float> mask((size_t)n_tokens * b->n_cells, 0.0f);
    for (int t = 0; t < n_tokens; ++t) {
        const int seq = __builtin_ctz(seq_masks[t]);               // the reference masks by the token's first sequence id
        for (int i = 0; i < b->n_kv; ++i)
            if (!(b->cell_seq[i] >> seq & 1u) || b->cell_pos[i] > positions[t]) mask[(size_t)t * b->n_cells + i] = -INFINITY;
    }
    b->n_seq = n_tokens;
    if (b->has_shift) {          // pending position shifts: the K rows are rotated ahead of the step's layers (llm_build_k_shift runs first in the graph)
        PI_HIP_TRY(hipMemcpyAsync(b->d_delta, b->cell_delta.data(), sizeof(int32_t) * b->n_cells, hipMemcpyHostToDevice, m->stream));
        PI_HIP_TRY(hipStreamSynchronize(m->stream));
        PI_TRY(pi_k_k_shift_cells(b->cells_k, m->hp.n_layer, b->n_cells, m->hp.n_head_kv, m->hd, m->hp.arch == PI_ARCH_FALCON ? 2 : 0, m->theta_scale,
                                  m->freq_scale, b->d_delta, m->stream));
        b->has_shift = false;
        std::fill(b->cell_delta.begin(), b->cell_delta.end(), 0);
    }
    PI_HIP_TRY(hipMemcpyAsync(b->d_tokens, tokens, sizeof(int32_t) * n_tokens, hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipMemcpyAsync(b->d_pos, positions, sizeof(int32_t) * n_tokens, hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipMemcpyAsync(b->cells_mask, mask.data(), sizeof(float) * mask.size(), hipMemcpyHostToDevice, m->stream));
    PI_HIP_TRY(hipMemsetAsync(b->d_step, 0, 4, m->stream));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    PI_TRY(batch_step(m, b));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    b->head += n_tokens;                                          // llama_decode moves the ring's head past the step's cells and wraps it
    if (b->head >= b->n_cells) b->head = 0;                       // (llama.cpp:6936-6943)
    if (next_tokens) PI_TRY(pi_memcpy_d2h(next_tokens, b->d_tokens, sizeof(int32_t) * n_tokens));
    if (logits_out) PI_TRY(pi_memcpy_d2h(logits_out, b->logits, sizeof(float) * (size_t)n_tokens * m->hp.n_vocab));
    return PI_OK;
}

// llama_kv_cache_seq_rm (llama.cpp:1757-1785): seq < 0 removes the range from every sequence; p1 < 0: to the end
int pi_model_kv_cells_seq_rm(pi_model * m, int seq, int p0, int p1) {
    if (!m || !m->cells || seq >= 32) return pi::fail(PI_E_ARG, "pi_model_kv_cells_seq_rm: bad arguments");
    BatchState * b = m->cells;
    int new_head = b->n_cells;
    if (p0 < 0) p0 = 0;
    if (p1 < 0) p1 = INT32_MAX;
    for (int i = 0; i < b->n_cells; ++i) {
        if (b->cell_pos[i] >= p0 && b->cell_pos[i] < p1) {
            if (seq < 0) b->cell_seq[i] = 0;
            else if (b->cell_seq[i] >> seq & 1u) b->cell_seq[i] &= ~(1u << seq);
            else continue;
            if (b->cell_seq[i] == 0) { b->cell_pos[i] = -1; if (new_head == b->n_cells) new_head = i; }
        }
    }
    if (new_head != b->n_cells) b->head = new_head;
    return PI_OK;
}

// llama_kv_cache_seq_cp (llama.cpp:1787-1803): the cells of src in [p0, p1) join dst as well; nothing is copied
int pi_model_kv_cells_seq_cp(pi_model * m, int src, int dst, int p0, int p1) {
    if (!m || !m->cells || src < 0 || dst < 0 || src >= 32 || dst >= 32) return pi::fail(PI_E_ARG, "pi_model_kv_cells_seq_cp: bad arguments");
    BatchState * b = m->cells;
    if (p0 < 0) p0 = 0;
    if (p1 < 0) p1 = INT32_MAX;
    b->head = 0;
    for (int i = 0; i < b->n_cells; ++i)
        if ((b->cell_seq[i] >> src & 1u) && b->cell_pos[i] >= p0 && b->cell_pos[i] < p1) b->cell_seq[i] |= 1u << dst;
    return PI_OK;
}

// llama_kv_cache_seq_keep (llama.cpp:1805-1822)
int pi_model_kv_cells_seq_keep(pi_model * m, int seq) {
    if (!m || !m->cells || seq < 0 || seq >= 32) return pi::fail(PI_E_ARG, "pi_model_kv_cells_seq_keep: bad arguments");
    BatchState * b = m->cells;
    int new_head = b->n_cells;
    for (int i = 0; i < b->n_cells; ++i) {
        if (!(b->cell_seq[i] >> seq & 1u)) { b->cell_pos[i] = -1; b->cell_seq[i] = 0; if (new_head == b->n_cells) new_head = i; }
        else b->cell_seq[i] = 1u << seq;
    }
    if (new_head != b->n_cells) b->head = new_head;
    return PI_OK;
}

// llama_kv_cache_seq_shift (llama.cpp:1824-1848): the positions move now, the K rows at the start of the next step
int pi_model_kv_cells_seq_shift(pi_model * m, int seq, int p0, int p1, int delta) {
    if (!m || !m->cells || seq < 0 || seq >= 32) return pi::fail(PI_E_ARG, "pi_model_kv_cells_seq_shift: bad arguments");
    BatchState * b = m->cells;
    int new_head = b->n_cells;
    if (p0 < 0) p0 = 0;
    if (p1 < 0) p1 = INT32_MAX;
    for (int i = 0; i < b->n_cells; ++i) {
        if ((b->cell_seq[i] >> seq & 1u) && b->cell_pos[i] >= p0 && b->cell_pos[i] < p1) {
            b->has_shift = true;
            b->cell_pos[i] += delta;
            b->cell_delta[i] += delta;
            if (b->cell_pos[i] < 0) { b->cell_pos[i] = -1; b->cell_seq[i] = 0; if (new_head == b->n_cells) new_head = i; }
        }
    }
    b->head = new_head != b->n_cells ? new_head : 0;
    return PI_OK;
}

// llama_kv_cache_clear (llama.cpp:1745-1751)
int pi_model_kv_cells_clear(pi_model * m) {
    if (!m || !m->cells) return pi::fail(PI_E_ARG, "pi_model_kv_cells_clear: bad arguments");
    BatchState * b = m->cells;
    std::fill(b->cell_pos.begin(), b->cell_pos.end(), -1);
    std::fill(b->cell_seq.begin(), b->cell_seq.end(), 0u);
    b->head = 0;
    return PI_OK;
}

int pi_model_kv_cells_state(pi_model * m, int32_t * cell_pos, uint32_t * cell_seq, int32_t * head) {
    if (!m || !m->cells) return pi::fail(PI_E_ARG, "pi_model_kv_cells_state: bad arguments");
    BatchState * b = m->cells;
    if (cell_pos) memcpy(cell_pos, b->cell_pos.data(), sizeof(int32_t) * b->n_cells);
    if (cell_seq) memcpy(cell_seq, b->cell_seq.data(), sizeof(uint32_t) * b->n_cells);
    if (head) *head = b->head;
    return b->n_cells;
}

int pi_model_batch_union(pi_model * m, int32_t * n_union_per_layer) {
    if (!m || !m->batch || !n_union_per_layer) return pi::fail(PI_E_ARG, "pi_model_batch_union: bad arguments");
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    return pi_memcpy_d2h(n_union_per_layer, m->batch->n_union, sizeof(int32_t) * m->hp.n_layer);
}

}  // extern "C"

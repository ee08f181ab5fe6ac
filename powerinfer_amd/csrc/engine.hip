// Decode loop with resident weights: the per-token operator sequence that llama.cpp builds as a ggml graph
// (build_llama_variants, llama.cpp:4949-5084; build_falcon, llama.cpp:5326-5468; llm_build_ffn_sparse,
// llama.cpp:4652-4757) issued as a fixed chain of fused HIP kernels on one stream and, for the greedy
// token loop, captured once into a HIP graph and replayed per token (the reference rebuilds and walks a
// ~40-node-per-layer graph every token, llama.cpp:6408, 6922).
#include "runtime.hpp"
#include "cold_path.hpp"
#include <limits.h>
#include "engine_internal.hpp"
#include "../../include/powerinfer_hip.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <utility>
#include <vector>

namespace {

size_t row_bytes(int type, int64_t ne0) {
    switch (type) {
        case PI_TYPE_F32: case PI_TYPE_I32: return (size_t)ne0 * 4;
        case PI_TYPE_F16:  return (size_t)ne0 * 2;
        case PI_TYPE_Q4_0: return (size_t)(ne0 / 32) * 18;
        default: return 0;
    }
}

__global__ void set_state_kernel(int32_t * token, int32_t * pos, int32_t t, int32_t p) {
    if (threadIdx.x == 0) { *token = t; *pos = p; }
}

// greedy choice of the finished step + bookkeeping for the next one: the chosen token becomes the next
// input, the position advances, the token and the step's total active-row count are logged
__global__ __launch_bounds__(1024) void argmax_advance_kernel(const float * __restrict__ logits, int n, int32_t * token, int32_t * pos,
                                                              int32_t * step, int32_t * out_tokens, int32_t * out_active,
                                                              const int32_t * __restrict__ n_active, int n_layer, int max_steps) {
    __shared__ float bv[16];
    __shared__ int   bi[16];
    __shared__ int stot;
    float best = -INFINITY; int idx = n;
    // the bookkeeping operands are requested with the logits: one memory round trip for the whole kernel at vocabularies up to 32 K
    int act = 0;
    for (int l = threadIdx.x; l < n_layer; l += blockDim.x) act += n_active[l];
    const int s_in = *step, p_in = *pos;
    for (int base = 0; base < n; base += 8 * 4 * 1024) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = base + (u * 1024 + (int)threadIdx.x) * 4;
            if (i + 3 < n) v[u] = *reinterpret_cast<const float4 *>(logits + i);
            else v[u] = make_float4(i < n ? logits[i] : -INFINITY, i + 1 < n ? logits[i + 1] : -INFINITY, i + 2 < n ? logits[i + 2] : -INFINITY, -INFINITY);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = base + (u * 1024 + (int)threadIdx.x) * 4;
            if (v[u].x > best) { best = v[u].x; idx = i; }
            if (v[u].y > best) { best = v[u].y; idx = i + 1; }
            if (v[u].z > best) { best = v[u].z; idx = i + 2; }
            if (v[u].w > best) { best = v[u].w; idx = i + 3; }
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(idx, o, 64);
        if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (wave == 0) {                       // n_layer <= 1024 entries were spread over the threads; at most a few waves hold non-zeros
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) act += __shfl_xor(act, o, 64);
    }
    if (threadIdx.x == 0) stot = 0;
    if (lane == 0) { bv[wave] = best; bi[wave] = idx; }
    __syncthreads();
    if (wave != 0 && act != 0) atomicAdd(&stot, act);      // layers beyond the first 64 (LDS atomic, integer: order does not matter)
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); ++w)
            if (bv[w] > best || (bv[w] == best && bi[w] < idx)) { best = bv[w]; idx = bi[w]; }
        if (idx >= n) idx = 0;
        const int tot = act + stot;
        const int s = s_in;
        if (s < max_steps) { out_tokens[s] = idx; out_active[s] = tot; }
        *token = idx;
        *pos = p_in + 1;
        *step = s + 1;
    }
}

// dst row i = src row perm[i]; rows of row_bytes (a multiple of 16) bytes, one workgroup per row
__global__ __launch_bounds__(256) void gather_rows_kernel(const unsigned char * __restrict__ src, unsigned char * __restrict__ dst,
                                                          const int32_t * __restrict__ perm, size_t row_bytes) {
    const uint4 * s = reinterpret_cast<const uint4 *>(src + (size_t)perm[blockIdx.x] * row_bytes);
    uint4 * d = reinterpret_cast<uint4 *>(dst + (size_t)blockIdx.x * row_bytes);
    for (size_t i = threadIdx.x; i < row_bytes / 16; i += blockDim.x) d[i] = s[i];
}

__global__ void add_vec_kernel(float * __restrict__ y, const float * __restrict__ a, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = __fadd_rn(y[i], a[i]);
}

}  // namespace

namespace {

int upload_tensor(pi_model * m, Tensor & t, int type, const void * data, int64_t ne0, int64_t ne1, int on_device) {
    const size_t bytes = row_bytes(type, ne0) * (size_t)ne1;
    if (bytes == 0) return pi::fail(PI_E_ARG, "pi_model_set_tensor: unsupported type or empty tensor");
    t.type = type; t.ne0 = ne0; t.ne1 = ne1;
    if (on_device) { t.dev = const_cast<void *>(data); t.owned = false; return PI_OK; }
    t.dev = m->alloc<unsigned char>(bytes);
    if (!t.dev) return PI_E_HIP;
    t.owned = true;
    return pi_memcpy_h2d(t.dev, data, bytes);
}

bool hp_arch_is_falcon(const pi_model * m) { return m->hp.arch == PI_ARCH_FALCON; }

bool is_ffn_matrix(int kind) { return kind == PI_T_FFN_GATE || kind == PI_T_FFN_UP || kind == PI_T_FFN_DOWN_T; }

pi_norm make_norm(int kind, float eps, const Tensor & w, const Tensor * b) {
    pi_norm n{kind, eps, (const float *)w.dev, b ? (const float *)b->dev : nullptr};
    return n;
}

#define PI_TRY(expr) do { int _rc = (expr); if (_rc != PI_OK) return _rc; } while (0)

// ---- one layer, everything on the GPU --------------------------------------------------------------
int layer_forward(pi_model * m, int il, bool last_token) {
    const pi_hparams & hp = m->hp;
    const int d = hp.n_embd, ff = hp.n_ff, hd = m->hd, gqa = m->gqa;
    hipStream_t st = m->stream;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    Tensor & wqkv = m->L(il, PI_T_WQKV);
    Tensor & wo = m->L(il, PI_T_WO);
    Tensor & fc1 = m->L(il, PI_T_FC1);
    Tensor & fc2 = m->L(il, PI_T_FC2);
    Tensor & up = m->L(il, PI_T_FFN_UP);
    Tensor & gate = m->L(il, PI_T_FFN_GATE);
    Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    Tensor & bucket = m->L(il, PI_T_GPU_BUCKET);
    const int r = (int)fc1.ne1;
    const size_t kv_off = (size_t)il * hp.n_head_kv * hp.n_ctx * hd;
    int32_t * n_act = m->n_active + il;
    const int32_t * bk = (const int32_t *)bucket.dev;
    const int n_bucket = bk ? (int)bucket.ne0 : 0;
    const bool q4 = up.type == PI_TYPE_Q4_0;
    const bool layer_hybrid = bk != nullptr;
    float * x = m->x;

    const bool branch = falcon && m->stream2 && !layer_hybrid && !q4 && !m->capture && pi_k_sparse_ffn_supported(ff, r, d);
    if (branch) {
        pi_norm fnb = make_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B));
        PI_HIP_TRY(hipEventRecord(m->ev_fork[il], st));
        PI_HIP_TRY(hipStreamWaitEvent(m->stream2, m->ev_fork[il], 0));
        PI_TRY(pi_k_gemv(fc1.type, fc1.dev, r, d, x, nullptr, PI_EPI_RELU, nullptr, nullptr, m->hidden, m->stream2));
        PI_TRY(pi_k_sparse_ffn_partials(fc2.dev, ff, r, m->hidden, hp.sparse_threshold, up.dev, nullptr, down.dev, d, x, &fnb,
                                               nullptr, nullptr, m->ws, m->stream2));
    }

    // attention
    pi_norm an;
    if (!falcon) an = make_norm(1, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), nullptr);
    else if (m->L(il, PI_T_ATTN_NORM_2).dev) an = make_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM_2), &m->L(il, PI_T_ATTN_NORM_2_B));
    else an = make_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B));
    PI_TRY(pi_k_gemv(wqkv.type, wqkv.dev, d + 2 * gqa, d, x, &an, PI_EPI_NONE, nullptr, nullptr, m->qkv, st));
    if (m->attn_parts > 1) {
        PI_TRY(pi_k_attn_split(m->qkv, 0, m->rope_table, m->k_cache + kv_off, m->v_cache + kv_off, 0, 1, hp.n_head, hp.n_head_kv, hd, falcon ? 2 : 0,
                               hp.n_ctx, m->attn_parts, m->d_pos, m->attn_scratch, m->att, 0, nullptr, st));
    } else if (m->rope_table) {
        PI_TRY(pi_k_attn_fused(m->qkv, m->rope_table, m->k_cache + kv_off, m->v_cache + kv_off, hp.n_head, hp.n_head_kv, hd, falcon ? 2 : 0,
                               hp.n_ctx, m->d_pos, m->att, st));
    } else {
        PI_TRY(pi_k_rope_kv_store(m->qkv, hp.n_head, hp.n_head_kv, hd, falcon ? 2 : 0, m->theta_scale, m->freq_scale, m->d_pos, hp.n_ctx,
                                  m->q_rot, m->k_cache + kv_off, m->v_cache + kv_off, st));
        PI_TRY(pi_k_attn_decode(m->q_rot, m->k_cache + kv_off, m->v_cache + kv_off, hp.n_head, hp.n_head_kv, hd, hp.n_ctx, m->d_pos, m->att, st));
    }

    const float * pred_in; const float * ffn_in; pi_norm fn;
    if (!falcon) {
        // ffn_inp = wo.att + x   (ggml_add(cur, inpSA), llama.cpp:5022)
        PI_TRY(pi_k_gemv(wo.type, wo.dev, d, d, m->att, nullptr, PI_EPI_ADD, x, nullptr, m->ffn_inp, st));
        pred_in = m->ffn_inp; ffn_in = m->ffn_inp;
        fn = make_norm(1, hp.norm_eps, m->L(il, PI_T_FFN_NORM), nullptr);
    } else {
        PI_TRY(pi_k_gemv(wo.type, wo.dev, d, d, m->att, nullptr, PI_EPI_NONE, nullptr, nullptr, m->attn_out, st));
        pred_in = x; ffn_in = x;                       // Falcon: predictor sees the layer input, FFN sees attn_norm(layer input)
        fn = make_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B));
    }

    // predictor
    if (!branch) PI_TRY(pi_k_gemv(fc1.type, fc1.dev, r, d, pred_in, nullptr, PI_EPI_RELU, nullptr, nullptr, m->hidden, st));
    if (branch) {
        // Falcon's attention and FFN both read the layer input: the predictor + sparse FFN partials run on a second stream
        // beside q|k|v -> attention -> wo, and only the final reduction (FFN + attention output + input) waits for both
        PI_HIP_TRY(hipEventRecord(m->ev_join[il], m->stream2));
        PI_HIP_TRY(hipStreamWaitEvent(st, m->ev_join[il], 0));
        PI_TRY(pi_k_sparse_ffn_reduce(ff, d, PI_EPI_ADD2, m->attn_out, x, m->x2, n_act, m->ws, st));
        std::swap(m->x, m->x2);
        return PI_OK;
    }
    if (!layer_hybrid && !q4 && pi_k_sparse_ffn_supported(ff, r, d)) {
        // one launch for fc2 + mask + gate/up + each workgroup's share of the down projection, one small reduction
        const void * gp = falcon ? nullptr : gate.dev;
        if (m->capture && last_token) {
            float * ffo = m->cap_ffn + (size_t)il * d;
            PI_TRY(pi_k_sparse_ffn(fc2.dev, ff, r, m->hidden, hp.sparse_threshold, up.dev, gp, down.dev, d, ffn_in, &fn,
                                          PI_EPI_NONE, nullptr, nullptr, ffo, m->pred_logits, nullptr, n_act, m->ws, st));
            PI_HIP_TRY(hipMemcpyAsync(m->x2, ffo, sizeof(float) * d, hipMemcpyDeviceToDevice, st));
            PI_TRY(pi::add_vec(m->x2, falcon ? m->attn_out : m->ffn_inp, d, st));
            if (falcon) PI_TRY(pi::add_vec(m->x2, x, d, st));
            PI_HIP_TRY(hipMemcpyAsync(m->cap_logits + (size_t)il * ff, m->pred_logits, sizeof(float) * ff, hipMemcpyDeviceToDevice, st));
            PI_HIP_TRY(hipMemcpyAsync(m->cap_src + (size_t)il * d, ffn_in, sizeof(float) * d, hipMemcpyDeviceToDevice, st));
        } else if (!falcon) {
            PI_TRY(pi_k_sparse_ffn(fc2.dev, ff, r, m->hidden, hp.sparse_threshold, up.dev, gp, down.dev, d, ffn_in, &fn,
                                          PI_EPI_ADD, m->ffn_inp, nullptr, m->x2, nullptr, nullptr, n_act, m->ws, st));
        } else {
            PI_TRY(pi_k_sparse_ffn(fc2.dev, ff, r, m->hidden, hp.sparse_threshold, up.dev, gp, down.dev, d, ffn_in, &fn,
                                          PI_EPI_ADD2, m->attn_out, x, m->x2, nullptr, nullptr, n_act, m->ws, st));
        }
        std::swap(m->x, m->x2);
        return PI_OK;
    }
    if (layer_hybrid && !q4 && m->hot_words[il] && up.type == PI_TYPE_F16 && fc2.type == PI_TYPE_F16 && pi_k_sparse_ffn_hot_supported(ff, r, d)) {
        // F16 hybrid layer at a width the fused kernels cover: the resident share's whole FFN is one launch, the host share works
        // from the pinned buffers it fills, the reduction merges both
        const bool cap = m->capture && last_token;
        if (pi::cold_layer_async(m->cold, il) && !m->capture) PI_TRY(pi::cold_layer_f16_queue(m->cold, il, m, st));
        else PI_TRY(pi::cold_layer_f16(m->cold, il, m, st, cap));
        if (cap) PI_HIP_TRY(hipMemcpyAsync(m->cap_src + (size_t)il * d, ffn_in, sizeof(float) * d, hipMemcpyDeviceToDevice, st));
        std::swap(m->x, m->x2);
        return PI_OK;
    }
    if (q4 && fc2.type == PI_TYPE_F16 && pi_k_pred_upgate_q4_supported(ff, r, d) && (!layer_hybrid || m->hot_words[il])) {
        // Q4_0 at d = 4096: fc2 + mask + up/gate of the resident neurons in one launch, the down projection as partial vectors
        // plus one reduction; a hybrid layer's host share works between the two from the buffers the first kernel fills
        const void * gp = falcon ? nullptr : gate.dev;
        const bool cap = m->capture && last_token;
        if (layer_hybrid && !m->rest_on_gpu) {
            // nothing is launched between the two halves unless the parity hooks are on: the stream waits for the host threads itself
            if (pi::cold_layer_async(m->cold, il) && !m->capture) PI_TRY(pi::cold_layer_q4_queue(m->cold, il, m, st));
            else PI_TRY(pi::cold_layer_q4(m->cold, il, m, st, cap));
        } else {
            // every neuron on the GPU, or the non-resident neurons' rows read from pinned host memory: one launch carries the predictor,
            // the up/gate rows and - a workgroup's 32 neurons being one Q8_0 block of h - the down rows; then the reduction
            const uint32_t * hw = layer_hybrid ? m->hot_words[il] : nullptr;
            const int32_t * hpx = layer_hybrid ? m->hot_prefix[il] : nullptr;
            PI_TRY(pi_k_sparse_ffn_q4_partials(fc2.dev, ff, r, m->hidden, hp.sparse_threshold, up.dev, gp, down.dev,
                                               layer_hybrid ? m->rest_up[il] : nullptr, (layer_hybrid && !falcon) ? m->rest_gate[il] : nullptr,
                                               layer_hybrid ? m->rest_down[il] : nullptr, d, ffn_in, &fn, hw, hpx, m->pred_logits, m->h_dense, m->ws, st));
            if (cap) {
                float * ffo = m->cap_ffn + (size_t)il * d;
                PI_TRY(pi_k_sparse_ffn_q4_reduce(ff, d, PI_EPI_NONE, nullptr, nullptr, ffo, n_act, m->ws, st));
                PI_HIP_TRY(hipMemcpyAsync(m->x2, ffo, sizeof(float) * d, hipMemcpyDeviceToDevice, st));
                PI_TRY(pi::add_vec(m->x2, falcon ? m->attn_out : m->ffn_inp, d, st));
                if (falcon) PI_TRY(pi::add_vec(m->x2, x, d, st));
                PI_HIP_TRY(hipMemcpyAsync(m->cap_logits + (size_t)il * ff, m->pred_logits, sizeof(float) * ff, hipMemcpyDeviceToDevice, st));
            } else if (!falcon) {
                PI_TRY(pi_k_sparse_ffn_q4_reduce(ff, d, PI_EPI_ADD, m->ffn_inp, nullptr, m->x2, n_act, m->ws, st));
            } else {
                PI_TRY(pi_k_sparse_ffn_q4_reduce(ff, d, PI_EPI_ADD2, m->attn_out, x, m->x2, n_act, m->ws, st));
            }
        }
        if (cap) PI_HIP_TRY(hipMemcpyAsync(m->cap_src + (size_t)il * d, ffn_in, sizeof(float) * d, hipMemcpyDeviceToDevice, st));
        std::swap(m->x, m->x2);
        return PI_OK;
    }
    // F16 layers that live entirely on the GPU take the fused route: the up/gate kernel reads the mask words itself
    const bool fused = !layer_hybrid && !q4;
    const int n_rows = layer_hybrid ? n_bucket : ff;
    PI_TRY(pi_k_predictor_fc2(fc2.dev, ff, r, m->hidden, hp.sparse_threshold, bk, n_bucket, m->pred_logits,
                              fused ? nullptr : m->list, fused ? nullptr : n_act,
                              (q4 || layer_hybrid) ? m->h_dense : nullptr, m->ws, st));
    if (layer_hybrid) PI_TRY(pi::cold_stage_inputs(m->cold, il, m, st));

    // sparse FFN, GPU share
    PI_TRY(pi_k_sparse_upgate(up.type, up.dev, falcon ? nullptr : gate.dev, d, ff, ffn_in, &fn, fused ? 1 : 0, m->list, n_act, bk, m->h_c,
                              (q4 || layer_hybrid) ? m->h_dense : nullptr, nullptr, nullptr, m->ws, st));

    if (!layer_hybrid && m->capture && last_token) {
        // parity hook: keep the bare FFN output, then add the residuals in the reference's order
        float * ffo = m->cap_ffn + (size_t)il * d;
        PI_TRY(pi_k_sparse_axpy(down.type, down.dev, d, n_rows, m->h_c, q4 ? m->h_dense : nullptr, nullptr, m->list, n_act,
                                PI_EPI_NONE, nullptr, nullptr, ffo, m->ws, st));
        PI_HIP_TRY(hipMemcpyAsync(m->x2, ffo, sizeof(float) * d, hipMemcpyDeviceToDevice, st));
        PI_TRY(pi::add_vec(m->x2, falcon ? m->attn_out : m->ffn_inp, d, st));
        if (falcon) PI_TRY(pi::add_vec(m->x2, x, d, st));
    } else if (!layer_hybrid) {
        if (!falcon) PI_TRY(pi_k_sparse_axpy(down.type, down.dev, d, n_rows, m->h_c, q4 ? m->h_dense : nullptr, nullptr, m->list, n_act,
                                             PI_EPI_ADD, m->ffn_inp, nullptr, m->x2, m->ws, st));
        else         PI_TRY(pi_k_sparse_axpy(down.type, down.dev, d, n_rows, m->h_c, q4 ? m->h_dense : nullptr, nullptr, m->list, n_act,
                                             PI_EPI_ADD2, m->attn_out, x, m->x2, m->ws, st));
    } else {
        // hot/cold merge (llm_build_sparse_mul_mat / llm_build_sparse_axpy hybrid variants, llama.cpp:4581-4593, 4635-4646)
        PI_TRY(pi::cold_layer_merge(m->cold, il, m, st));
    }
    std::swap(m->x, m->x2);

    if (m->capture && last_token) {
        PI_HIP_TRY(hipMemcpyAsync(m->cap_logits + (size_t)il * ff, m->pred_logits, sizeof(float) * ff, hipMemcpyDeviceToDevice, st));
        PI_HIP_TRY(hipMemcpyAsync(m->cap_src + (size_t)il * d, ffn_in, sizeof(float) * d, hipMemcpyDeviceToDevice, st));
    }
    return PI_OK;
}

// one token: embedding -> layers -> (final norm + lm-head + greedy)
int token_forward(pi_model * m, bool want_logits, bool last_token) {
    const pi_hparams & hp = m->hp;
    hipStream_t st = m->stream;
    // the host threads expect this token's hybrid layers (a graph under construction runs nothing: its replays are announced one by one)
    if (pi::cold_async(m->cold) && !m->capture && !m->building_graph) PI_TRY(pi::cold_post_token(m->cold));
    PI_TRY(pi_k_embed(m->glob[PI_T_TOK_EMBD].type, m->glob[PI_T_TOK_EMBD].dev, hp.n_embd, m->d_token, m->x, st));
    for (int il = 0; il < hp.n_layer; ++il) PI_TRY(layer_forward(m, il, last_token));
    if (want_logits) {
        const bool falcon = hp.arch == PI_ARCH_FALCON;
        pi_norm on = make_norm(falcon ? 2 : 1, hp.norm_eps, m->glob[PI_T_OUTPUT_NORM], falcon ? &m->glob[PI_T_OUTPUT_NORM_B] : nullptr);
        PI_TRY(pi_k_gemv(m->glob[PI_T_OUTPUT].type, m->glob[PI_T_OUTPUT].dev, hp.n_vocab, hp.n_embd, m->x, &on, PI_EPI_NONE, nullptr, nullptr, m->logits, st));
    }
    return PI_OK;
}

int launch_advance(pi_model * m) {
    hipLaunchKernelGGL(argmax_advance_kernel, dim3(1), dim3(1024), 0, m->stream, m->logits, m->hp.n_vocab, m->d_token, m->d_pos, m->d_step,
                       m->d_out_tokens, m->d_out_active, m->n_active, m->hp.n_layer, m->max_steps);
    return pi::check_launch("argmax_advance");
}

}  // namespace

namespace {
__global__ void merge_shares_kernel(float * __restrict__ dst, const float * cold, const float * hot, const float * __restrict__ r1,
                                    const float * __restrict__ r2, float * __restrict__ keep, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = __fadd_rn(cold[i], hot[i]);
    if (keep) keep[i] = v;
    v = __fadd_rn(v, r1[i]);
    if (r2) v = __fadd_rn(v, r2[i]);
    dst[i] = v;
}
}  // namespace

// entries used by the cold path to add its share into the layer output on the model's stream
namespace pi {
int merge_shares(float * dst, const float * cold, const float * hot, const float * r1, const float * r2, float * keep, int n, hipStream_t st) {
    hipLaunchKernelGGL(merge_shares_kernel, dim3((n + 255) / 256), dim3(256), 0, st, dst, cold, hot, r1, r2, keep, n);
    return check_launch("merge_shares");
}
int add_vec(float * y, const float * a, int n, hipStream_t st) {
    hipLaunchKernelGGL(add_vec_kernel, dim3((n + 255) / 256), dim3(256), 0, st, y, a, n);
    return check_launch("add_vec");
}
}  // namespace pi

namespace pi {
// One edit of a sequence's cache (k, v: [n_layer * n_head_kv][n_ctx][hd]; d_pos: the device word holding its next position;
// kv_pos: the cells' positions while they are not 0 .. n-1): cells whose position lies in [p0, p1) are dropped (!shift) or moved
// by delta positions (dropped if that takes them below 0).  Returns the number of live cells, or a negative error.
int kv_edit(pi_model * m, __half * k_cache, __half * v_cache, int32_t * d_pos, std::vector<int32_t> & kv_pos, int p0, int p1, int delta, bool shift) {
    const pi_hparams & hp = m->hp;
    hipStream_t st = m->stream;
    PI_HIP_TRY(hipStreamSynchronize(st));
    if (kv_pos.empty()) {
        int32_t n = 0;
        PI_TRY(pi_memcpy_d2h(&n, d_pos, 4));
        if (n < 0 || n > hp.n_ctx) return pi::fail(PI_E_STATE, "KV edit: the device position is out of range");
        kv_pos.resize(n);
        for (int i = 0; i < n; ++i) kv_pos[i] = i;
    }
    if (p0 < 0) p0 = 0;
    if (p1 < 0) p1 = INT32_MAX;
    const int n_old = (int)kv_pos.size();
    std::vector<int32_t> dl(n_old ? n_old : 1, 0), map, pos;
    bool any_shift = false;
    for (int i = 0; i < n_old; ++i) {
        int p = kv_pos[i];
        if (p >= p0 && p < p1) {
            if (!shift) continue;                     // removed
            p += delta;
            if (p < 0) continue;                      // shifted out (llama.cpp:1836-1840)
            dl[i] = delta; any_shift = any_shift || delta != 0;
        }
        map.push_back(i); pos.push_back(p);
    }
    const int n_new = (int)map.size();
    const int rows = hp.n_layer * hp.n_head_kv;
    if (!m->kv_map) { m->kv_map = m->alloc<int32_t>(hp.n_ctx); if (!m->kv_map) return PI_E_HIP; }
    if (any_shift) {
        PI_TRY(pi_memcpy_h2d(m->kv_map, dl.data(), sizeof(int32_t) * n_old));
        PI_TRY(pi_k_k_shift(k_cache, rows, hp.n_ctx, m->hd, hp.arch == PI_ARCH_FALCON ? 2 : 0, m->theta_scale, m->freq_scale, m->kv_map, n_old, st));
        PI_HIP_TRY(hipStreamSynchronize(st));
    }
    bool moved = false;
    for (int j = 0; j < n_new; ++j) moved = moved || map[j] != j;
    if (moved) {
        if (!m->kv_stage) { m->kv_stage = m->alloc<__half>((size_t)rows * hp.n_ctx * m->hd); if (!m->kv_stage) return PI_E_HIP; }
        PI_TRY(pi_memcpy_h2d(m->kv_map, map.data(), sizeof(int32_t) * n_new));
        PI_TRY(pi_k_kv_compact(k_cache, m->kv_stage, rows, hp.n_ctx, m->hd, m->kv_map, n_new, st));
        PI_TRY(pi_k_kv_compact(v_cache, m->kv_stage, rows, hp.n_ctx, m->hd, m->kv_map, n_new, st));
        PI_HIP_TRY(hipStreamSynchronize(st));
    }
    bool identity = true;
    for (int j = 0; j < n_new; ++j) identity = identity && pos[j] == j;
    if (identity) {
        kv_pos.clear();
        const int32_t n = n_new;
        PI_TRY(pi_memcpy_h2d(d_pos, &n, 4));          // generation continues at position n
    } else {
        kv_pos = pos;
    }
    return n_new;
}
}  // namespace pi

extern "C" {

pi_model * pi_model_create(const pi_hparams * hp) {
    if (!hp || hp->n_embd <= 0 || hp->n_ff <= 0 || hp->n_head <= 0 || hp->n_head_kv <= 0 || hp->n_layer <= 0 || hp->n_vocab <= 0 || hp->n_ctx <= 0 ||
        hp->n_embd % hp->n_head || hp->n_head % hp->n_head_kv || (hp->arch != PI_ARCH_LLAMA && hp->arch != PI_ARCH_FALCON)) {
        pi::set_error("pi_model_create: inconsistent hyper-parameters");
        return nullptr;
    }
    if (pi_init(0) != PI_OK) return nullptr;
    pi_model * m = new pi_model();
    m->hp = *hp;
    m->hd = hp->n_embd / hp->n_head;
    m->gqa = m->hd * hp->n_head_kv;
    m->layers.resize((size_t)hp->n_layer * PI_T_COUNT);
    m->theta_scale = powf(hp->rope_freq_base, -2.0f / (float)m->hd);       // ggml.c:11196
    m->freq_scale = hp->rope_freq_scale == 0.0f ? 1.0f : hp->rope_freq_scale;
    return m;
}

void pi_model_free(pi_model * m) {
    if (!m) return;
    if (m->graph_exec) (void)hipGraphExecDestroy(m->graph_exec);
    if (m->graph) (void)hipGraphDestroy(m->graph);
    if (m->ev0) (void)hipEventDestroy(m->ev0);
    if (m->ev1) (void)hipEventDestroy(m->ev1);
    for (hipEvent_t e : m->ev_fork) if (e) (void)hipEventDestroy(e);
    for (hipEvent_t e : m->ev_join) if (e) (void)hipEventDestroy(e);
    if (m->stream2) (void)hipStreamDestroy(m->stream2);
    if (m->cold) pi::cold_destroy(m->cold);
    pi::batch_destroy(m);
    if (m->ws) pi_workspace_destroy(m->ws);
    for (void * p : m->owned) pi_free(p);
    for (void * p : m->pinned) (void)hipHostFree(p);
    if (m->stream) (void)hipStreamDestroy(m->stream);
    delete m;
}

int pi_model_set_tensor(pi_model * m, int layer, int kind, int type, const void * data, int64_t ne0, int64_t ne1, int on_device) {
    if (!m || !data || kind < 0 || kind >= PI_T_COUNT || ne0 <= 0 || ne1 <= 0) return pi::fail(PI_E_ARG, "pi_model_set_tensor: bad arguments");
    if (m->finalized) return pi::fail(PI_E_STATE, "pi_model_set_tensor: model already finalized");
    if (kind <= PI_T_OUTPUT) return upload_tensor(m, m->glob[kind], type, data, ne0, ne1, on_device);
    if (layer < 0 || layer >= m->hp.n_layer) return pi::fail(PI_E_ARG, "pi_model_set_tensor: layer out of range");
    Tensor & t = m->L(layer, kind);
    if (is_ffn_matrix(kind) && !on_device) {
        // sliced at finalize if the layer turns out to have a GPU bucket; remember the host copy until then
        t.type = type; t.ne0 = ne0; t.ne1 = ne1; t.host = data;
        return PI_OK;
    }
    if (kind == PI_T_GPU_IDX) { t.type = type; t.ne0 = ne0; t.ne1 = ne1; t.host = data; return PI_OK; }   // host-only (cold path)
    if (kind == PI_T_NEURON_RATE) {                                                                       // host-only, copied (finalize)
        if (type != PI_TYPE_F32 || on_device || ne0 * ne1 != m->hp.n_ff) return pi::fail(PI_E_ARG, "pi_model_set_tensor: neuron rates are host F32 [n_ff]");
        if (m->neuron_rate.empty()) m->neuron_rate.resize(m->hp.n_layer);
        m->neuron_rate[layer].assign((const float *)data, (const float *)data + m->hp.n_ff);
        return PI_OK;
    }
    if (kind == PI_T_GPU_BUCKET) { t.host = data; }
    return upload_tensor(m, t, type, data, ne0, ne1, on_device);
}

}  // extern "C"

namespace {
// Deals the neurons of layer il out by firing rate over the workgroups of the fused F16 launch: the workgroup ranges take the neurons of
// rank 0, 1, 2, ... in turn (first slot of every range, then the second, ...), so each range holds the same mix of busy and idle neurons
// and every workgroup expects the same number of active rows.  fc2 / up / gate / down_t rows move alike into storage the model owns.
int deal_neurons_by_rate(pi_model * m, int il) {
    const pi_hparams & hp = m->hp;
    const int d = hp.n_embd, ff = hp.n_ff;
    const std::vector<float> & rate = m->neuron_rate[il];
    Tensor & fc2 = m->L(il, PI_T_FC2); Tensor & up = m->L(il, PI_T_FFN_UP);
    if (rate.empty() || m->L(il, PI_T_GPU_BUCKET).dev || up.type != PI_TYPE_F16 || fc2.type != PI_TYPE_F16) return PI_OK;
    const int n_wg = pi_k_sparse_ffn_workgroups(ff, (int)fc2.ne0, d);
    if (n_wg <= 0) return PI_OK;
    std::vector<int32_t> order(ff);
    for (int i = 0; i < ff; ++i) order[i] = i;
    std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return rate[a] > rate[b]; });
    std::vector<int32_t> & perm = m->ffn_perm[il];
    perm.resize(ff);
    int next = 0;
    for (int j = 0; next < ff; ++j)
        for (int b = 0; b < n_wg; ++b) {
            const int lo = (int)((long long)ff * b / n_wg), hi = (int)((long long)ff * (b + 1) / n_wg);
            if (lo + j < hi) perm[lo + j] = order[next++];
        }
    int32_t * dperm = (int32_t *)pi_malloc(sizeof(int32_t) * ff);
    if (!dperm) return PI_E_HIP;
    int rc = pi_memcpy_h2d(dperm, perm.data(), sizeof(int32_t) * ff);
    for (int k : {PI_T_FC2, PI_T_FFN_UP, PI_T_FFN_GATE, PI_T_FFN_DOWN_T}) {
        Tensor & t = m->L(il, k);
        if (rc != PI_OK || !t.dev) continue;                    // Falcon has no gate
        const size_t rb = row_bytes(t.type, t.ne0);
        unsigned char * moved = m->alloc<unsigned char>(rb * (size_t)ff);
        if (!moved) { rc = PI_E_HIP; break; }
        hipLaunchKernelGGL(gather_rows_kernel, dim3(ff), dim3(256), 0, nullptr, (const unsigned char *)t.dev, moved, dperm, rb);
        rc = pi::check_launch("gather_rows");
        if (rc == PI_OK && hipDeviceSynchronize() != hipSuccess) rc = pi::fail(PI_E_HIP, "gather_rows: device error");
        if (t.owned) for (auto & o : m->owned) if (o == t.dev) { pi_free(o); o = nullptr; }
        t.dev = moved; t.owned = true;
    }
    pi_free(dperm);
    return rc;
}
}  // namespace

namespace pi {
// the up / gate / down rows of layer il's non-resident neurons, in ascending neuron order, in pinned host memory that kernels read directly
int gather_rest_rows(pi_model * m, int il) {
    const pi_hparams & hp = m->hp;
    const int d = hp.n_embd, ff = hp.n_ff;
    Tensor & bucket = m->L(il, PI_T_GPU_BUCKET);
    if (!bucket.dev || m->rest_up[il]) return PI_OK;
    const int32_t * gi = (const int32_t *)m->L(il, PI_T_GPU_IDX).host;
    if (!gi) return pi::fail(PI_E_STATE, "gather_rest_rows: the layer has no gpu_idx");
    std::vector<int> rest;
    for (int j = 0; j < ff; ++j) if (gi[j] != 1) rest.push_back(j);
    if ((int)rest.size() + (int)bucket.ne0 != ff) return pi::fail(PI_E_ARG, "gather_rest_rows: gpu_idx and gpu_bucket disagree");
    for (int k : {PI_T_FFN_UP, PI_T_FFN_GATE, PI_T_FFN_DOWN_T}) {
        if (k == PI_T_FFN_GATE && hp.arch == PI_ARCH_FALCON) continue;
        Tensor & t = m->L(il, k);
        if (!t.host) return pi::fail(PI_E_STATE, "gather_rest_rows: the host copy of the FFN matrices is needed");
        const size_t rb = row_bytes(t.type, d);
        void * pin = nullptr;
        PI_HIP_TRY(hipHostMalloc(&pin, rb * (rest.empty() ? 1 : rest.size()), hipHostMallocDefault));
        m->pinned.push_back(pin);
        for (size_t i = 0; i < rest.size(); ++i) memcpy((unsigned char *)pin + rb * i, (const unsigned char *)t.host + rb * (size_t)rest[i], rb);
        (k == PI_T_FFN_UP ? m->rest_up : k == PI_T_FFN_GATE ? m->rest_gate : m->rest_down)[il] = pin;
    }
    return PI_OK;
}
}  // namespace pi

extern "C" {

int pi_model_finalize(pi_model * m) {
    if (!m) return pi::fail(PI_E_ARG, "pi_model_finalize: null model");
    if (m->finalized) return PI_OK;
    const pi_hparams & hp = m->hp;
    const int d = hp.n_embd, ff = hp.n_ff, gqa = m->gqa;
    PI_HIP_TRY(hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking));
    {
        const char * nb = getenv("PI_NO_BRANCH");          // PI_NO_BRANCH=1: Falcon layers run their two branches one after the other
        if (hp_arch_is_falcon(m) && !(nb && nb[0] == '1')) {
            PI_HIP_TRY(hipStreamCreateWithFlags(&m->stream2, hipStreamNonBlocking));
            m->ev_fork.resize(m->hp.n_layer); m->ev_join.resize(m->hp.n_layer);
            for (int il = 0; il < m->hp.n_layer; ++il) {
                PI_HIP_TRY(hipEventCreateWithFlags(&m->ev_fork[il], hipEventDisableTiming));
                PI_HIP_TRY(hipEventCreateWithFlags(&m->ev_join[il], hipEventDisableTiming));
            }
        }
    }
    PI_HIP_TRY(hipEventCreate(&m->ev0));
    PI_HIP_TRY(hipEventCreate(&m->ev1));

    for (int k : {PI_T_TOK_EMBD, PI_T_OUTPUT_NORM, PI_T_OUTPUT})
        if (!m->glob[k].dev) return pi::fail(PI_E_STATE, "pi_model_finalize: token_embd / output_norm / output missing");
    if (hp.arch == PI_ARCH_FALCON && !m->glob[PI_T_OUTPUT_NORM_B].dev) return pi::fail(PI_E_STATE, "pi_model_finalize: output_norm bias missing");

    int max_r = 0;
    for (int il = 0; il < hp.n_layer; ++il) {
        // pack q, k, v rows into one matrix so that one mat-vec produces q | k | v
        Tensor & wqkv = m->L(il, PI_T_WQKV);
        if (!wqkv.dev) {
            Tensor & wq = m->L(il, PI_T_WQ); Tensor & wk = m->L(il, PI_T_WK); Tensor & wv = m->L(il, PI_T_WV);
            if (!wq.dev || !wk.dev || !wv.dev) return pi::fail(PI_E_STATE, "pi_model_finalize: attention projections missing");
            if (wq.type != wk.type || wq.type != wv.type || wq.ne0 != d || wk.ne0 != d || wv.ne0 != d || wq.ne1 != d || wk.ne1 != gqa || wv.ne1 != gqa)
                return pi::fail(PI_E_ARG, "pi_model_finalize: attention projection shapes/types disagree");
            const size_t rb = row_bytes(wq.type, d);
            unsigned char * p = m->alloc<unsigned char>(rb * (size_t)(d + 2 * gqa));
            if (!p) return PI_E_HIP;
            PI_TRY(pi_memcpy_d2d(p, wq.dev, rb * d));
            PI_TRY(pi_memcpy_d2d(p + rb * d, wk.dev, rb * gqa));
            PI_TRY(pi_memcpy_d2d(p + rb * (d + gqa), wv.dev, rb * gqa));
            wqkv.type = wq.type; wqkv.dev = p; wqkv.ne0 = d; wqkv.ne1 = d + 2 * gqa; wqkv.owned = true;
            for (Tensor * t : {&wq, &wk, &wv}) {
                if (t->owned) {   // release the separate copies
                    for (auto & o : m->owned) if (o == t->dev) { pi_free(o); o = nullptr; }
                }
                t->dev = nullptr;
            }
        }
        if (wqkv.ne0 != d || wqkv.ne1 != d + 2 * gqa) return pi::fail(PI_E_ARG, "pi_model_finalize: wqkv shape");
        for (int k : {PI_T_ATTN_NORM, PI_T_WO, PI_T_FC1, PI_T_FC2})
            if (!m->L(il, k).dev) return pi::fail(PI_E_STATE, "pi_model_finalize: a layer tensor is missing (attn_norm / wo / fc1 / fc2)");
        if (hp.arch == PI_ARCH_LLAMA && !m->L(il, PI_T_FFN_NORM).dev) return pi::fail(PI_E_STATE, "pi_model_finalize: ffn_norm missing");
        if (hp.arch == PI_ARCH_FALCON && !m->L(il, PI_T_ATTN_NORM_B).dev) return pi::fail(PI_E_STATE, "pi_model_finalize: attn_norm bias missing");
        Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
        if (fc2.type != PI_TYPE_F16) return pi::fail(PI_E_UNSUPPORTED, "pi_model_finalize: predictor fc2 must be F16");
        if (fc1.ne0 != d || fc2.ne1 != ff || fc2.ne0 != fc1.ne1 || fc1.ne1 % 8) return pi::fail(PI_E_ARG, "pi_model_finalize: predictor shapes (fc1 {d, r}, fc2 {r, ff}, r % 8 == 0)");
        if ((int)fc1.ne1 > max_r) max_r = (int)fc1.ne1;

        // FFN matrices: whole on the GPU, or the bucket's rows only
        Tensor & bucket = m->L(il, PI_T_GPU_BUCKET);
        const int32_t * bk_host = (const int32_t *)bucket.host;
        const int n_bucket = bucket.dev ? (int)bucket.ne0 : 0;
        if (bucket.dev) {
            if (!m->L(il, PI_T_GPU_IDX).host) return pi::fail(PI_E_STATE, "pi_model_finalize: a layer with gpu_bucket needs gpu_idx");
            m->hybrid = true;
        }
        for (int k : {PI_T_FFN_UP, PI_T_FFN_GATE, PI_T_FFN_DOWN_T}) {
            Tensor & t = m->L(il, k);
            if (k == PI_T_FFN_GATE && hp.arch == PI_ARCH_FALCON) continue;
            if (t.dev) continue;                                     // adopted device tensor
            if (!t.host) return pi::fail(PI_E_STATE, "pi_model_finalize: an FFN matrix is missing");
            if (t.ne0 != d || t.ne1 != ff) return pi::fail(PI_E_ARG, "pi_model_finalize: FFN matrices must be {n_embd, n_ff}");
            const size_t rb = row_bytes(t.type, d);
            if (!bucket.dev) {
                t.dev = m->alloc<unsigned char>(rb * (size_t)ff);
                if (!t.dev) return PI_E_HIP;
                t.owned = true;
                PI_TRY(pi_memcpy_h2d(t.dev, t.host, rb * (size_t)ff));
                t.host = nullptr;
            } else {
                // compact [n_bucket][d] matrix in bucket order: gather on the host, one upload
                std::vector<unsigned char> tmp(rb * (size_t)(n_bucket ? n_bucket : 1));
                for (int i = 0; i < n_bucket; ++i) {
                    if (bk_host[i] < 0 || bk_host[i] >= ff || (i && bk_host[i] <= bk_host[i - 1]))
                        return pi::fail(PI_E_ARG, "pi_model_finalize: gpu_bucket must be strictly ascending neuron indices");
                    memcpy(tmp.data() + rb * i, (const unsigned char *)t.host + rb * (size_t)bk_host[i], rb);
                }
                t.dev = m->alloc<unsigned char>(tmp.size());
                if (!t.dev) return PI_E_HIP;
                t.owned = true;
                PI_TRY(pi_memcpy_h2d(t.dev, tmp.data(), tmp.size()));
            }
        }
    }

    // hot words / prefix of hybrid layers for the kernels that walk the neurons in groups of 32
    m->hot_words.assign(hp.n_layer, nullptr); m->hot_prefix.assign(hp.n_layer, nullptr);
    if (ff % 32 == 0) {
        for (int il = 0; il < hp.n_layer; ++il) {
            Tensor & bucket = m->L(il, PI_T_GPU_BUCKET);
            if (!bucket.dev) continue;
            const int32_t * bk_host = (const int32_t *)bucket.host;
            std::vector<uint32_t> words(ff / 32, 0u);
            std::vector<int32_t> prefix(ff / 32, 0);
            for (int i = 0; i < (int)bucket.ne0; ++i) words[bk_host[i] >> 5] |= 1u << (bk_host[i] & 31);
            for (int g = 1; g < ff / 32; ++g) prefix[g] = prefix[g - 1] + __builtin_popcount(words[g - 1]);
            m->hot_words[il] = m->alloc<uint32_t>(ff / 32); m->hot_prefix[il] = m->alloc<int32_t>(ff / 32);
            if (!m->hot_words[il] || !m->hot_prefix[il]) return PI_E_HIP;
            PI_TRY(pi_memcpy_h2d(m->hot_words[il], words.data(), sizeof(uint32_t) * words.size()));
            PI_TRY(pi_memcpy_h2d(m->hot_prefix[il], prefix.data(), sizeof(int32_t) * prefix.size()));
        }
    }

    // neurons dealt out by firing rate for the fused F16 kernel (see PI_T_NEURON_RATE)
    m->ffn_perm.assign(hp.n_layer, {});
    for (int il = 0; il < hp.n_layer && !m->neuron_rate.empty(); ++il) PI_TRY(deal_neurons_by_rate(m, il));

    // non-resident rows the GPU is to read itself: gathered in ascending neuron order into pinned host memory
    m->rest_up.assign(hp.n_layer, nullptr); m->rest_gate.assign(hp.n_layer, nullptr); m->rest_down.assign(hp.n_layer, nullptr);
    if (m->hybrid && m->rest_on_gpu) {
        for (int il = 0; il < hp.n_layer; ++il) {
            if (!m->L(il, PI_T_GPU_BUCKET).dev) continue;
            if (m->L(il, PI_T_FFN_UP).type != PI_TYPE_Q4_0 || !m->hot_words[il] || !pi_k_pred_upgate_q4_supported(ff, (int)m->L(il, PI_T_FC1).ne1, d))
                return pi::fail(PI_E_UNSUPPORTED, "pi_model_finalize: rest_on_gpu covers Q4_0 layers at n_embd 4096 with a predictor of rank 512 or 1024 and n_ff % 32 == 0");
            PI_TRY(pi::gather_rest_rows(m, il));
        }
    }

    m->ws = pi_workspace_create(ff, d);
    if (!m->ws) return PI_E_HIP;
    const size_t kv = (size_t)hp.n_layer * hp.n_head_kv * hp.n_ctx * m->hd;
    m->x = m->alloc<float>(d); m->x2 = m->alloc<float>(d); m->qkv = m->alloc<float>(d + 2 * gqa); m->q_rot = m->alloc<float>(d);
    m->att = m->alloc<float>(d); m->attn_out = m->alloc<float>(d); m->ffn_inp = m->alloc<float>(d); m->hidden = m->alloc<float>(max_r);
    m->pred_logits = m->alloc<float>(ff); m->h_c = m->alloc<float>(ff); m->h_dense = m->alloc<float>(ff); m->logits = m->alloc<float>(hp.n_vocab);
    m->cold_out = m->alloc<float>(d);
    m->list = m->alloc<int32_t>(ff); m->n_active = m->alloc<int32_t>(hp.n_layer);
    m->d_token = m->alloc<int32_t>(1); m->d_pos = m->alloc<int32_t>(1); m->d_step = m->alloc<int32_t>(1);
    m->d_out_tokens = m->alloc<int32_t>(m->max_steps); m->d_out_active = m->alloc<int32_t>(m->max_steps);
    m->k_cache = m->alloc<__half>(kv); m->v_cache = m->alloc<__half>(kv);
    m->cap_ffn = m->alloc<float>((size_t)hp.n_layer * d); m->cap_logits = m->alloc<float>((size_t)hp.n_layer * ff); m->cap_src = m->alloc<float>((size_t)hp.n_layer * d);
    if (!m->x || !m->x2 || !m->qkv || !m->q_rot || !m->att || !m->attn_out || !m->ffn_inp || !m->hidden || !m->pred_logits || !m->h_c || !m->h_dense ||
        !m->logits || !m->cold_out || !m->list || !m->n_active || !m->d_token || !m->d_pos || !m->d_step || !m->d_out_tokens || !m->d_out_active ||
        !m->k_cache || !m->v_cache || !m->cap_ffn || !m->cap_logits || !m->cap_src)
        return PI_E_HIP;
    PI_TRY(pi_memset(m->k_cache, 0, kv * 2));
    PI_TRY(pi_memset(m->v_cache, 0, kv * 2));
    // fused RoPE + attention when the head geometry and the context fit its single-pass kernel (the launcher's own test);
    // otherwise the rope_kv_store + attn_decode pair, whose smaller workgroup leaves room for a longer context
    // Long contexts (1024 cells and up, or more than one workgroup's LDS holds): the cells of every head are split over as many
    // workgroups as fill the chip (a compute unit pulls about 1/256 of the HBM rate, so one workgroup per head leaves the K / V rows
    // of a long context to n_head units), at least as many as bring a part's scores into LDS.
    const bool fused_ok = pi_k_attn_fused_supported(m->hd, hp.n_ctx) != 0;
    if (!fused_ok || hp.n_ctx >= 1024) {
        const int n_cu = pi::compute_units();
        // measured at 32 heads of 128: 8 parts are best up to about 4 k cells (one workgroup per unit), 16 beyond (41.9 against 55.8 us
        // at 8 k cells, 124 against 195 us at 32 k), 32 are slower again
        const int wg_cap = hp.n_ctx >= 4096 ? 2 * n_cu : n_cu;
        int parts = 2;
        while (parts < 16 && parts * 2 * hp.n_head <= wg_cap) parts *= 2;
        while (parts < 64 && !pi_k_attn_split_supported(m->hd, hp.n_ctx, parts)) parts *= 2;
        if (pi_k_attn_split_supported(m->hd, hp.n_ctx, parts)) {
            m->attn_parts = parts;
            m->attn_scratch = m->alloc<float>(pi_k_attn_split_scratch_floats(1, hp.n_head, m->hd, parts));
            if (!m->attn_scratch) return PI_E_HIP;
        }
    }
    if (fused_ok || m->attn_parts > 1) {
        m->rope_table = m->alloc<float>((size_t)hp.n_ctx * m->hd);
        if (!m->rope_table) return PI_E_HIP;
        PI_TRY(pi_k_rope_table(m->rope_table, hp.n_ctx, m->hd, hp.arch == PI_ARCH_FALCON ? 2 : 0, m->theta_scale, m->freq_scale, nullptr));
    }
    else if (!pi_k_attn_decode_supported(m->hd, hp.n_ctx))
        return pi::fail(PI_E_UNSUPPORTED, "pi_model_finalize: head size or context outside every attention kernel (head size a multiple of 8 that divides 512, at most 64 parts of the context per head)");
    PI_TRY(pi_memset(m->n_active, 0, sizeof(int32_t) * hp.n_layer));
    PI_TRY(pi_memset(m->d_step, 0, 4));
    PI_TRY(pi_memset(m->h_dense, 0, sizeof(float) * ff));
    if (m->hybrid && !m->rest_on_gpu) {
        m->cold = pi::cold_create(m);
        if (!m->cold) return PI_E_STATE;
    }
    PI_HIP_TRY(hipDeviceSynchronize());
    m->finalized = true;
    return PI_OK;
}

int pi_model_kv_clear(pi_model * m) {
    if (!m || !m->finalized) return pi::fail(PI_E_STATE, "pi_model_kv_clear: model not finalized");
    const size_t kv = (size_t)m->hp.n_layer * m->hp.n_head_kv * m->hp.n_ctx * m->hd;
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    PI_TRY(pi_memset(m->k_cache, 0, kv * 2));
    PI_TRY(pi_memset(m->v_cache, 0, kv * 2));
    m->kv_pos.clear();
    PI_TRY(pi_memset(m->d_pos, 0, 4));
    return PI_OK;
}

int pi_model_kv_seq_rm(pi_model * m, int p0, int p1) {
    if (!m || !m->finalized) return pi::fail(PI_E_STATE, "pi_model_kv_seq_rm: model not finalized");
    return pi::kv_edit(m, m->k_cache, m->v_cache, m->d_pos, m->kv_pos, p0, p1, 0, false);
}

int pi_model_kv_seq_shift(pi_model * m, int p0, int p1, int delta) {
    if (!m || !m->finalized) return pi::fail(PI_E_STATE, "pi_model_kv_seq_shift: model not finalized");
    return pi::kv_edit(m, m->k_cache, m->v_cache, m->d_pos, m->kv_pos, p0, p1, delta, true);
}

int pi_model_decode(pi_model * m, const int32_t * tokens, int n_tokens, int n_past, float * logits_out) {
    if (!m || !m->finalized) return pi::fail(PI_E_STATE, "pi_model_decode: model not finalized");
    if (!m->kv_pos.empty()) return pi::fail(PI_E_STATE, "pi_model_decode: the KV cells' positions are not contiguous (shift the cells behind a removed range first)");
    if (!tokens || n_tokens <= 0 || n_past < 0 || n_past + n_tokens > m->hp.n_ctx) return pi::fail(PI_E_ARG, "pi_model_decode: token range exceeds the context");
    for (int i = 0; i < n_tokens; ++i)
        if (tokens[i] < 0 || tokens[i] >= m->hp.n_vocab) return pi::fail(PI_E_ARG, "pi_model_decode: token id out of range");
    int first = 0;
    if (n_tokens > 2) {
        // the prompt goes through in chunks (weights read once per chunk): up to 512 tokens where the dense chunk path covers the
        // model (F16 or Q4_0 matrices, hybrid layers included), up to 16 for the remainder of an F16 model that is whole on the
        // device; what is left, and at least the last token, takes the single-token path below, which produces the logits
        const bool wide = pi::prefill_wide_supported(m), small = pi::prefill_supported(m);
        const int wide_max = wide ? pi::prefill_wide_max(m) : 0;
        while (n_tokens - 1 - first >= 2) {
            const int left = n_tokens - 1 - first;
            if (wide && left > 16) {
                const int T = left < wide_max ? left : wide_max;
                PI_TRY(pi::prefill_wide_chunk(m, tokens + first, T, n_past + first));
                first += T;
            } else if (small) {
                const int T = left < 16 ? left : 16;
                PI_TRY(pi::prefill_chunk(m, tokens + first, T, n_past + first));
                first += T;
            } else {
                break;
            }
        }
    }
    for (int i = first; i < n_tokens; ++i) {
        const bool last = i == n_tokens - 1;
        hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(64), 0, m->stream, m->d_token, m->d_pos, tokens[i], n_past + i);
        PI_TRY(pi::check_launch("set_state"));
        PI_TRY(token_forward(m, last, last));
    }
    // greedy choice on the device; the state then points at the next position
    PI_HIP_TRY(hipMemsetAsync(m->d_step, 0, 4, m->stream));
    PI_TRY(launch_advance(m));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    if (m->cold) PI_TRY(pi::cold_drain(m->cold));
    int32_t tok = -1;
    PI_TRY(pi_memcpy_d2h(&tok, m->d_token, 4));
    if (logits_out) PI_TRY(pi_memcpy_d2h(logits_out, m->logits, sizeof(float) * m->hp.n_vocab));
    return tok;
}

int pi_model_generate(pi_model * m, int n_steps, int32_t * out_tokens, float * ms_out) {
    if (!m || !m->finalized) return pi::fail(PI_E_STATE, "pi_model_generate: model not finalized");
    if (n_steps <= 0 || n_steps > m->max_steps || !out_tokens) return pi::fail(PI_E_ARG, "pi_model_generate: bad step count");
    if (!m->kv_pos.empty()) return pi::fail(PI_E_STATE, "pi_model_generate: the KV cells' positions are not contiguous (shift the cells behind a removed range first)");
    int32_t pos = 0;
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    PI_TRY(pi_memcpy_d2h(&pos, m->d_pos, 4));
    if (pos + n_steps > m->hp.n_ctx) return pi::fail(PI_E_ARG, "pi_model_generate: would run past the context");
    PI_HIP_TRY(hipMemsetAsync(m->d_step, 0, 4, m->stream));

    // PI_NO_GRAPH=1 issues the same launches eagerly (useful under tracing tools that cannot follow graph replays)
    const char * no_graph = getenv("PI_NO_GRAPH");
    // a model with host threads replays a graph too when every hybrid layer hands over through the stream's own wait kernels
    const bool host_in_loop = m->hybrid && !m->rest_on_gpu && !pi::cold_every_layer_async(m->cold);
    const bool use_graph = !host_in_loop && !m->capture && !(no_graph && no_graph[0] == '1');
    const bool announce = use_graph && pi::cold_async(m->cold);
    // the token, the position and the step counter advance on the device, so one captured token is replayed for every step (graphs
    // of 2..32 tokens per replay measured the same or slower: 523.9 tok/s with 1, 523.3 with 8, 517 with 16, 508 with 32 on the 7B shape)
    if (use_graph && !m->graph_exec) {
        PI_HIP_TRY(hipStreamBeginCapture(m->stream, hipStreamCaptureModeThreadLocal));
        m->building_graph = true;
        int rc = token_forward(m, true, false);
        m->building_graph = false;
        if (rc == PI_OK) rc = launch_advance(m);
        hipGraph_t g = nullptr;
        const hipError_t e = hipStreamEndCapture(m->stream, &g);
        if (rc != PI_OK) { if (g) (void)hipGraphDestroy(g); return rc; }
        if (e != hipSuccess) return pi::hip_fail(e, "hipStreamEndCapture");
        m->graph = g;
        PI_HIP_TRY(hipGraphInstantiate(&m->graph_exec, g, nullptr, nullptr, 0));
    }
    PI_HIP_TRY(hipEventRecord(m->ev0, m->stream));
    for (int s = 0; s < n_steps; ++s) {
        if (use_graph) {
            if (announce) PI_TRY(pi::cold_post_token(m->cold));
            PI_HIP_TRY(hipGraphLaunch(m->graph_exec, m->stream));
        } else {
            PI_TRY(token_forward(m, true, false));
            PI_TRY(launch_advance(m));
        }
    }
    PI_HIP_TRY(hipEventRecord(m->ev1, m->stream));
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    if (m->cold) PI_TRY(pi::cold_drain(m->cold));
    if (ms_out) PI_HIP_TRY(hipEventElapsedTime(ms_out, m->ev0, m->ev1));
    PI_TRY(pi_memcpy_d2h(out_tokens, m->d_out_tokens, sizeof(int32_t) * n_steps));
    return PI_OK;
}

int pi_model_time_section(pi_model * m, int section, int rounds, float * ms_total, int * launches) {
    if (!m || !m->finalized || !ms_total || !launches || rounds <= 0) return pi::fail(PI_E_ARG, "pi_model_time_section: bad arguments");
    if (m->hybrid) return pi::fail(PI_E_UNSUPPORTED, "pi_model_time_section: not available for hybrid models");
    const pi_hparams & hp = m->hp;
    const int d = hp.n_embd, ff = hp.n_ff, gqa = m->gqa;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    hipStream_t st = m->stream;
    PI_HIP_TRY(hipStreamSynchronize(st));
    int n = 0;
    PI_HIP_TRY(hipEventRecord(m->ev0, st));
    for (int r = 0; r < rounds; ++r) {
        if (section == 2) {
            pi_norm on = make_norm(falcon ? 2 : 1, hp.norm_eps, m->glob[PI_T_OUTPUT_NORM], falcon ? &m->glob[PI_T_OUTPUT_NORM_B] : nullptr);
            PI_TRY(pi_k_gemv(m->glob[PI_T_OUTPUT].type, m->glob[PI_T_OUTPUT].dev, hp.n_vocab, d, m->x, &on, PI_EPI_NONE, nullptr, nullptr, m->logits, st));
            ++n;
            continue;
        }
        for (int il = 0; il < hp.n_layer; ++il) {
            if (section == 0) {
                Tensor & wqkv = m->L(il, PI_T_WQKV);
                pi_norm an = falcon ? make_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B))
                                    : make_norm(1, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), nullptr);
                PI_TRY(pi_k_gemv(wqkv.type, wqkv.dev, d + 2 * gqa, d, m->x, &an, PI_EPI_NONE, nullptr, nullptr, m->qkv, st));
                ++n;
            } else if (section == 1) {
                // the sparse FFN block as the decode loop issues it, on the activations the last token left behind
                Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
                Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
                const bool q4 = up.type == PI_TYPE_Q4_0;
                pi_norm fn = falcon ? make_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B))
                                    : make_norm(1, hp.norm_eps, m->L(il, PI_T_FFN_NORM), nullptr);
                // Falcon's predictor and FFN read the layer input; LLaMA's read the post-attention residual stream
                const float * fin = falcon ? m->x : m->ffn_inp;
                PI_TRY(pi_k_gemv(fc1.type, fc1.dev, (int)fc1.ne1, d, fin, nullptr, PI_EPI_RELU, nullptr, nullptr, m->hidden, st));
                if (!q4 && pi_k_sparse_ffn_supported(ff, (int)fc1.ne1, d)) {
                    PI_TRY(pi_k_sparse_ffn(fc2.dev, ff, (int)fc1.ne1, m->hidden, hp.sparse_threshold, up.dev, falcon ? nullptr : gate.dev, down.dev, d,
                                                  fin, &fn, PI_EPI_ADD, fin, nullptr, m->x2, nullptr, nullptr, m->n_active + il, m->ws, st));
                    ++n;
                    continue;
                }
                if (q4 && fc2.type == PI_TYPE_F16 && pi_k_pred_upgate_q4_supported(ff, (int)fc1.ne1, d)) {
                    PI_TRY(pi_k_sparse_ffn_q4_partials(fc2.dev, ff, (int)fc1.ne1, m->hidden, hp.sparse_threshold, up.dev, falcon ? nullptr : gate.dev, down.dev,
                                                       nullptr, nullptr, nullptr, d, fin, &fn, nullptr, nullptr, m->pred_logits, m->h_dense, m->ws, st));
                    PI_TRY(pi_k_sparse_ffn_q4_reduce(ff, d, PI_EPI_ADD, fin, nullptr, m->x2, m->n_active + il, m->ws, st));
                    ++n;
                    continue;
                }
                PI_TRY(pi_k_predictor_fc2(fc2.dev, ff, (int)fc1.ne1, m->hidden, hp.sparse_threshold, nullptr, 0, m->pred_logits,
                                          q4 ? m->list : nullptr, q4 ? m->n_active + il : nullptr, q4 ? m->h_dense : nullptr, m->ws, st));
                PI_TRY(pi_k_sparse_upgate(up.type, up.dev, falcon ? nullptr : gate.dev, d, ff, fin, &fn, q4 ? 0 : 1, m->list, m->n_active + il, nullptr, m->h_c,
                                          q4 ? m->h_dense : nullptr, nullptr, nullptr, m->ws, st));
                PI_TRY(pi_k_sparse_axpy(down.type, down.dev, d, ff, m->h_c, q4 ? m->h_dense : nullptr, nullptr, m->list, m->n_active + il,
                                        PI_EPI_ADD, m->ffn_inp, nullptr, m->x2, m->ws, st));
                ++n;
            } else if (section == 3 || section == 4) {
                // one kernel of the fused F16 block alone: 3 the predictor + gate/up/down kernel, 4 the reduction of its partial vectors
                Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
                Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
                if (up.type != PI_TYPE_F16 || !pi_k_sparse_ffn_supported(ff, (int)fc1.ne1, d))
                    return pi::fail(PI_E_UNSUPPORTED, "pi_model_time_section: the fused F16 block does not cover this model");
                pi_norm fn = falcon ? make_norm(2, hp.norm_eps, m->L(il, PI_T_ATTN_NORM), &m->L(il, PI_T_ATTN_NORM_B))
                                    : make_norm(1, hp.norm_eps, m->L(il, PI_T_FFN_NORM), nullptr);
                const float * fin = falcon ? m->x : m->ffn_inp;
                if (section == 3)
                    PI_TRY(pi_k_sparse_ffn_partials(fc2.dev, ff, (int)fc1.ne1, m->hidden, hp.sparse_threshold, up.dev, falcon ? nullptr : gate.dev, down.dev, d,
                                                           fin, &fn, nullptr, nullptr, m->ws, st));
                else
                    PI_TRY(pi_k_sparse_ffn_reduce(ff, d, PI_EPI_ADD, fin, nullptr, m->x2, m->n_active + il, m->ws, st));
                ++n;
            } else {
                return pi::fail(PI_E_ARG, "pi_model_time_section: unknown section");
            }
        }
    }
    PI_HIP_TRY(hipEventRecord(m->ev1, st));
    PI_HIP_TRY(hipStreamSynchronize(st));
    PI_HIP_TRY(hipEventElapsedTime(ms_total, m->ev0, m->ev1));
    *launches = n;
    return PI_OK;
}

int pi_model_set_rest_on_gpu(pi_model * m, int enable) {
    if (!m) return pi::fail(PI_E_ARG, "pi_model_set_rest_on_gpu: null model");
    if (m->finalized) return pi::fail(PI_E_STATE, "pi_model_set_rest_on_gpu: call before pi_model_finalize");
    m->rest_on_gpu = enable != 0;
    return PI_OK;
}

int pi_model_set_capture(pi_model * m, int enable) {
    if (!m) return pi::fail(PI_E_ARG, "pi_model_set_capture: null model");
    m->capture = enable != 0;
    return PI_OK;
}

int pi_model_get_capture(pi_model * m, float * ffn_out, float * pred_logits, int32_t * n_active, float * ffn_src) {
    if (!m || !m->finalized) return pi::fail(PI_E_STATE, "pi_model_get_capture: model not finalized");
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    if (ffn_out) PI_TRY(pi_memcpy_d2h(ffn_out, m->cap_ffn, sizeof(float) * (size_t)m->hp.n_layer * m->hp.n_embd));
    if (pred_logits) {
        PI_TRY(pi_memcpy_d2h(pred_logits, m->cap_logits, sizeof(float) * (size_t)m->hp.n_layer * m->hp.n_ff));
        // layers whose neurons were dealt out by rate computed their logits in that order: hand them back in file order
        std::vector<float> tmp;
        for (int il = 0; il < m->hp.n_layer; ++il) {
            const std::vector<int32_t> & perm = m->ffn_perm[il];
            if (perm.empty()) continue;
            float * row = pred_logits + (size_t)il * m->hp.n_ff;
            tmp.assign(row, row + m->hp.n_ff);
            for (int i = 0; i < m->hp.n_ff; ++i) row[perm[i]] = tmp[i];
        }
    }
    if (n_active) PI_TRY(pi_memcpy_d2h(n_active, m->n_active, sizeof(int32_t) * m->hp.n_layer));
    if (ffn_src) PI_TRY(pi_memcpy_d2h(ffn_src, m->cap_src, sizeof(float) * (size_t)m->hp.n_layer * m->hp.n_embd));
    return PI_OK;
}

int pi_model_step_active(pi_model * m, int32_t * per_step_total, int n_steps) {
    if (!m || !m->finalized || !per_step_total || n_steps <= 0 || n_steps > m->max_steps) return pi::fail(PI_E_ARG, "pi_model_step_active: bad arguments");
    PI_HIP_TRY(hipStreamSynchronize(m->stream));
    return pi_memcpy_d2h(per_step_total, m->d_out_active, sizeof(int32_t) * n_steps);
}

}  // extern "C"

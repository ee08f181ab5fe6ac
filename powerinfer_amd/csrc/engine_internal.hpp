// Internal layout of the decode engine's model object (shared by the engine and the host cold path).
#pragma once

#include "../../include/powerinfer_hip.h"
#include "cold_path.hpp"

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <unordered_map>
#include <vector>

struct Tensor {
    int          type = -1;
    void *       dev = nullptr;      // device address (rows possibly sliced to the GPU bucket)
    const void * host = nullptr;     // borrowed host copy (hybrid layers: full-size matrices for the cold path)
    int64_t      ne0 = 0, ne1 = 0;   // as given by the caller
    bool         owned = false;
};


struct BatchState;

struct pi_model {
    pi_hparams hp{};
    std::vector<Tensor> layers;           // [n_layer][PI_T_COUNT]
    Tensor glob[4];
    std::vector<void *> owned;            // every device allocation made by the model
    bool finalized = false, hybrid = false;
    int hd = 0, gqa = 0, max_steps = 4096;
    hipStream_t stream = nullptr;
    hipStream_t stream2 = nullptr;         // Falcon: the FFN branch runs beside the attention branch (both read the layer input)
    std::vector<hipEvent_t> ev_fork, ev_join;
    pi_workspace * ws = nullptr;
    float theta_scale = 0.0f;
    float freq_scale = 1.0f;          // linear RoPE scaling (1 = none)

    float *x = nullptr, *x2 = nullptr, *qkv = nullptr, *q_rot = nullptr, *att = nullptr, *attn_out = nullptr, *ffn_inp = nullptr;
    float *hidden = nullptr, *pred_logits = nullptr, *h_c = nullptr, *h_dense = nullptr, *logits = nullptr, *cold_out = nullptr;
    int32_t *list = nullptr, *n_active = nullptr, *d_token = nullptr, *d_pos = nullptr, *d_step = nullptr;
    int32_t *d_out_tokens = nullptr, *d_out_active = nullptr;
    __half *k_cache = nullptr, *v_cache = nullptr;
    float *rope_table = nullptr;          // float2 [n_ctx][hd/2] (cos, sin), when the fused or the split attention kernel is used
    int    attn_parts = 1;                // > 1: the cells of every head are split over this many workgroups (long contexts)
    float *attn_scratch = nullptr;        // partial results of those workgroups for one token
    float *attn_scratch_chunk = nullptr;  // and for a prompt chunk (allocated at the first chunk that needs it)

    hipGraphExec_t graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;

    bool building_graph = false;          // token_forward is being recorded into a graph, not run
    bool capture = false;
    float *cap_ffn = nullptr, *cap_logits = nullptr, *cap_src = nullptr;       // device
    pi::ColdPath * cold = nullptr;
    std::vector<int32_t> kv_pos;          // positions of the cache cells while an edit left them non-contiguous; empty: cell i holds position i
    __half * kv_stage = nullptr;          // [n_layer * n_head_kv][n_ctx][hd] staging for cell compaction, allocated at the first edit
    int32_t * kv_map = nullptr;           // [n_ctx] device copy of the cell map / deltas of an edit
    std::vector<uint32_t *> hot_words;    // per hybrid layer: bit j of word g set iff neuron 32g+j is GPU-resident (device)
    std::vector<int32_t *> hot_prefix;    //                   GPU-resident neurons before group g = row of the compact matrices
    // hybrid layers whose non-resident rows the GPU reads from pinned host memory itself (pi_model_set_rest_on_gpu): per layer
    // the up / gate / down rows of the non-resident neurons in ascending order; no host threads, the token loop replays as a graph
    bool rest_on_gpu = false;
    std::vector<void *> rest_up, rest_gate, rest_down;
    std::vector<void *> pinned;           // hipHostMalloc allocations owned by the model
    // layers whose neurons were dealt out by firing rate (PI_T_NEURON_RATE): position -> neuron of the file; empty: file order
    std::vector<std::vector<float>>   neuron_rate;     // per layer, as given (empty: none)
    std::vector<std::vector<int32_t>> ffn_perm;
    BatchState * batch = nullptr;         // per-sequence caches and step buffers of batched decoding
    BatchState * cells = nullptr;         // the KV cache with cells shared between sequences and its step buffers (pi_model_kv_cells_*)
    BatchState * prefill = nullptr;       // step buffers for prompt chunks of the model's own sequence
    BatchState * prefill_wide = nullptr;  // the same for chunks of up to 512 tokens (dense mat-muls, weights read once per chunk)
    pi_gemm_lib * gemm_lib = nullptr;     // hipBLASLt plans of those mat-muls (PI_PREFILL_GEMM=own keeps them on this library's kernel, 128 tokens a chunk)
    // multi-token steps of a Q4_0 model on integer matrix cores: every Q4_0 matrix once more as 16-byte-aligned quants and fp16
    // scales (pi_k_q4_split), made at the first such step; q4_steps says the model takes that route
    struct Q4Split { const void * quants; const void * scales; };
    std::unordered_map<const Tensor *, Q4Split> q4_split;
    bool q4_steps = false;
    std::vector<__half *> down_rows;      // per layer: the down projection with the neurons contiguous ([n_embd][n_ff]), made at the first wide chunk
                                          // (null for Q4_0 and hybrid layers, whose matrices are expanded into the chunk's scratch instead)

    Tensor & L(int il, int kind) { return layers[(size_t)il * PI_T_COUNT + kind]; }

    template <typename T> T * alloc(size_t count) {
        void * p = pi_malloc(sizeof(T) * (count ? count : 1));
        if (p) owned.push_back(p);
        return (T *)p;
    }
};

namespace pi {
int  kv_edit(pi_model * m, __half * k_cache, __half * v_cache, int32_t * d_pos, std::vector<int32_t> & kv_pos, int p0, int p1, int delta, bool shift);
void batch_destroy(pi_model * m);       // frees the batched-decoding state (graphs; device buffers belong to the model)
bool prefill_supported(pi_model * m);   // F16 weights, every neuron on the GPU, shapes the multi-token kernels cover
int  prefill_chunk(pi_model * m, const int32_t * tokens, int T, int n_past);
bool prefill_wide_supported(pi_model * m);   // F16 or Q4_0 matrices (fp16 predictor), hybrid layers included; n_embd, n_ff and the predictor rank multiples of 256
int  gather_rest_rows(pi_model * m, int il);  // hybrid layer: rows of the non-resident neurons into pinned host memory (rest_up / rest_gate / rest_down)
int  prefill_wide_max(pi_model * m);         // longest chunk: 512 through the library mat-mul, 128 on this library's own kernel (PI_PREFILL_GEMM=own)
int  prefill_wide_chunk(pi_model * m, const int32_t * tokens, int T, int n_past);     // 16 < T <= prefill_wide_max
}

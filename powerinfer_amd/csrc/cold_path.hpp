// CPU share of a hybrid (hot/cold split) layer: the neurons that are not GPU-resident are computed on host
// threads from the same predictor logits and merged into the layer output
// (llm_build_sparse_mul_mat / llm_build_sparse_axpy hybrid variants, llama.cpp:4581-4593, 4635-4646).
#pragma once

#include <hip/hip_runtime.h>

struct pi_model;

namespace pi {

struct ColdPath;

ColdPath * cold_create(pi_model * m);
void       cold_destroy(ColdPath * c);
// Runs right after the predictor of layer `il` has been queued on `st`: starts the copies the host share needs.
int        cold_stage_inputs(ColdPath * c, int il, pi_model * m, hipStream_t st);
// Runs after the GPU share's up/gate launch of layer `il` has been queued on `st`; leaves the merged layer
// output (cold + hot + residuals) in m->x2.
int        cold_layer_merge(ColdPath * c, int il, pi_model * m, hipStream_t st);

// Q4_0 hybrid layer at d = 4096 on the fused kernels: queues fc2 + mask + resident up/gate, computes the host share from the
// buffers that launch fills, queues the down projection and the merge; leaves the layer output in m->x2.
int        cold_layer_q4(ColdPath * c, int il, pi_model * m, hipStream_t st, bool capture);
// The same for an F16 hybrid layer at a width the fused F16 kernels cover: the resident share needs nothing from the host, so
// its whole FFN (gate/up/down partial vectors) is queued at once and only the final reduction waits for the host share.
int        cold_layer_f16(ColdPath * c, int il, pi_model * m, hipStream_t st, bool capture);

// Hybrid layers (Q4_0, and F16 at 4096 columns) with nothing launched between the two halves: the stream holds hand-over kernels, a service thread computes the
// host share when the device signals and answers through flag words in pinned memory.  cold_post_token announces one token's
// hybrid layers to the service thread (call it once per token whose kernels are queued with cold_layer_q4_queue), cold_drain
// confirms after a stream synchronisation that every hand-over completed.  PI_COLD_SYNC=1 keeps the launching thread in the loop.
bool       cold_async(const ColdPath * c);
bool       cold_every_layer_async(const ColdPath * c);   // no hybrid layer needs the launching thread: the token loop can be one graph
int        cold_post_token(ColdPath * c);
int        cold_drain(ColdPath * c);
int        cold_layer_q4_queue(ColdPath * c, int il, pi_model * m, hipStream_t st);
int        cold_layer_f16_queue(ColdPath * c, int il, pi_model * m, hipStream_t st);     // F16 layers at 4096 columns: one hand-over each way
bool       cold_layer_async(const ColdPath * c, int il);

int add_vec(float * y, const float * a, int n, hipStream_t st);
// dst = ((cold + hot) + r1) [+ r2]; `cold` may be pinned host memory; `keep` (optional) receives cold + hot
int merge_shares(float * dst, const float * cold, const float * hot, const float * r1, const float * r2, float * keep, int n, hipStream_t st);

}  // namespace pi

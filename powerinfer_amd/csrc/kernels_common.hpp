// What the kernel files of this library share: block-wide reductions, activation staging, the epilogue of the mat-vecs, the launchers'
// view of a norm, and the workspace behind the pi_k_* launchers.  Device helpers sit in an unnamed namespace: every translation unit
// gets its own copy, and none of them is exported.
#pragma once
#include "device_utils.hpp"
#include "runtime.hpp"
#include "../../include/powerinfer_hip.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

namespace {

constexpr int kBlock = 256;                 // 4 waves
constexpr int kWavesPerBlock = kBlock / PI_WAVE;

struct NormArgs { int kind; float eps; const float * w; const float * b; };

// ---------------------------------------------------------------------------------------------------
// block-wide reductions (double, fixed order: lanes by butterfly, waves 0..n-1 sequentially)
// ---------------------------------------------------------------------------------------------------
__device__ double block_sum_f64(double v, double * red) {
    v = pi_wave_sum_f64(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    double s = 0.0;
    for (int i = 0; i < nw; ++i) s += red[i];
    return s;
}
__device__ float block_max_f32(float v, float * red) {
    v = pi_wave_max(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float s = red[0];
    for (int i = 1; i < nw; ++i) s = fmaxf(s, red[i]);
    return s;
}

// ---------------------------------------------------------------------------------------------------
// Activation staging.  x (fp32, global) -> optional norm -> rounded to fp16 -> LDS.
// RMSNorm as ggml.c:9238-9284 (double sum of fp32 squares, scale = 1/sqrtf(mean+eps), then * w as a
// second fp32 multiply: llm_build_norm, llama.cpp:4420-4450); LayerNorm as ggml.c:9169-9236.
// ---------------------------------------------------------------------------------------------------
__device__ void stage_x_f16(__half * xs, const float * __restrict__ x, int cols, NormArgs na, double * red) {
    float mean = 0.0f, scale = 1.0f;
    if (na.kind == 1) {
        double s = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float v = x[i]; s += (double)__fmul_rn(v, v); }
        s = block_sum_f64(s, red);
        scale = pi_inv_sqrt((float)(s / cols) + na.eps);
    } else if (na.kind == 2) {
        double s = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) s += (double)x[i];
        s = block_sum_f64(s, red);
        mean = (float)(s / cols);
        double s2 = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float v = __fsub_rn(x[i], mean); s2 += (double)__fmul_rn(v, v); }
        s2 = block_sum_f64(s2, red);
        scale = pi_inv_sqrt((float)(s2 / cols) + na.eps);
    }
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        float v = x[i];
        if (na.kind != 0) {
            v = __fmul_rn(na.kind == 2 ? __fsub_rn(v, mean) : v, scale);
            if (na.w) v = __fmul_rn(v, na.w[i]);
            if (na.b) v = __fadd_rn(v, na.b[i]);
        }
        xs[i] = __float2half_rn(v);
    }
    __syncthreads();
}

// Fast staging for cols % 256 == 0.  These kernels run a few microseconds, so what they wait for matters more
// than what they compute: the activation vector and the norm weights are brought in with direct global->LDS
// loads (no registers, a handful of instructions) issued together with the first weight loads, so that the
// whole prologue costs one memory round trip; the code is kept small because every launch starts with a
// cold instruction cache.
// LDS layout (floats): xraw[cols] | wn[cols] | then xs as fp16[cols].
__device__ __forceinline__ void stage_fast_issue(float * lds, const float * __restrict__ x, NormArgs na, int cols) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool has_w = na.kind != 0 && na.w != nullptr;
    const int nw = blockDim.x >> 6;
    for (int base = wave * 256; base < cols; base += nw * 256) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(x + base + lane * 4),
                                         (__attribute__((address_space(3))) void *)(lds + base), 16, 0, 0);
        if (has_w)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(na.w + base + lane * 4),
                                             (__attribute__((address_space(3))) void *)(lds + cols + base), 16, 0, 0);
    }
}
// call after the loads above have landed (s_waitcnt + barrier); leaves fp16 activations in xs
__device__ __forceinline__ void stage_fast_finish(__half * xs, const float * lds, NormArgs na, int cols, double * red) {
    const float * xraw = lds;
    const float * wn = lds + cols;
    float mean = 0.0f, scale = 1.0f;
    if (na.kind == 1) {
        double s = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float v = xraw[i]; s += (double)__fmul_rn(v, v); }
        s = block_sum_f64(s, red);
        scale = pi_inv_sqrt((float)(s / cols) + na.eps);
    } else if (na.kind == 2) {
        double s = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) s += (double)xraw[i];
        s = block_sum_f64(s, red);
        mean = (float)(s / cols);
        double s2 = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float v = __fsub_rn(xraw[i], mean); s2 += (double)__fmul_rn(v, v); }
        s2 = block_sum_f64(s2, red);
        scale = pi_inv_sqrt((float)(s2 / cols) + na.eps);
    }
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        float v = xraw[i];
        if (na.kind != 0) {
            v = __fmul_rn(na.kind == 2 ? __fsub_rn(v, mean) : v, scale);
            if (na.w) v = __fmul_rn(v, wn[i]);
            if (na.b) v = __fadd_rn(v, na.b[i]);
        }
        xs[i] = __float2half_rn(v);
    }
    __syncthreads();
}
__host__ __device__ inline size_t stage_fast_lds_bytes(int cols) { return (size_t)cols * (4 + 4 + 2); }

// Q8_0 staging for Q4_0 weights: per block of 32, d = amax/127 kept as fp16, q = rint(x * 127/amax)
// (x86 path of quantize_row_q8_0, ggml-quants.c:702-760).  LDS layout: int8 q[cols] then float d[cols/32].
__device__ void stage_x_q8(int8_t * xq, float * xd, const float * __restrict__ x, int cols, NormArgs na, double * red, float * xtmp) {
    // normalised values first (fp32) into xtmp (LDS), then quantise per 32-block
    if (na.kind == 0) {
        for (int i = threadIdx.x; i < cols; i += blockDim.x) xtmp[i] = x[i];
    } else if (na.kind == 1) {
        double s = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float v = x[i]; s += (double)__fmul_rn(v, v); }
        s = block_sum_f64(s, red);
        const float scale = pi_inv_sqrt((float)(s / cols) + na.eps);
        for (int i = threadIdx.x; i < cols; i += blockDim.x) {
            float v = __fmul_rn(x[i], scale);
            if (na.w) v = __fmul_rn(v, na.w[i]);
            if (na.b) v = __fadd_rn(v, na.b[i]);
            xtmp[i] = v;
        }
    } else {
        double s = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) s += (double)x[i];
        s = block_sum_f64(s, red);
        const float mean = (float)(s / cols);
        double s2 = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float v = __fsub_rn(x[i], mean); s2 += (double)__fmul_rn(v, v); }
        s2 = block_sum_f64(s2, red);
        const float scale = pi_inv_sqrt((float)(s2 / cols) + na.eps);
        for (int i = threadIdx.x; i < cols; i += blockDim.x) {
            float v = __fmul_rn(__fsub_rn(x[i], mean), scale);
            if (na.w) v = __fmul_rn(v, na.w[i]);
            if (na.b) v = __fadd_rn(v, na.b[i]);
            xtmp[i] = v;
        }
    }
    __syncthreads();
    // 32 consecutive lanes own one block of 32 values
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        const float v = xtmp[i];
        float amax = fabsf(v);
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, PI_WAVE));
        const float d = pi_div(amax, 127.0f);
        const float id = (amax != 0.0f) ? pi_div(127.0f, amax) : 0.0f;
        xq[i] = (int8_t)(int)rintf(__fmul_rn(v, id));
        if ((i & 31) == 0) xd[i >> 5] = pi_round_f16(d);
    }
    __syncthreads();
}

__device__ __forceinline__ float apply_epilogue(float v, int epi, const float * add1, const float * add2, int row) {
    if (epi == PI_EPI_RELU) return fmaxf(v, 0.0f);
    if (epi == PI_EPI_ADD)  return __fadd_rn(v, add1[row]);
    if (epi == PI_EPI_ADD2) return __fadd_rn(__fadd_rn(v, add1[row]), add2[row]);
    return v;
}

// shapes and operand types the step kernels and their callers agree on
typedef _Float16 pi_h8 __attribute__((ext_vector_type(8)));
typedef float    pi_f4 __attribute__((ext_vector_type(4)));
constexpr int kBtMaxT = 16;
constexpr int kChunkMaxT = 512;           // longest chunk of the attention, embedding and elementwise kernels of a prompt chunk
constexpr int kBmGroups = 32;
constexpr int kAxpyTile = PI_WAVE * 8;

// exclusive prefix sum of one int per thread over the workgroup (wave scans, then the waves' totals in order); *total = the sum
__device__ int block_exclusive_scan_i32(int v, int * total, int * sred) {
    // inclusive scan within the wave
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    int inc = v;
#pragma unroll
    for (int o = 1; o < PI_WAVE; o <<= 1) { const int t = __shfl_up(inc, o, PI_WAVE); if (lane >= o) inc += t; }
    __syncthreads();
    if (lane == PI_WAVE - 1) sred[wave] = inc;
    __syncthreads();
    int base = 0, tot = 0;
    for (int i = 0; i < nw; ++i) { const int s = sred[i]; if (i < wave) base += s; tot += s; }
    *total = tot;
    return base + inc - v;
}

__device__ void compact_from_words(const uint32_t * words, int ff, const int32_t * __restrict__ bucket, int n_bucket,
                                   int32_t * __restrict__ list, int32_t * __restrict__ n_active, int * sred) {
    int base = 0;
    if (bucket == nullptr) {
        const int nwords = (ff + 31) / 32;
        for (int w0 = 0; w0 < nwords; w0 += blockDim.x) {
            const int w = w0 + threadIdx.x;
            uint32_t bits = (w < nwords) ? words[w] : 0u;
            int tot;
            int off = base + block_exclusive_scan_i32(__popc(bits), &tot, sred);
            while (bits) { const int b = __ffs(bits) - 1; bits &= bits - 1; list[off++] = w * 32 + b; }
            base += tot;
        }
    } else {
        for (int r0 = 0; r0 < n_bucket; r0 += blockDim.x) {
            const int r = r0 + threadIdx.x;
            int act = 0;
            if (r < n_bucket) { const int n = bucket[r]; act = (words[n >> 5] >> (n & 31)) & 1u; }
            int tot;
            const int off = base + block_exclusive_scan_i32(act, &tot, sred);
            if (act) list[off] = r;
            base += tot;
        }
    }
    if (threadIdx.x == 0) *n_active = base;
}

__device__ __forceinline__ int select_nth_bit(uint32_t bits, int n) {      // index of the n-th (0-based) set bit
    for (int i = 0; i < n; ++i) bits &= bits - 1;
    return __ffs(bits) - 1;
}

// Q4_0 dot of one 32-weight block against the staged Q8_0 activations: exact int32 sum of products,
// then * (d_w * d_x) into fp32 (vec_dot_q4_0_q8_0, ggml-quants.c:2512-2650)
__device__ __forceinline__ float q4_block_dot(const pi_block_q4_0 * __restrict__ wb, const int8_t * __restrict__ xq, float dx, float acc) {
    uint16_t dbits; uint32_t q[4];
    __builtin_memcpy(&dbits, &wb->d, 2);
    __builtin_memcpy(q, wb->qs, 16);
    const int * x32 = reinterpret_cast<const int *>(xq);          // 32 int8 = 8 dwords, 4-byte aligned in LDS
    int sum = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int lo = (int)(q[j] & 0x0F0F0F0Fu);                  // elements 4j .. 4j+3
        const int hi = (int)((q[j] >> 4) & 0x0F0F0F0Fu);           // elements 16+4j .. 16+4j+3
        sum = __builtin_amdgcn_sdot4(lo, x32[j], sum, false);
        sum = __builtin_amdgcn_sdot4(hi, x32[4 + j], sum, false);
    }
    // nibbles were used unsigned: subtract 8 * sum(x) of the block
    int sx = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) sx = __builtin_amdgcn_sdot4(0x01010101, x32[j], sx, false);
    sum -= 8 * sx;
    return fmaf(__fmul_rn(pi_f16_from_bits(dbits), dx), (float)sum, acc);
}

// Angle of pair i at position p as the CPU path forms it (ggml.c:11196-11319, rope_yarn with ext_factor 0, ggml.c:11124-11146):
// theta advanced from p by repeated fp32 multiplication with theta_scale, then multiplied by freq_scale (linear scaling); the
// NeoX layout (mode 2) multiplies the starting angle by freq_scale as well (ggml.c:11292), so it is scaled twice there.  With
// freq_scale 1 every extra product is exact.
__host__ __device__ inline float rope_angle(float p, int i, int mode, float theta_scale, float freq_scale) {
    float theta = (mode & 2) ? p * freq_scale : p;
    for (int j = 0; j < i; ++j) theta = theta * theta_scale;
    return freq_scale * theta;
}

inline NormArgs to_norm(const pi_norm * n) {
    NormArgs a{0, 0.0f, nullptr, nullptr};
    if (n) { a.kind = n->kind; a.eps = n->eps; a.w = n->w; a.b = n->b; }
    return a;
}

}  // namespace

struct pi_workspace {
    int max_ff, max_d;
    uint32_t *     words;          // [max_ff/32 + 1]
    uint32_t *     words_hot;      // [max_ff/32 + 1]  mask & GPU-resident neurons (Q4_0 fused route)
    unsigned int * counters;       // [64]: [0] predictor ticket, [1..] axpy tile tickets
    float *        partial;        // [kAxpyGroups][max_d]
    int32_t *      hq;             // [max_ff]  Q4_0 axpy: int8 value of h per active row
    float *        hd;             // [max_ff]  and its Q8_0 block scale
    float *        ffn_partial;    // [max(max_ff/32, 32 * 16)][max_d]  partial outputs of the fused sparse FFN / of the batched axpy
    __half *       hc_batch;       // [16][max_ff + 16]  fp16 h of the union rows for a batched step, token-major
    unsigned char * row_any;       // [max_ff]  batched step: neuron active for at least one token
    int            pf_parts, pf_words;   // partial vectors and activity words the last fused F16 launch left for its reduction
};
constexpr int kAxpyGroups = 32;

// launches of kernels_batch.hip that the Q4_0 step kernels reuse
namespace pi {
void launch_union_active(const unsigned char * row_any, int ff, uint32_t * words, int32_t * union_rows, int32_t * n_union, hipStream_t st);
void launch_batch_reduce(const float * partial, int n_groups, int T, int cols, int epilogue, const float * add1, const float * add2, float * out, hipStream_t st);
}

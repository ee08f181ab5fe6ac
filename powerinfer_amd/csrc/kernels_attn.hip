// Attention and the KV cache: RoPE + KV store, decode attention (one workgroup per head; cells split over several workgroups and
// merged), attention of prompt chunks on the matrix cores, K-shift and cache compaction.
#include "kernels_common.hpp"

namespace {

// ---------------------------------------------------------------------------------------------------
// K-shift (llm_build_k_shift, llama.cpp:4332-4381): cached K rows whose position changed by delta[cell] are rotated in place
// by that many positions, the RoPE of fp16 data (ggml_compute_forward_rope_f16, ggml.c:11327-11478): fp16 -> fp32, angle
// delta * theta_i with theta advanced by repeated fp32 multiplication, back to fp16.  Cache layout [row][n_ctx][hd] with
// row = (layer, kv head).  grid = (cells, rows), hd/2 threads; cells with delta 0 are left alone (the reference rotates them
// by angle 0, which returns the same bits).
// ---------------------------------------------------------------------------------------------------
__global__ void k_shift_kernel(__half * __restrict__ k_cache, int n_ctx, int hd, int mode, float theta_scale, float freq_scale,
                               const int32_t * __restrict__ delta) {
    const int cell = blockIdx.x, i = threadIdx.x;
    const int dl = delta[cell];
    if (dl == 0) return;
    __half * row = k_cache + ((size_t)blockIdx.y * n_ctx + cell) * hd;
    const float theta = rope_angle((float)dl, i, mode, theta_scale, freq_scale);
    const float c = cosf(theta), sn = sinf(theta);
    const int i0 = (mode & 2) ? i : 2 * i;
    const int i1 = (mode & 2) ? i + hd / 2 : 2 * i + 1;
    const float x0 = __half2float(row[i0]), x1 = __half2float(row[i1]);
    row[i0] = __float2half_rn(__fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, sn)));
    row[i1] = __float2half_rn(__fadd_rn(__fmul_rn(x0, sn), __fmul_rn(x1, c)));
}

// the same on the reference's own layout, K cells [layer][cell][kv head][hd]: grid = (cells, layers * kv heads)
__global__ void k_shift_cells_kernel(__half * __restrict__ k_cache, int n_cells, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale,
                                     const int32_t * __restrict__ delta) {
    const int cell = blockIdx.x, i = threadIdx.x;
    const int dl = delta[cell];
    if (dl == 0) return;
    const int layer = blockIdx.y / n_head_kv, kvh = blockIdx.y % n_head_kv;
    __half * row = k_cache + (((size_t)layer * n_cells + cell) * n_head_kv + kvh) * hd;
    const float theta = rope_angle((float)dl, i, mode, theta_scale, freq_scale);
    const float c = cosf(theta), sn = sinf(theta);
    const int i0 = (mode & 2) ? i : 2 * i;
    const int i1 = (mode & 2) ? i + hd / 2 : 2 * i + 1;
    const float x0 = __half2float(row[i0]), x1 = __half2float(row[i1]);
    row[i0] = __float2half_rn(__fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, sn)));
    row[i1] = __float2half_rn(__fadd_rn(__fmul_rn(x0, sn), __fmul_rn(x1, c)));
}

// Cell compaction of one cache (K or V) after cells were removed: new cell j takes old cell map[j] (map ascending, so the cells
// keep their order).  Two launches through a staging buffer [rows][n_new][hd] because source and destination ranges overlap.
// grid = (n_new, rows), hd/8 threads (16 bytes each).
__global__ void kv_gather_kernel(const __half * __restrict__ cache, __half * __restrict__ stage, const int32_t * __restrict__ map, int n_new, int n_ctx, int hd) {
    const pi_u32x4 * src = reinterpret_cast<const pi_u32x4 *>(cache + ((size_t)blockIdx.y * n_ctx + map[blockIdx.x]) * hd);
    pi_u32x4 * dst = reinterpret_cast<pi_u32x4 *>(stage + ((size_t)blockIdx.y * n_new + blockIdx.x) * hd);
    dst[threadIdx.x] = src[threadIdx.x];
}
__global__ void kv_place_kernel(__half * __restrict__ cache, const __half * __restrict__ stage, int n_new, int n_ctx, int hd) {
    const pi_u32x4 * src = reinterpret_cast<const pi_u32x4 *>(stage + ((size_t)blockIdx.y * n_new + blockIdx.x) * hd);
    pi_u32x4 * dst = reinterpret_cast<pi_u32x4 *>(cache + ((size_t)blockIdx.y * n_ctx + blockIdx.x) * hd);
    dst[threadIdx.x] = src[threadIdx.x];
}

// ---------------------------------------------------------------------------------------------------
// RoPE + KV store for one token (ggml.c:11163-11325; theta advanced by repeated fp32 multiplication as
// the CPU path does, so the angle is bit-identical and only cosf/sinf may differ in the last place).
// grid = n_head + 2*n_head_kv blocks of hd/2 threads.
// ---------------------------------------------------------------------------------------------------
__global__ void rope_kv_store_kernel(const float * __restrict__ qkv, int n_head, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale,
                                     const int32_t * __restrict__ pos_p, int n_ctx, float * __restrict__ q_rot,
                                     __half * __restrict__ k_cache, __half * __restrict__ v_cache, int qkv_stride, int q_stride) {
    // blockIdx.y = token of a prompt chunk (same sequence, its own position); 0 for single-token decoding
    qkv += (size_t)blockIdx.y * qkv_stride;
    q_rot += (size_t)blockIdx.y * q_stride;
    pos_p += blockIdx.y;
    const int h = blockIdx.x, i = threadIdx.x;           // i = pair index
    const int pos = *pos_p;
    if (h < n_head + n_head_kv) {
        const float * src = qkv + (size_t)h * hd;
        const float theta = rope_angle((float)pos, i, mode, theta_scale, freq_scale);
        const float c = cosf(theta), s = sinf(theta);
        const int i0 = (mode & 2) ? i : 2 * i;
        const int i1 = (mode & 2) ? i + hd / 2 : 2 * i + 1;
        const float x0 = src[i0], x1 = src[i1];
        const float y0 = __fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, s));
        const float y1 = __fadd_rn(__fmul_rn(x0, s), __fmul_rn(x1, c));
        if (h < n_head) {
            q_rot[(size_t)h * hd + i0] = y0;
            q_rot[(size_t)h * hd + i1] = y1;
        } else {
            __half * dst = k_cache + ((size_t)(h - n_head) * n_ctx + pos) * hd;
            dst[i0] = __float2half_rn(y0);
            dst[i1] = __float2half_rn(y1);
        }
    } else {
        const int hv = h - n_head - n_head_kv;
        const float * src = qkv + (size_t)(n_head + n_head_kv + hv) * hd;
        __half * dst = v_cache + ((size_t)hv * n_ctx + pos) * hd;
        dst[2 * i]     = __float2half_rn(src[2 * i]);
        dst[2 * i + 1] = __float2half_rn(src[2 * i + 1]);
    }
}

// ---------------------------------------------------------------------------------------------------
// Decode attention: one block per query head over cells [0, pos].
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void attn_decode_kernel(const float * __restrict__ q_rot, const __half * __restrict__ k_cache,
                                                             const __half * __restrict__ v_cache, int n_head, int n_head_kv, int hd,
                                                             int n_ctx, const int32_t * __restrict__ pos_p, float * __restrict__ out,
                                                             int q_stride, int out_stride, __half * __restrict__ out16) {
    // blockIdx.y = token of a prompt chunk: it sees the cache cells up to its own position (causal mask)
    q_rot += (size_t)blockIdx.y * q_stride;
    out += (size_t)blockIdx.y * out_stride;
    if (out16) out16 += (size_t)blockIdx.y * out_stride;
    pos_p += blockIdx.y;
    extern __shared__ __align__(16) unsigned char smem[];
    float * s    = reinterpret_cast<float *>(smem);               // [n_kv] scores, then probabilities
    float * part = s + n_ctx;                                     // [groups][hd] partial outputs
    __shared__ double red[16];
    __shared__ float redf[16];
    const int h = blockIdx.x, kvh = h / (n_head / n_head_kv);
    const int n_kv = *pos_p + 1;
    const int lpp = hd / 8;                                       // lanes per position (16 B each)
    const int tid = threadIdx.x;
    const int sub = tid % lpp, grp = tid / lpp, ngrp = blockDim.x / lpp;
    const float scale = pi_inv_sqrt((float)hd);

    // q chunk of this lane, rounded to fp16 as the CPU dot does
    float qf[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[i] = pi_round_f16(q_rot[(size_t)h * hd + sub * 8 + i]);

    const __half * kb = k_cache + (size_t)kvh * n_ctx * hd;
    for (int c0 = 0; c0 < n_kv; c0 += ngrp) {
        const int c = c0 + grp;
        float d = 0.0f;
        if (c < n_kv) d = pi_dot8(pi_ld16(kb + (size_t)c * hd + sub * 8), qf, 0.0f);
        for (int o = lpp / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, PI_WAVE);
        if (c < n_kv && sub == 0) s[c] = __fmul_rn(d, scale);
    }
    __syncthreads();

    float mx = -INFINITY;
    for (int c = tid; c < n_kv; c += blockDim.x) mx = fmaxf(mx, s[c]);
    mx = block_max_f32(mx, redf);
    double sum = 0.0;
    for (int c = tid; c < n_kv; c += blockDim.x) {
        // exp through fp16 in and out: the CPU path's lookup table holds fp16(expf(fp32(fp16(x - max))))
        const float e = pi_round_f16(expf(pi_round_f16(__fsub_rn(s[c], mx))));
        s[c] = e;
        sum += (double)e;
    }
    sum = block_sum_f64(sum, red);                                // includes the barriers that publish s[]
    const float inv = (float)(1.0 / sum);

    const __half * vb = v_cache + (size_t)kvh * n_ctx * hd;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    for (int c = grp; c < n_kv; c += ngrp) {
        const float p = pi_round_f16(__fmul_rn(s[c], inv));       // probabilities are rounded to fp16 before the V product
        float vf[8];
        pi_unpack8(pi_ld16(vb + (size_t)c * hd + sub * 8), vf);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = fmaf(vf[i], p, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[grp * hd + sub * 8 + i] = acc[i];
    __syncthreads();
    for (int e = tid; e < hd; e += blockDim.x) {
        float v = part[e];
        for (int g = 1; g < ngrp; ++g) v += part[g * hd + e];
        out[(size_t)h * hd + e] = v;
        if (out16) out16[(size_t)h * hd + e] = __float2half_rn(v);
    }
}

// cos/sin of every (position, pair) the way the CPU path forms them: theta advanced by repeated fp32
// multiplication (ggml.c:11269-11319), so the angle is bit-identical and only cosf/sinf can differ in the
// last place.  table[p][i] = (cos, sin) for pair i of position p.
// ---------------------------------------------------------------------------------------------------
// RoPE + KV store + decode attention in one launch, one workgroup per query head.  The workgroup rotates its
// own q head and the k head of its group (cos/sin from the table), rounds k and v to fp16 as the cache does,
// and attends over cells [0, pos) from the cache plus the new cell from LDS, so it never reads what this
// launch writes; the first query head of each group stores k and v.
// ---------------------------------------------------------------------------------------------------
constexpr int kAttnBlock = 1024;        // 16 waves per head: 64 (hd 128) or 128 (hd 64) cache cells per pass
constexpr int kAttnPre = 4;             // passes whose K and V rows are requested before the prologue
constexpr int kAttnBatch = 4;           // passes behind those whose rows are requested together
// BLOCK threads per head: kAttnBlock for a single sequence and for steps whose workgroups all fit on the chip at once (two of 1024
// threads per compute unit); half of that where they do not (16 sequences x 40 heads are 640 workgroups against 512 places: a
// quarter of the units ran a second round, 48 us at 530 cells; with 512 threads four fit a unit and all 640 run together).
template <int BLOCK>
__global__ __launch_bounds__(BLOCK, 8) void attn_fused_kernel(const float * __restrict__ qkv, const float2 * __restrict__ rope_table,
                                                            __half * __restrict__ k_cache, __half * __restrict__ v_cache,
                                                            int n_head, int n_head_kv, int hd, int mode, int n_ctx,
                                                            const int32_t * __restrict__ pos_p, float * __restrict__ out,
                                                            int qkv_stride, size_t cache_seq_stride, int out_stride, __half * __restrict__ out16, int out16_ol,
                                                            int8_t * __restrict__ q8_q, float * __restrict__ q8_d, int * __restrict__ q8_s) {
    // q8_q != nullptr: the output also as the Q8_0 blocks an integer mat-mul of a Q4_0 matrix multiplies with (the blocks, scales and
    // -8 * sums pi_k_norm_q8_blocks makes of the same values: a head's hd outputs are whole blocks of 32, one per half-wave)
    // blockIdx.y = sequence of a batched step (its own token, position and cache); 0 for single-sequence decoding
    // out16_ol != 0: the fp16 copy in the operand layout of the 16-token mat-muls (pi_ol_index) instead of [sequence][out_stride]
    qkv += (size_t)blockIdx.y * qkv_stride;
    k_cache += (size_t)blockIdx.y * cache_seq_stride;
    v_cache += (size_t)blockIdx.y * cache_seq_stride;
    out += (size_t)blockIdx.y * out_stride;
    if (out16 && !out16_ol) out16 += (size_t)blockIdx.y * out_stride;      // optional fp16 copy: the input of the next mat-mul of a batched step
    pos_p += blockIdx.y;
    extern __shared__ __align__(16) unsigned char smem[];
    float * s    = reinterpret_cast<float *>(smem);               // [n_ctx] scores, then probabilities
    float * part = s + n_ctx;                                     // [groups][hd]
    float * qs   = part + (BLOCK / (hd / 8)) * hd;                    // [hd] rotated q, rounded to fp16
    float * kcur = qs + hd;                                       // [hd] rotated k of this position, rounded to fp16
    float * vcur = kcur + hd;                                     // [hd]
    __shared__ double red[16];
    __shared__ float redf[16];
    const int h = blockIdx.x, grp_sz = n_head / n_head_kv, kvh = h / grp_sz;
    const int tid = threadIdx.x;
    const int pos = *pos_p, n_kv = pos + 1;
    const float * qsrc = qkv + (size_t)h * hd;
    const float * ksrc = qkv + (size_t)(n_head + kvh) * hd;
    const float * vsrc = qkv + (size_t)(n_head + n_head_kv + kvh) * hd;
    __half * kdst = k_cache + ((size_t)kvh * n_ctx + pos) * hd;
    __half * vdst = v_cache + ((size_t)kvh * n_ctx + pos) * hd;
    const bool leader = (h % grp_sz) == 0;
    // the cache cells of the first kAttnPre passes do not depend on anything computed here: their K and V rows are requested
    // now and travel during the rotation, the scores and the softmax (one memory round trip instead of three in a row)
    const int lpp = hd / 8;
    const int sub = tid % lpp, grp = tid / lpp, ngrp = BLOCK / lpp;
    const __half * kb = k_cache + (size_t)kvh * n_ctx * hd;
    const __half * vb = v_cache + (size_t)kvh * n_ctx * hd;
    pi_u32x4 kpre[kAttnPre], vpre[kAttnPre];
#pragma unroll
    for (int i = 0; i < kAttnPre; ++i) {
        const int c = i * ngrp + grp;
        if (c < pos) { kpre[i] = pi_ld16(kb + (size_t)c * hd + sub * 8); vpre[i] = pi_ld16(vb + (size_t)c * hd + sub * 8); }
    }
    if (tid < hd / 2) {
        const float2 cs = rope_table[(size_t)pos * (hd / 2) + tid];
        const int i0 = (mode & 2) ? tid : 2 * tid;
        const int i1 = (mode & 2) ? tid + hd / 2 : 2 * tid + 1;
        const float q0 = qsrc[i0], q1 = qsrc[i1], k0 = ksrc[i0], k1 = ksrc[i1];
        qs[i0] = pi_round_f16(__fsub_rn(__fmul_rn(q0, cs.x), __fmul_rn(q1, cs.y)));
        qs[i1] = pi_round_f16(__fadd_rn(__fmul_rn(q0, cs.y), __fmul_rn(q1, cs.x)));
        const __half ka = __float2half_rn(__fsub_rn(__fmul_rn(k0, cs.x), __fmul_rn(k1, cs.y)));
        const __half kb = __float2half_rn(__fadd_rn(__fmul_rn(k0, cs.y), __fmul_rn(k1, cs.x)));
        kcur[i0] = __half2float(ka); kcur[i1] = __half2float(kb);
        if (leader) { kdst[i0] = ka; kdst[i1] = kb; }
    } else if (tid < hd / 2 + hd) {
        const int e = tid - hd / 2;
        const __half v = __float2half_rn(vsrc[e]);
        vcur[e] = __half2float(v);
        if (leader) vdst[e] = v;
    }
    __syncthreads();

    const float scale = pi_inv_sqrt((float)hd);
    float qf[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[i] = qs[sub * 8 + i];
#pragma unroll
    for (int i = 0; i < kAttnPre; ++i) {
        if (i * ngrp < n_kv) {
            const int c = i * ngrp + grp;
            float d = 0.0f;
            if (c < pos) d = pi_dot8(kpre[i], qf, 0.0f);
            else if (c == pos) {
#pragma unroll
                for (int k = 0; k < 8; ++k) d = fmaf(kcur[sub * 8 + k], qf[k], d);
            }
            for (int o = lpp / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, PI_WAVE);
            if (c < n_kv && sub == 0) s[c] = __fmul_rn(d, scale);
        }
    }
    // the passes behind the prefetched ones, kAttnBatch at a time: their rows are requested together and cost one trip to memory
    // instead of one each (the same dots in the same order)
    for (int c0 = kAttnPre * ngrp; c0 < n_kv; c0 += kAttnBatch * ngrp) {
        pi_u32x4 kk[kAttnBatch];
#pragma unroll
        for (int u = 0; u < kAttnBatch; ++u) {
            const int c = c0 + u * ngrp + grp;
            if (c < pos) kk[u] = pi_ld16(kb + (size_t)c * hd + sub * 8);
        }
#pragma unroll
        for (int u = 0; u < kAttnBatch; ++u) {
            if (c0 + u * ngrp < n_kv) {
                const int c = c0 + u * ngrp + grp;
                float d = 0.0f;
                if (c < pos) d = pi_dot8(kk[u], qf, 0.0f);
                else if (c == pos) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) d = fmaf(kcur[sub * 8 + i], qf[i], d);
                }
                for (int o = lpp / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, PI_WAVE);
                if (c < n_kv && sub == 0) s[c] = __fmul_rn(d, scale);
            }
        }
    }
    __syncthreads();

    float mx = -INFINITY;
    for (int c = tid; c < n_kv; c += BLOCK) mx = fmaxf(mx, s[c]);
    mx = block_max_f32(mx, redf);
    double sum = 0.0;
    for (int c = tid; c < n_kv; c += BLOCK) {
        const float e = pi_round_f16(expf(pi_round_f16(__fsub_rn(s[c], mx))));
        s[c] = e;
        sum += (double)e;
    }
    sum = block_sum_f64(sum, red);
    const float inv = (float)(1.0 / sum);

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int i = 0; i < kAttnPre; ++i) {
        const int c = i * ngrp + grp;
        if (c < n_kv) {
            const float p = pi_round_f16(__fmul_rn(s[c], inv));
            float vf[8];
            if (c < pos) pi_unpack8(vpre[i], vf);
            else {
#pragma unroll
                for (int k = 0; k < 8; ++k) vf[k] = vcur[sub * 8 + k];
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) acc[k] = fmaf(vf[k], p, acc[k]);
        }
    }
    for (int c0 = kAttnPre * ngrp; c0 < n_kv; c0 += kAttnBatch * ngrp) {
        pi_u32x4 vv[kAttnBatch];
#pragma unroll
        for (int u = 0; u < kAttnBatch; ++u) {
            const int c = c0 + u * ngrp + grp;
            if (c < pos) vv[u] = pi_ld16(vb + (size_t)c * hd + sub * 8);
        }
#pragma unroll
        for (int u = 0; u < kAttnBatch; ++u) {
            const int c = c0 + u * ngrp + grp;
            if (c < n_kv) {
                const float p = pi_round_f16(__fmul_rn(s[c], inv));
                float vf[8];
                if (c < pos) pi_unpack8(vv[u], vf);
                else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) vf[i] = vcur[sub * 8 + i];
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] = fmaf(vf[i], p, acc[i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[grp * hd + sub * 8 + i] = acc[i];
    __syncthreads();
    for (int e = tid; e < hd; e += BLOCK) {
        float v = part[e];
        for (int g = 1; g < ngrp; ++g) v += part[g * hd + e];
        out[(size_t)h * hd + e] = v;
        if (out16) out16[out16_ol ? pi_ol_index(blockIdx.y, h * hd + e) : (size_t)h * hd + e] = __float2half_rn(v);
        if (q8_q) {                                               // (hd % 32 == 0: the lanes of a block run this together)
            float amax = fabsf(v);
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, PI_WAVE));
            const float d = pi_round_f16(pi_div(amax, 127.0f)), id = (amax != 0.0f) ? pi_div(127.0f, amax) : 0.0f;
            const int q = (int)rintf(__fmul_rn(v, id));
            int sq = q;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) sq += __shfl_xor(sq, o, PI_WAVE);
            const int i = h * hd + e, eb = i & 31, t = blockIdx.y;
            q8_q[(((size_t)(i >> 5) * 4 + ((eb & 15) >> 2)) * 16 + t) * 8 + (eb >> 4) * 4 + (eb & 3)] = (int8_t)q;
            if (eb == 0) { q8_d[(size_t)(i >> 5) * 16 + t] = d; q8_s[(size_t)(i >> 5) * 16 + t] = -8 * sq; }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Attention of one token with the cache cells of a head split over several workgroups (grid: head x part x sequence).  A compute unit
// pulls about 1/256 of the chip's HBM rate, so one workgroup per head leaves the K / V rows of a long context to 32 or 128 units
// (18 us per 7B layer at 600 cells, growing by 2.4 us per 100 cells); with n_parts workgroups per head every unit takes a share and
// the score buffer in LDS holds n_ctx / n_parts cells instead of all of them.
// Part s owns cells [n_kv * s / n, n_kv * (s + 1) / n); the last part holds the new cell: it rotates and stores k, stores v, and
// uses them from LDS.  Every part rotates q, computes its scores, e_i = fp16(exp(fp16(s_i - m))) with ITS maximum m (the rounding
// points of the CPU path's table, ggml.c:10747-10759), l = sum e_i in double and acc = sum v_i * e_i, and hands (m, l, acc) to
// attn_merge_kernel, which rescales by exp(m - M), adds the parts in order and divides by the total.  Against one workgroup per head,
// which knows the global maximum before it rounds, results differ in the last places of the fp16 roundings (1e-4 of the output).
// ---------------------------------------------------------------------------------------------------
// FROM_CACHE: the token's own K / V row is in the cache already and qkv holds its rotated q only ([n_head * hd] per token; a prompt chunk
// behind rope_kv_store_kernel): nothing is rotated or stored, every cell is read from the cache.
constexpr int kAttnPartBlock = 512;
constexpr int kAttnPartPre = 4;
template <bool FROM_CACHE>
__global__ __launch_bounds__(kAttnPartBlock) void attn_part_kernel(const float * __restrict__ qkv, const float2 * __restrict__ rope_table,
                                                                   __half * __restrict__ k_cache, __half * __restrict__ v_cache,
                                                                   int n_head, int n_head_kv, int hd, int mode, int n_ctx, int s_cap,
                                                                   const int32_t * __restrict__ pos_p, float * __restrict__ part_acc, float * __restrict__ part_ml,
                                                                   int qkv_stride, size_t cache_seq_stride) {
    qkv += (size_t)blockIdx.z * qkv_stride;
    k_cache += (size_t)blockIdx.z * cache_seq_stride;
    v_cache += (size_t)blockIdx.z * cache_seq_stride;
    pos_p += blockIdx.z;
    extern __shared__ __align__(16) unsigned char smem[];
    float * s    = reinterpret_cast<float *>(smem);               // [s_cap] scores of this part, then e_i
    float * part = s + s_cap;                                     // [groups][hd]
    float * qs   = part + (kAttnPartBlock / (hd / 8)) * hd;       // [hd] rotated q, rounded to fp16
    float * kcur = qs + hd;                                       // [hd] rotated k of this position, rounded to fp16
    float * vcur = kcur + hd;                                     // [hd]
    __shared__ double red[16];
    __shared__ float redf[16];
    const int h = blockIdx.x, n_parts = gridDim.y, sp = blockIdx.y, grp_sz = n_head / n_head_kv, kvh = h / grp_sz;
    const int tid = threadIdx.x;
    const int pos = *pos_p, n_kv = pos + 1;
    const int lo = (int)((long long)n_kv * sp / n_parts), hi = (int)((long long)n_kv * (sp + 1) / n_parts);
    const bool owns_new = !FROM_CACHE && sp == n_parts - 1;        // hi == n_kv: the new cell is this part's last
    const size_t slot = ((size_t)blockIdx.z * n_head + h) * n_parts + sp;
    if (hi - lo > s_cap) return;                                  // cannot happen for pos < n_ctx (the launcher sizes s_cap); never write past LDS
    const float * qsrc = qkv + (size_t)h * hd;
    const float * ksrc = qkv + (size_t)(n_head + kvh) * hd;
    const float * vsrc = qkv + (size_t)(n_head + n_head_kv + kvh) * hd;
    const int lpp = hd / 8;
    const int sub = tid % lpp, grp = tid / lpp, ngrp = kAttnPartBlock / lpp;
    const __half * kb = k_cache + (size_t)kvh * n_ctx * hd;
    const __half * vb = v_cache + (size_t)kvh * n_ctx * hd;
    const int n_old = (owns_new ? hi - 1 : hi) - lo;              // cells of this part that live in the cache
    pi_u32x4 kpre[kAttnPartPre], vpre[kAttnPartPre];
#pragma unroll
    for (int i = 0; i < kAttnPartPre; ++i) {
        const int c = i * ngrp + grp;
        if (c < n_old) { kpre[i] = pi_ld16(kb + (size_t)(lo + c) * hd + sub * 8); vpre[i] = pi_ld16(vb + (size_t)(lo + c) * hd + sub * 8); }
    }
    if (FROM_CACHE) {
        if (tid < hd) qs[tid] = pi_round_f16(qsrc[tid]);
    } else if (tid < hd / 2) {
        const float2 cs = rope_table[(size_t)pos * (hd / 2) + tid];
        const int i0 = (mode & 2) ? tid : 2 * tid;
        const int i1 = (mode & 2) ? tid + hd / 2 : 2 * tid + 1;
        const float q0 = qsrc[i0], q1 = qsrc[i1];
        qs[i0] = pi_round_f16(__fsub_rn(__fmul_rn(q0, cs.x), __fmul_rn(q1, cs.y)));
        qs[i1] = pi_round_f16(__fadd_rn(__fmul_rn(q0, cs.y), __fmul_rn(q1, cs.x)));
        if (owns_new) {
            const float k0 = ksrc[i0], k1 = ksrc[i1];
            const __half ka = __float2half_rn(__fsub_rn(__fmul_rn(k0, cs.x), __fmul_rn(k1, cs.y)));
            const __half kc = __float2half_rn(__fadd_rn(__fmul_rn(k0, cs.y), __fmul_rn(k1, cs.x)));
            kcur[i0] = __half2float(ka); kcur[i1] = __half2float(kc);
            if ((h % grp_sz) == 0) { __half * kdst = k_cache + ((size_t)kvh * n_ctx + pos) * hd; kdst[i0] = ka; kdst[i1] = kc; }
        }
    } else if (owns_new && tid < hd / 2 + hd) {
        const int e = tid - hd / 2;
        const __half v = __float2half_rn(vsrc[e]);
        vcur[e] = __half2float(v);
        if ((h % grp_sz) == 0) v_cache[((size_t)kvh * n_ctx + pos) * hd + e] = v;
    }
    __syncthreads();

    const float scale = pi_inv_sqrt((float)hd);
    const int n_mine = hi - lo;
    float qf[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[i] = qs[sub * 8 + i];
#pragma unroll
    for (int i = 0; i < kAttnPartPre; ++i) {
        if (i * ngrp < n_mine) {
            const int c = i * ngrp + grp;
            float d = 0.0f;
            if (c < n_old) d = pi_dot8(kpre[i], qf, 0.0f);
            else if (c < n_mine) {
#pragma unroll
                for (int k = 0; k < 8; ++k) d = fmaf(kcur[sub * 8 + k], qf[k], d);
            }
            for (int o = lpp / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, PI_WAVE);
            if (c < n_mine && sub == 0) s[c] = __fmul_rn(d, scale);
        }
    }
    for (int c0 = kAttnPartPre * ngrp; c0 < n_mine; c0 += ngrp) {
        const int c = c0 + grp;
        float d = 0.0f;
        if (c < n_old) d = pi_dot8(pi_ld16(kb + (size_t)(lo + c) * hd + sub * 8), qf, 0.0f);
        else if (c < n_mine) {
#pragma unroll
            for (int i = 0; i < 8; ++i) d = fmaf(kcur[sub * 8 + i], qf[i], d);
        }
        for (int o = lpp / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, PI_WAVE);
        if (c < n_mine && sub == 0) s[c] = __fmul_rn(d, scale);
    }
    __syncthreads();

    float mx = -INFINITY;
    for (int c = tid; c < n_mine; c += kAttnPartBlock) mx = fmaxf(mx, s[c]);
    mx = block_max_f32(mx, redf);
    double sum = 0.0;
    for (int c = tid; c < n_mine; c += kAttnPartBlock) {
        const float e = pi_round_f16(expf(pi_round_f16(__fsub_rn(s[c], mx))));
        s[c] = e;
        sum += (double)e;
    }
    sum = block_sum_f64(sum, red);

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int i = 0; i < kAttnPartPre; ++i) {
        const int c = i * ngrp + grp;
        if (c < n_mine) {
            const float p = s[c];
            float vf[8];
            if (c < n_old) pi_unpack8(vpre[i], vf);
            else {
#pragma unroll
                for (int k = 0; k < 8; ++k) vf[k] = vcur[sub * 8 + k];
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) acc[k] = fmaf(vf[k], p, acc[k]);
        }
    }
    for (int c = kAttnPartPre * ngrp + grp; c < n_mine; c += ngrp) {
        const float p = s[c];
        float vf[8];
        if (c < n_old) pi_unpack8(pi_ld16(vb + (size_t)(lo + c) * hd + sub * 8), vf);
        else {
#pragma unroll
            for (int i = 0; i < 8; ++i) vf[i] = vcur[sub * 8 + i];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = fmaf(vf[i], p, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[grp * hd + sub * 8 + i] = acc[i];
    __syncthreads();
    for (int e = tid; e < hd; e += kAttnPartBlock) {
        float v = part[e];
        for (int g = 1; g < ngrp; ++g) v += part[g * hd + e];
        part_acc[slot * hd + e] = v;
    }
    if (tid == 0) { part_ml[slot * 2] = n_mine > 0 ? mx : -INFINITY; part_ml[slot * 2 + 1] = (float)sum; }
}

// out[h][e] = sum_s acc_s[e] * exp(m_s - M) / sum_s l_s * exp(m_s - M), parts in ascending order; one workgroup of hd threads per head
__global__ void attn_merge_kernel(const float * __restrict__ part_acc, const float * __restrict__ part_ml, int n_parts, int hd,
                                  float * __restrict__ out, int out_stride, __half * __restrict__ out16) {
    const int h = blockIdx.x, n_head = gridDim.x, e = threadIdx.x;
    const size_t slot0 = ((size_t)blockIdx.y * n_head + h) * n_parts;
    float M = -INFINITY;
    for (int sp = 0; sp < n_parts; ++sp) M = fmaxf(M, part_ml[(slot0 + sp) * 2]);
    float L = 0.0f, v = 0.0f;
    for (int sp = 0; sp < n_parts; ++sp) {
        const float m = part_ml[(slot0 + sp) * 2], l = part_ml[(slot0 + sp) * 2 + 1];
        if (l > 0.0f) {
            const float w = expf(__fsub_rn(m, M));
            L = fmaf(l, w, L);
            v = fmaf(part_acc[(slot0 + sp) * hd + e], w, v);
        }
    }
    v = pi_div(v, L);
    out[(size_t)blockIdx.y * out_stride + (size_t)h * hd + e] = v;
    if (out16) out16[(size_t)blockIdx.y * out_stride + (size_t)h * hd + e] = __float2half_rn(v);
}

// ---------------------------------------------------------------------------------------------------
// Attention of a prompt chunk on the matrix cores: a workgroup owns 16 consecutive tokens of one query head and the four waves
// split the cache cells.  Three phases, with the rounding points of attn_decode_kernel (and so of the CPU path):
//   1. scores: S[cell][token] = K[cell] . fp16(q[token]) by 16x16x32 MFMAs (a K row is read in operand layout straight from
//      the cache, q stays in registers), times 1/sqrt(hd), into LDS as s[token][cell];
//   2. softmax per token over the cells it may see (cell <= its position): maximum, fp16(exp(fp16(s - max))), the sum in double,
//      p = fp16(e / sum); cells beyond the token's position become exact zeros;
//   3. out[token][:] = sum over cells of p * V[cell][:]: the V cache keeps a cell's head contiguous, the MFMA wants eight cells of
//      one column per lane, so a wave reads eight cells of a column pair (4 bytes per lane, a whole row per instruction), packs
//      them with two byte permutes per pair of cells and drops two 16-byte columns into its private LDS tile (32 cells a tile),
//      from where the operand comes back with one 16-byte read.  No workgroup barrier inside the loops: the tile belongs to one
//      wave and the LDS operations of a wave complete in order.  The waves' partial outputs meet in LDS in wave order.
// HD = 128 or 64.  LDS: 16 x (cells rounded up to 32, + 4) floats of scores + 4 x HD x 80 bytes of V tiles.
// ---------------------------------------------------------------------------------------------------
constexpr int kAcVtStride = 40;                // halves per row of the transposed V tile: 32 cells + 8 of padding (conflict-free both ways)
template <int HD>
__global__ __launch_bounds__(kBlock) void attn_chunk_mfma_kernel(const float * __restrict__ q_rot, const __half * __restrict__ k_cache,
                                                                 const __half * __restrict__ v_cache, int n_head, int n_head_kv, int n_ctx,
                                                                 const int32_t * __restrict__ pos_p, int T, float * __restrict__ out,
                                                                 int q_stride, int out_stride, __half * __restrict__ out16, int s_stride) {
    static_assert(HD == 128 || HD == 64, "head size");
    extern __shared__ __align__(16) unsigned char smem[];
    float * s = reinterpret_cast<float *>(smem);                                       // [16][s_stride]
    unsigned char * vt_all = smem + sizeof(float) * 16 * (size_t)s_stride;             // [4 waves][HD][kAcVtStride] halves
    const int h = blockIdx.x, kvh = h / (n_head / n_head_kv);
    const int t0 = blockIdx.y * 16;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i = lane & 15, g = lane >> 4;
    // cells the furthest-reaching token of the tile sees
    int n_kv = pos_p[min(t0 + i, T - 1)] + 1;
    for (int o = 8; o > 0; o >>= 1) n_kv = max(n_kv, __shfl_xor(n_kv, o, PI_WAVE));
    n_kv = min(n_kv, s_stride - 4);                // the launcher sized the scores for the cells its caller announced
    const int n_t16 = (n_kv + 15) / 16, n_t32 = (n_kv + 31) / 32;

    // ---- 1. scores --------------------------------------------------------------------------------------------------------
    {
        const float * qp = q_rot + (size_t)min(t0 + i, T - 1) * q_stride + (size_t)h * HD + 8 * g;
        pi_h8 qf[HD / 32];
#pragma unroll
        for (int ks = 0; ks < HD / 32; ++ks) {
            const float4 a = *reinterpret_cast<const float4 *>(qp + ks * 32), b = *reinterpret_cast<const float4 *>(qp + ks * 32 + 4);
            qf[ks] = pi_h8{(_Float16)a.x, (_Float16)a.y, (_Float16)a.z, (_Float16)a.w, (_Float16)b.x, (_Float16)b.y, (_Float16)b.z, (_Float16)b.w};
        }
        const float scale = pi_inv_sqrt((float)HD);
        const __half * kb = k_cache + (size_t)kvh * n_ctx * HD + 8 * g;
        // six tiles of K rows are in flight per wave: the loads come from L2 and a wave has little else to hide their latency behind
        constexpr int D1 = 6;
        pi_u32x4 a[D1][HD / 32];
        // (requests past the last tile re-read the last cell: unconditional loads keep the count of outstanding ones static, which
        // is what lets the compiler wait for the oldest tile only)
        auto issue = [&](pi_u32x4 * dst, int kt) {
            const int c = min(kt * 16 + i, n_kv - 1);
#pragma unroll
            for (int ks = 0; ks < HD / 32; ++ks) dst[ks] = pi_ld16(kb + (size_t)c * HD + ks * 32);
        };
#pragma unroll
        for (int u = 0; u < D1; ++u) issue(a[u], wave + u * kWavesPerBlock);
        for (int kt0 = wave; kt0 < n_t16; kt0 += D1 * kWavesPerBlock) {
#pragma unroll
            for (int u = 0; u < D1; ++u) {
                const int kt = kt0 + u * kWavesPerBlock;
                if (kt < n_t16) {
                    pi_f4 acc = pi_f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int ks = 0; ks < HD / 32; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, a[u][ks]), qf[ks], acc, 0, 0, 0);
                    // acc[r] = S[cell kt*16 + 4g + r][token i]
                    *reinterpret_cast<float4 *>(s + (size_t)i * s_stride + kt * 16 + 4 * g) =
                        float4{__fmul_rn(acc[0], scale), __fmul_rn(acc[1], scale), __fmul_rn(acc[2], scale), __fmul_rn(acc[3], scale)};
                }
                issue(a[u], kt + D1 * kWavesPerBlock);
            }
        }
    }
    __syncthreads();

    // ---- 2. softmax: 16 lanes per token, four cells per lane and step ------------------------------------------------------------
    {
        const int q = threadIdx.x >> 4, j = threadIdx.x & 15;
        const int nq = min(pos_p[min(t0 + q, T - 1)] + 1, n_kv);
        float * sq = s + (size_t)q * s_stride;
        float mx = -INFINITY;
        for (int c = 4 * j; c < nq; c += 64) {
            const float4 v = *reinterpret_cast<const float4 *>(sq + c);
            mx = fmaxf(mx, v.x);
            if (c + 1 < nq) mx = fmaxf(mx, v.y);
            if (c + 2 < nq) mx = fmaxf(mx, v.z);
            if (c + 3 < nq) mx = fmaxf(mx, v.w);
        }
        for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, PI_WAVE));
        double sum = 0.0;
        for (int c = 4 * j; c < nq; c += 64) {
            float4 v = *reinterpret_cast<const float4 *>(sq + c);
            // exp through fp16 in and out, as the CPU path's lookup table does; cells past the token's own position count as zero
            v.x = pi_round_f16(expf(pi_round_f16(__fsub_rn(v.x, mx))));
            v.y = c + 1 < nq ? pi_round_f16(expf(pi_round_f16(__fsub_rn(v.y, mx)))) : 0.0f;
            v.z = c + 2 < nq ? pi_round_f16(expf(pi_round_f16(__fsub_rn(v.z, mx)))) : 0.0f;
            v.w = c + 3 < nq ? pi_round_f16(expf(pi_round_f16(__fsub_rn(v.w, mx)))) : 0.0f;
            *reinterpret_cast<float4 *>(sq + c) = v;
            sum += (double)v.x; sum += (double)v.y; sum += (double)v.z; sum += (double)v.w;
        }
        for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, PI_WAVE);
        const float inv = (float)(1.0 / sum);
        for (int c = 4 * j; c < n_t32 * 32; c += 64) {
            float4 v = float4{0.0f, 0.0f, 0.0f, 0.0f};
            if (c < nq) {
                v = *reinterpret_cast<const float4 *>(sq + c);
                v.x = pi_round_f16(__fmul_rn(v.x, inv)); v.y = pi_round_f16(__fmul_rn(v.y, inv));
                v.z = pi_round_f16(__fmul_rn(v.z, inv)); v.w = pi_round_f16(__fmul_rn(v.w, inv));       // zeros past nq stay zeros
            }
            *reinterpret_cast<float4 *>(sq + c) = v;
        }
    }
    __syncthreads();

    // ---- 3. p . V -------------------------------------------------------------------------------------------------------------
    pi_f4 acc[HD / 16];
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) acc[dt] = pi_f4{0.0f, 0.0f, 0.0f, 0.0f};
    unsigned char * myvt = vt_all + (size_t)wave * HD * kAcVtStride * 2;
    {
        constexpr int LPR = HD / 2;                 // lanes per V row, 4 bytes (a column pair) each
        constexpr int GPI = PI_WAVE / LPR;          // groups of eight cells per load instruction
        const int dp = lane % LPR, sub = lane / LPR;
        const __half * vb = v_cache + (size_t)kvh * n_ctx * HD + 2 * dp;
        // the cells of the next three tiles are on their way while a tile is packed and multiplied; cells past the end may hold
        // anything and enter as zeros
        constexpr int D3 = 3;
        unsigned vq[D3][4 / GPI][8];
        auto issue = [&](unsigned (*dst)[8], int kt) {
#pragma unroll
            for (int rnd = 0; rnd < 4 / GPI; ++rnd)
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int c = kt * 32 + (rnd * GPI + sub) * 8 + k;
                    dst[rnd][k] = *reinterpret_cast<const unsigned *>(vb + (size_t)min(c, n_kv - 1) * HD);
                }
        };
#pragma unroll
        for (int u = 0; u < D3; ++u) issue(vq[u], wave + u * kWavesPerBlock);
        for (int kt0 = wave; kt0 < n_t32; kt0 += D3 * kWavesPerBlock) {
#pragma unroll
            for (int u = 0; u < D3; ++u) {
                const int kt = kt0 + u * kWavesPerBlock;
                if (kt < n_t32) {
                    const int c0 = kt * 32;
#pragma unroll
                    for (int rnd = 0; rnd < 4 / GPI; ++rnd) {
                        const int grp8 = rnd * GPI + sub;   // which eight cells of the tile
                        unsigned v[8];
#pragma unroll
                        for (int k = 0; k < 8; ++k) v[k] = c0 + grp8 * 8 + k < n_kv ? vq[u][rnd][k] : 0u;
                        pi_u32x4 lo, hi;
                        lo.x = __builtin_amdgcn_perm(v[1], v[0], 0x05040100u); hi.x = __builtin_amdgcn_perm(v[1], v[0], 0x07060302u);
                        lo.y = __builtin_amdgcn_perm(v[3], v[2], 0x05040100u); hi.y = __builtin_amdgcn_perm(v[3], v[2], 0x07060302u);
                        lo.z = __builtin_amdgcn_perm(v[5], v[4], 0x05040100u); hi.z = __builtin_amdgcn_perm(v[5], v[4], 0x07060302u);
                        lo.w = __builtin_amdgcn_perm(v[7], v[6], 0x05040100u); hi.w = __builtin_amdgcn_perm(v[7], v[6], 0x07060302u);
                        *reinterpret_cast<pi_u32x4 *>(myvt + ((size_t)(2 * dp) * kAcVtStride + grp8 * 8) * 2) = lo;
                        *reinterpret_cast<pi_u32x4 *>(myvt + ((size_t)(2 * dp + 1) * kAcVtStride + grp8 * 8) * 2) = hi;
                    }
                    const float * pp = s + (size_t)i * s_stride + c0 + 8 * g;
                    const float4 p0 = *reinterpret_cast<const float4 *>(pp), p1 = *reinterpret_cast<const float4 *>(pp + 4);
                    const pi_h8 pa = pi_h8{(_Float16)p0.x, (_Float16)p0.y, (_Float16)p0.z, (_Float16)p0.w, (_Float16)p1.x, (_Float16)p1.y, (_Float16)p1.z, (_Float16)p1.w};
#pragma unroll
                    for (int dt = 0; dt < HD / 16; ++dt) {
                        const pi_u32x4 b = *reinterpret_cast<const pi_u32x4 *>(myvt + ((size_t)(dt * 16 + i) * kAcVtStride + 8 * g) * 2);
                        acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, __builtin_bit_cast(pi_h8, b), acc[dt], 0, 0, 0);
                    }
                }
                issue(vq[u], kt + D3 * kWavesPerBlock);
            }
        }
    }
    // acc[dt][r] = out[token 4g + r][dt*16 + i] over this wave's cells; the four partial tiles meet in wave order
    constexpr int PS = HD + 4;
    float * mypart = reinterpret_cast<float *>(myvt);                                  // [16][PS], inside the wave's own tile
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) mypart[(4 * g + r) * PS + dt * 16 + i] = acc[dt][r];
    __syncthreads();
    for (int e = threadIdx.x; e < 16 * HD; e += kBlock) {
        const int q = e / HD, d = e % HD, t = t0 + q;
        if (t < T) {
            float v = 0.0f;
#pragma unroll
            for (int w = 0; w < kWavesPerBlock; ++w) v += reinterpret_cast<const float *>(vt_all + (size_t)w * HD * kAcVtStride * 2)[q * PS + d];
            out[(size_t)t * out_stride + (size_t)h * HD + d] = v;
            if (out16) out16[(size_t)t * out_stride + (size_t)h * HD + d] = __float2half_rn(v);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// One token's attention on the layouts of the reference's own KV cache (llm_build_kv_store / llm_build_kqv, llama.cpp:4383-4418,
// 4764-4850): K cells [cell][n_head_kv * hd] fp16, V transposed [n_head_kv * hd][n_ctx] fp16.  What its graph spreads over eleven nodes
// - RoPE of q and k, the two copies into the cache, K.q, scale, + mask, soft-max, V.p and the gather of the heads - is one launch, one
// workgroup per query head, with the CPU path's rounding points: q and p rounded to fp16 in front of their products (the mat-muls
// against fp16 operands, ggml.c:9703-9716), exp through fp16 on both sides (ggml.c:10747-10759), the sum of the exponentials in double.
// The new cell's K and V rows are used from LDS (every head of a group computes them, the group's first head stores them), so no
// workgroup depends on another's stores.  Cells whose mask entry is -inf get probability 0 whatever the cache holds there.
// RoPE as rope_kernel of the boundary computes it: angle advanced by repeated fp32 multiplication, cosf / sinf, * mscale.
// ---------------------------------------------------------------------------------------------------
// A step of T tokens (grid.y; token u's q, k, v at stride tok_stride, its cell cell0 + u, its mask row at mask_stride, its output at
// out_stride): the K and V rows of all T new cells are formed in LDS by every workgroup, so a token attends the other tokens of its
// step (where its mask allows) without waiting for their stores - what the reference gets by storing the whole batch first.
__global__ __launch_bounds__(kBlock) void attn_ggml_kernel(const float * __restrict__ q, const float * __restrict__ k, const float * __restrict__ v, int tok_stride,
                                                           const int32_t * __restrict__ pos, int mode, float theta_scale, float freq_scale, float mscale,
                                                           __half * __restrict__ k_cache, __half * __restrict__ v_cache,
                                                           int n_head, int n_head_kv, int hd, int n_ctx, int n_kv, int T, int cell0,
                                                           const float * __restrict__ kq_scale, const float * __restrict__ kq_mask, int mask_stride,
                                                           float * __restrict__ out, int out_stride) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int n_kv8 = (n_kv + 7) & ~7;                                     // the V rows are read eight cells at a time
    float * sc = reinterpret_cast<float *>(smem);                          // [n_kv8] scores, then probabilities (zeros behind n_kv)
    __half * q16 = reinterpret_cast<__half *>(sc + n_kv8);                 // [hd]
    __half * k16 = q16 + hd;                                               // [T][hd] the step's new K rows
    __half * v16 = k16 + (size_t)T * hd;                                   // [T][hd] and V rows
    __shared__ double red[kWavesPerBlock];
    __shared__ float  redf[kWavesPerBlock];
    const int h = blockIdx.x, tok = blockIdx.y, kvh = h / (n_head / n_head_kv), gqa = n_head_kv * hd;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const bool owner = h % (n_head / n_head_kv) == 0;                      // this head's workgroup stores the group's new K / V rows of its token
    const int cell = cell0 + tok;
    kq_mask += (size_t)tok * mask_stride;
    out += (size_t)tok * out_stride;
    if (tid < hd / 2) {
        const int i = tid;
        const int i0 = (mode & 2) ? i : 2 * i, i1 = (mode & 2) ? i + hd / 2 : 2 * i + 1;
        for (int u = 0; u < T; ++u) {
            float theta = (float)pos[u];
            if (mode & 2) theta = __fmul_rn(theta, freq_scale);
            for (int j = 0; j < i; ++j) theta = __fmul_rn(theta, theta_scale);
            const float th = __fmul_rn(freq_scale, theta);
            const float c = __fmul_rn(cosf(th), mscale), sn = __fmul_rn(sinf(th), mscale);
            if (u == tok) {
                const float q0 = q[(size_t)u * tok_stride + h * hd + i0], q1 = q[(size_t)u * tok_stride + h * hd + i1];
                q16[i0] = __float2half_rn(__fsub_rn(__fmul_rn(q0, c), __fmul_rn(q1, sn)));
                q16[i1] = __float2half_rn(__fadd_rn(__fmul_rn(q0, sn), __fmul_rn(q1, c)));
            }
            const float k0 = k[(size_t)u * tok_stride + kvh * hd + i0], k1 = k[(size_t)u * tok_stride + kvh * hd + i1];
            const __half r0 = __float2half_rn(__fsub_rn(__fmul_rn(k0, c), __fmul_rn(k1, sn)));
            const __half r1 = __float2half_rn(__fadd_rn(__fmul_rn(k0, sn), __fmul_rn(k1, c)));
            k16[u * hd + i0] = r0; k16[u * hd + i1] = r1;
            if (owner && u == tok) { k_cache[(size_t)cell * gqa + kvh * hd + i0] = r0; k_cache[(size_t)cell * gqa + kvh * hd + i1] = r1; }
        }
    }
    if (tid < hd) {
        for (int u = 0; u < T; ++u) {
            const __half r = __float2half_rn(v[(size_t)u * tok_stride + kvh * hd + tid]);
            v16[u * hd + tid] = r;
            if (owner && u == tok) v_cache[(size_t)(kvh * hd + tid) * n_ctx + cell] = r;
        }
    }
    __syncthreads();

    // ---- scores: hd / 8 lanes per cell, 16 bytes of the cell's row each; four cells' rows in flight per lane -----------------
    const int lpc = hd / 8, cpw = PI_WAVE / lpc;                          // lanes per cell, cells per wave and pass
    const int sub = lane / lpc, l = lane % lpc;
    const pi_u32x4 qv = *reinterpret_cast<const pi_u32x4 *>(q16 + l * 8);
    const float scale = kq_scale[0];
    constexpr int SU = 4;
    const int cstep = kWavesPerBlock * cpw;
    for (int c0 = wave * cpw + sub; c0 < n_kv; c0 += SU * cstep) {
        pi_u32x4 kr[SU];
        float m[SU];
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            const int c = c0 + u * cstep;
            const int cc = c < n_kv ? c : n_kv - 1;                          // (clamped requests keep the loads unconditional)
            m[u] = kq_mask[cc];
            kr[u] = pi_ld16(k_cache + (size_t)cc * gqa + kvh * hd + l * 8);
        }
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            const int c = c0 + u * cstep;
            if (c >= cell0 && c < cell0 + T) kr[u] = *reinterpret_cast<const pi_u32x4 *>(k16 + (c - cell0) * hd + l * 8);
            float d = pi_dot8h(kr[u], qv, 0.0f);
            for (int o = 1; o < lpc; o <<= 1) d += __shfl_xor(d, o, PI_WAVE);
            if (c < n_kv && l == 0) sc[c] = m[u] == -INFINITY ? -INFINITY : __fadd_rn(__fmul_rn(d, scale), m[u]);
        }
    }
    __syncthreads();
    // ---- soft-max over the cells -------------------------------------------------------------------------------------------
    float mx = -INFINITY;
    for (int c = tid; c < n_kv; c += kBlock) mx = fmaxf(mx, sc[c]);
    mx = pi_wave_max(mx);
    if (lane == 0) redf[wave] = mx;
    __syncthreads();
    mx = redf[0];
    for (int w = 1; w < kWavesPerBlock; ++w) mx = fmaxf(mx, redf[w]);
    double sum = 0.0;
    for (int c = tid; c < n_kv; c += kBlock) {
        const float e = sc[c] == -INFINITY ? 0.0f : pi_round_f16(expf(pi_round_f16(__fsub_rn(sc[c], mx))));
        sc[c] = e; sum += (double)e;
    }
    sum = pi_wave_sum_f64(sum);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    double tot = 0.0;
    for (int w = 0; w < kWavesPerBlock; ++w) tot += red[w];
    const float inv = (float)(1.0 / tot);
    for (int c = tid; c < n_kv8; c += kBlock) sc[c] = c < n_kv ? __fmul_rn(sc[c], inv) : 0.0f;
    __syncthreads();
    // ---- out[dim] = sum over cells of fp16(p[cell]) * V[dim][cell].  Thread t owns column t % hd and every (kBlock / hd)-th group of
    // eight cells of it, four groups in flight; the column's partial sums meet in LDS (the scores' first floats are free by then
    // only after everyone has read its probabilities, hence the barrier in between) ------------------------------------------------
    {
        const int dim = tid % hd, part = tid / hd, nparts = kBlock / hd;      // hd <= kBlock and divides it (the launcher's test)
        const __half * vr = v_cache + (size_t)(kvh * hd + dim) * n_ctx;
        float acc = 0.0f;
        constexpr int VU = 4;
        for (int g0 = part; g0 * 8 < n_kv; g0 += VU * nparts) {
            pi_u32x4 vv[VU];
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                const int c0 = (g0 + u * nparts) * 8;
                vv[u] = pi_ld16(vr + (c0 < n_kv ? c0 : 0));
            }
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                const int c0 = (g0 + u * nparts) * 8;
                if (c0 < n_kv) {
                    for (int w = c0 > cell0 ? c0 - cell0 : 0; w < T && cell0 + w < c0 + 8; ++w)      // the step's own cells come from LDS
                        reinterpret_cast<__half *>(&vv[u])[cell0 + w - c0] = v16[w * hd + dim];
                    const float4 p0 = *reinterpret_cast<const float4 *>(sc + c0), p1 = *reinterpret_cast<const float4 *>(sc + c0 + 4);
                    __half2 ph[4] = {__floats2half2_rn(p0.x, p0.y), __floats2half2_rn(p0.z, p0.w), __floats2half2_rn(p1.x, p1.y), __floats2half2_rn(p1.z, p1.w)};
                    // a cell without probability contributes nothing, whatever its (possibly never written) V entry holds
                    const uint32_t * pw = reinterpret_cast<const uint32_t *>(ph);
                    uint32_t * vw = reinterpret_cast<uint32_t *>(&vv[u]);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if ((pw[j] & 0x0000ffffu) == 0u) vw[j] &= 0xffff0000u;
                        if ((pw[j] & 0xffff0000u) == 0u) vw[j] &= 0x0000ffffu;
                    }
                    acc = pi_dot8h(vv[u], *reinterpret_cast<const pi_u32x4 *>(ph), acc);
                }
            }
        }
        float * pacc = reinterpret_cast<float *>(v16 + (size_t)T * hd);       // [kBlock] floats behind the fp16 rows
        pacc[tid] = acc;
        __syncthreads();
        if (tid < hd) {
            float t = pacc[tid];
            for (int w = 1; w < nparts; ++w) t += pacc[tid + w * hd];
            out[h * hd + tid] = t;
        }
    }
}

}  // namespace

extern "C" {

int pi_k_rope_kv_store(const float * qkv, int n_head, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale,
                       const int32_t * pos, int n_ctx, float * q_rot, void * k_cache, void * v_cache, pi_stream_t stream) {
    if (!qkv || !pos || !q_rot || !k_cache || !v_cache) return pi::fail(PI_E_ARG, "pi_k_rope_kv_store: null pointer");
    if (n_head <= 0 || n_head_kv <= 0 || n_head % n_head_kv || hd <= 0 || hd % 2 || hd / 2 > 1024 || (mode != 0 && mode != 2))
        return pi::fail(PI_E_ARG, "pi_k_rope_kv_store: bad head geometry or mode");
    hipLaunchKernelGGL(rope_kv_store_kernel, dim3(n_head + 2 * n_head_kv), dim3(hd / 2), 0, (hipStream_t)stream,
                       qkv, n_head, n_head_kv, hd, mode, theta_scale, freq_scale, pos, n_ctx, q_rot, (__half *)k_cache, (__half *)v_cache, 0, 0);
    return pi::check_launch("pi_k_rope_kv_store");
}

int pi_k_attn_decode(const float * q_rot, const void * k_cache, const void * v_cache, int n_head, int n_head_kv,
                     int hd, int n_ctx, const int32_t * pos, float * out, pi_stream_t stream) {
    if (!q_rot || !k_cache || !v_cache || !pos || !out) return pi::fail(PI_E_ARG, "pi_k_attn_decode: null pointer");
    if (hd % 8 || kBlock % (hd / 8) || PI_WAVE % (hd / 8) || n_head % n_head_kv) return pi::fail(PI_E_ARG, "pi_k_attn_decode: head size must be 8 * (a divisor of 64)");
    const size_t sh = sizeof(float) * ((size_t)n_ctx + (size_t)(kBlock / (hd / 8)) * hd);
    if (sh > 60 * 1024) return pi::fail(PI_E_UNSUPPORTED, "pi_k_attn_decode: context too long for the single-pass kernel");
    hipLaunchKernelGGL(attn_decode_kernel, dim3(n_head), dim3(kBlock), sh, (hipStream_t)stream,
                       q_rot, (const __half *)k_cache, (const __half *)v_cache, n_head, n_head_kv, hd, n_ctx, pos, out, 0, 0, nullptr);
    return pi::check_launch("pi_k_attn_decode");
}

int pi_k_rope_table(void * table, int n_ctx, int hd, int mode, float theta_scale, float freq_scale, pi_stream_t stream) {
    if (!table || n_ctx <= 0 || hd <= 0 || hd % 2 || hd / 2 > 1024) return pi::fail(PI_E_ARG, "pi_k_rope_table: bad arguments");
    // A set-up call: the table is computed on the host with the C library's cosf / sinf -- the functions the CPU path itself calls
    // (ggml.c:11163-11325: theta = position, then *= theta_scale per pair) -- so rotated q and k start from bit-identical factors;
    // the device's own cosf / sinf may differ from them in the last place.
    const int half = hd / 2;
    std::vector<float> host((size_t)n_ctx * hd);
    for (int p = 0; p < n_ctx; ++p) {
        float theta = (mode & 2) ? (float)p * freq_scale : (float)p;             // rope_angle, one product per pair
        for (int i = 0; i < half; ++i) {
            const float th = freq_scale * theta;
            host[((size_t)p * half + i) * 2]     = cosf(th);
            host[((size_t)p * half + i) * 2 + 1] = sinf(th);
            theta *= theta_scale;
        }
    }
    PI_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    PI_HIP_TRY(hipMemcpy(table, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice));
    return PI_OK;
}

// LDS of attn_fused_kernel: the scores of every cell, one partial output row per group of hd/8 lanes, and q, k, v of the new cell
static bool attn_fused_geometry_ok(int hd) {
    return hd > 0 && hd % 8 == 0 && (kAttnBlock / 2) % (hd / 8) == 0 && PI_WAVE % (hd / 8) == 0 && hd / 2 + hd <= kAttnBlock / 2;
}
static size_t attn_fused_lds_bytes(int hd, int n_ctx, int block = kAttnBlock) {
    return sizeof(float) * ((size_t)n_ctx + (size_t)(block / (hd / 8)) * hd + 3 * (size_t)hd);
}
constexpr size_t kAttnLdsLimit = 60 * 1024;

int pi_k_attn_fused_supported(int hd, int n_ctx) {
    return attn_fused_geometry_ok(hd) && n_ctx > 0 && attn_fused_lds_bytes(hd, n_ctx) <= kAttnLdsLimit;
}

int pi_k_attn_decode_supported(int hd, int n_ctx) {
    return hd > 0 && hd % 8 == 0 && kBlock % (hd / 8) == 0 && PI_WAVE % (hd / 8) == 0 && n_ctx > 0 &&
           sizeof(float) * ((size_t)n_ctx + (size_t)(kBlock / (hd / 8)) * hd) <= kAttnLdsLimit;
}

int pi_k_attn_fused(const float * qkv, const void * rope_table, void * k_cache, void * v_cache, int n_head, int n_head_kv, int hd, int mode,
                    int n_ctx, const int32_t * pos, float * out, pi_stream_t stream) {
    if (!qkv || !rope_table || !k_cache || !v_cache || !pos || !out) return pi::fail(PI_E_ARG, "pi_k_attn_fused: null pointer");
    if (n_head <= 0 || n_head_kv <= 0 || n_head % n_head_kv || !attn_fused_geometry_ok(hd) || (mode != 0 && mode != 2))
        return pi::fail(PI_E_ARG, "pi_k_attn_fused: head size must be 8 * (a divisor of 64), at most 128; mode 0 or 2");
    const size_t sh = attn_fused_lds_bytes(hd, n_ctx);
    if (sh > kAttnLdsLimit) return pi::fail(PI_E_UNSUPPORTED, "pi_k_attn_fused: context too long for the single-pass kernel");
    hipLaunchKernelGGL(attn_fused_kernel<kAttnBlock>, dim3(n_head), dim3(kAttnBlock), sh, (hipStream_t)stream, qkv, (const float2 *)rope_table,
                       (__half *)k_cache, (__half *)v_cache, n_head, n_head_kv, hd, mode, n_ctx, pos, out, 0, (size_t)0, 0, nullptr, 0, nullptr, nullptr, nullptr);
    return pi::check_launch("pi_k_attn_fused");
}

// ---- attention with the cells of a head split over n_parts workgroups --------------------------------------------
static size_t attn_part_lds_bytes(int hd, int s_cap) {
    return sizeof(float) * ((size_t)s_cap + (size_t)(kAttnPartBlock / (hd / 8)) * hd + 3 * (size_t)hd);
}
static bool attn_part_geometry_ok(int hd) {
    return hd > 0 && hd % 8 == 0 && kAttnPartBlock % (hd / 8) == 0 && PI_WAVE % (hd / 8) == 0 && hd / 2 + hd <= kAttnPartBlock && hd <= 1024;
}
int pi_k_attn_split_supported(int hd, int n_ctx, int n_parts) {
    return attn_part_geometry_ok(hd) && n_ctx > 0 && n_parts >= 1 && n_parts <= 64 && attn_part_lds_bytes(hd, (n_ctx + n_parts - 1) / n_parts + 1) <= kAttnLdsLimit;
}
size_t pi_k_attn_split_scratch_floats(int n_seq, int n_head, int hd, int n_parts) { return (size_t)n_seq * n_head * n_parts * ((size_t)hd + 2); }

int pi_k_attn_split(const float * qkv, int qkv_stride, const void * rope_table, void * k_cache, void * v_cache, size_t cache_seq_stride,
                    int n_seq, int n_head, int n_head_kv, int hd, int mode, int n_ctx, int n_parts, const int32_t * pos, float * scratch,
                    float * out, int out_stride, void * out_f16, pi_stream_t stream) {
    if (!qkv || !rope_table || !k_cache || !v_cache || !pos || !out || !scratch || n_seq <= 0) return pi::fail(PI_E_ARG, "pi_k_attn_split: bad arguments");
    if (n_head <= 0 || n_head_kv <= 0 || n_head % n_head_kv || (mode != 0 && mode != 2) || !pi_k_attn_split_supported(hd, n_ctx, n_parts))
        return pi::fail(PI_E_UNSUPPORTED, "pi_k_attn_split: head size, context per part or part count outside the kernel (pi_k_attn_split_supported)");
    const int s_cap = (n_ctx + n_parts - 1) / n_parts + 1;
    float * acc = scratch;
    float * ml = scratch + (size_t)n_seq * n_head * n_parts * hd;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(attn_part_kernel<false>, dim3(n_head, n_parts, n_seq), dim3(kAttnPartBlock), attn_part_lds_bytes(hd, s_cap), st, qkv, (const float2 *)rope_table,
                       (__half *)k_cache, (__half *)v_cache, n_head, n_head_kv, hd, mode, n_ctx, s_cap, pos, acc, ml, qkv_stride, cache_seq_stride);
    hipLaunchKernelGGL(attn_merge_kernel, dim3(n_head, n_seq), dim3(hd), 0, st, acc, ml, n_parts, hd, out, out_stride, (__half *)out_f16);
    return pi::check_launch("pi_k_attn_split");
}

int pi_k_attn_split_cached(const float * q_rot, const void * k_cache, const void * v_cache, int n_tok, int n_head, int n_head_kv, int hd,
                           int n_ctx, int n_parts, const int32_t * pos, float * scratch, float * out, pi_stream_t stream) {
    if (!q_rot || !k_cache || !v_cache || !pos || !out || !scratch || n_tok <= 0 || n_tok > 65535) return pi::fail(PI_E_ARG, "pi_k_attn_split_cached: bad arguments");
    if (n_head <= 0 || n_head_kv <= 0 || n_head % n_head_kv || !pi_k_attn_split_supported(hd, n_ctx, n_parts))
        return pi::fail(PI_E_UNSUPPORTED, "pi_k_attn_split_cached: head size, context per part or part count outside the kernel (pi_k_attn_split_supported)");
    const int s_cap = (n_ctx + n_parts - 1) / n_parts + 1;
    float * acc = scratch;
    float * ml = scratch + (size_t)n_tok * n_head * n_parts * hd;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(attn_part_kernel<true>, dim3(n_head, n_parts, n_tok), dim3(kAttnPartBlock), attn_part_lds_bytes(hd, s_cap), st, q_rot, (const float2 *)nullptr,
                       (__half *)const_cast<void *>(k_cache), (__half *)const_cast<void *>(v_cache), n_head, n_head_kv, hd, 0, n_ctx, s_cap, pos, acc, ml, n_head * hd, (size_t)0);
    hipLaunchKernelGGL(attn_merge_kernel, dim3(n_head, n_tok), dim3(hd), 0, st, acc, ml, n_parts, hd, out, n_head * hd, (__half *)nullptr);
    return pi::check_launch("pi_k_attn_split_cached");
}

static int attn_fused_batch(const float * qkv, int qkv_stride, const void * rope_table, void * k_cache, void * v_cache, size_t cache_seq_stride,
                            int n_seq, int n_head, int n_head_kv, int hd, int mode, int n_ctx, const int32_t * pos, float * out, int out_stride,
                            void * out_f16, pi_stream_t stream, int out16_ol, void * q8_q = nullptr, float * q8_d = nullptr, int32_t * q8_s = nullptr) {
    if (q8_q && (hd % 32 || !q8_d || !q8_s)) return pi::fail(PI_E_ARG, "pi_k_attn_fused_batch_q8: head size % 32 == 0 and all three outputs required");
    if (!qkv || !rope_table || !k_cache || !v_cache || !pos || !out || n_seq <= 0 || n_seq > kBtMaxT) return pi::fail(PI_E_ARG, "pi_k_attn_fused_batch: bad arguments");
    if (n_head <= 0 || n_head_kv <= 0 || n_head % n_head_kv || !attn_fused_geometry_ok(hd) || (mode != 0 && mode != 2))
        return pi::fail(PI_E_ARG, "pi_k_attn_fused_batch: head size must be 8 * (a divisor of 64), at most 128; mode 0 or 2");
    const size_t sh = attn_fused_lds_bytes(hd, n_ctx);
    if (sh > kAttnLdsLimit) return pi::fail(PI_E_UNSUPPORTED, "pi_k_attn_fused_batch: context too long for the single-pass kernel");
    const int n_cu = pi::compute_units();
    if (n_cu > 0 && n_seq * n_head > 2 * n_cu)
        hipLaunchKernelGGL(attn_fused_kernel<kAttnBlock / 2>, dim3(n_head, n_seq), dim3(kAttnBlock / 2), attn_fused_lds_bytes(hd, n_ctx, kAttnBlock / 2), (hipStream_t)stream, qkv, (const float2 *)rope_table,
                           (__half *)k_cache, (__half *)v_cache, n_head, n_head_kv, hd, mode, n_ctx, pos, out, qkv_stride, cache_seq_stride, out_stride, (__half *)out_f16, out16_ol, (int8_t *)q8_q, q8_d, q8_s);
    else
        hipLaunchKernelGGL(attn_fused_kernel<kAttnBlock>, dim3(n_head, n_seq), dim3(kAttnBlock), sh, (hipStream_t)stream, qkv, (const float2 *)rope_table,
                           (__half *)k_cache, (__half *)v_cache, n_head, n_head_kv, hd, mode, n_ctx, pos, out, qkv_stride, cache_seq_stride, out_stride, (__half *)out_f16, out16_ol, (int8_t *)q8_q, q8_d, q8_s);
    return pi::check_launch("pi_k_attn_fused_batch");
}

int pi_k_attn_fused_batch(const float * qkv, int qkv_stride, const void * rope_table, void * k_cache, void * v_cache, size_t cache_seq_stride,
                          int n_seq, int n_head, int n_head_kv, int hd, int mode, int n_ctx, const int32_t * pos, float * out, int out_stride,
                          void * out_f16, pi_stream_t stream) {
    return attn_fused_batch(qkv, qkv_stride, rope_table, k_cache, v_cache, cache_seq_stride, n_seq, n_head, n_head_kv, hd, mode, n_ctx, pos, out, out_stride, out_f16, stream, 0);
}

int pi_k_attn_fused_batch_q8(const float * qkv, int qkv_stride, const void * rope_table, void * k_cache, void * v_cache, size_t cache_seq_stride,
                             int n_seq, int n_head, int n_head_kv, int hd, int mode, int n_ctx, const int32_t * pos, float * out, int out_stride,
                             void * q8_quants, float * q8_scales, int32_t * q8_sums, pi_stream_t stream) {
    if (!q8_quants) return pi::fail(PI_E_ARG, "pi_k_attn_fused_batch_q8: null pointer");
    return attn_fused_batch(qkv, qkv_stride, rope_table, k_cache, v_cache, cache_seq_stride, n_seq, n_head, n_head_kv, hd, mode, n_ctx, pos, out, out_stride, nullptr, stream, 0,
                            q8_quants, q8_scales, q8_sums);
}

int pi_k_attn_fused_batch_ol(const float * qkv, int qkv_stride, const void * rope_table, void * k_cache, void * v_cache, size_t cache_seq_stride,
                             int n_seq, int n_head, int n_head_kv, int hd, int mode, int n_ctx, const int32_t * pos, float * out, int out_stride,
                             void * out_ol, pi_stream_t stream) {
    return attn_fused_batch(qkv, qkv_stride, rope_table, k_cache, v_cache, cache_seq_stride, n_seq, n_head, n_head_kv, hd, mode, n_ctx, pos, out, out_stride, out_ol, stream, 1);
}

int pi_k_attn_chunk(const float * qkv, int qkv_stride, int T, int n_head, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale,
                    const int32_t * pos, int n_ctx, int n_kv_max, float * q_rot, void * k_cache, void * v_cache, float * out, int out_stride, void * out_f16,
                    pi_stream_t stream) {
    if (!qkv || !pos || !q_rot || !k_cache || !v_cache || !out || T <= 0 || T > kChunkMaxT) return pi::fail(PI_E_ARG, "pi_k_attn_chunk: bad arguments");
    if (n_kv_max <= 0 || n_kv_max > n_ctx) n_kv_max = n_ctx;                  // cells the furthest token of the chunk attends: what the scores in LDS are sized for
    if (n_head <= 0 || n_head_kv <= 0 || n_head % n_head_kv || hd <= 0 || hd % 8 || hd / 2 > 1024 || kBlock % (hd / 8) || PI_WAVE % (hd / 8) || (mode != 0 && mode != 2))
        return pi::fail(PI_E_ARG, "pi_k_attn_chunk: bad head geometry or mode");
    hipStream_t st = (hipStream_t)stream;
    // all K/V rows of the chunk are in the cache before any token of the chunk attends
    hipLaunchKernelGGL(rope_kv_store_kernel, dim3(n_head + 2 * n_head_kv, T), dim3(hd / 2), 0, st,
                       qkv, n_head, n_head_kv, hd, mode, theta_scale, freq_scale, pos, n_ctx, q_rot, (__half *)k_cache, (__half *)v_cache, qkv_stride, n_head * hd);
    // 16 tokens per workgroup on the matrix cores where the head size and the context fit (scores of 16 tokens in LDS)
    const int s_stride = ((n_kv_max + 31) & ~31) + 4;
    const size_t sh_mfma = sizeof(float) * 16 * (size_t)s_stride + (size_t)kWavesPerBlock * hd * kAcVtStride * 2;
    const char * own = getenv("PI_ATTN_CHUNK");
    if ((hd == 128 || hd == 64) && T > 1 && sh_mfma <= 156 * 1024 && !(own && !strcmp(own, "scalar"))) {
        static bool raised[2] = {false, false};
        if (!raised[hd == 64]) {
            if (hd == 128) PI_HIP_TRY(hipFuncSetAttribute((const void *)attn_chunk_mfma_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
            else           PI_HIP_TRY(hipFuncSetAttribute((const void *)attn_chunk_mfma_kernel<64>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
            raised[hd == 64] = true;
        }
        const dim3 grid(n_head, (T + 15) / 16);
        if (hd == 128) hipLaunchKernelGGL(attn_chunk_mfma_kernel<128>, grid, dim3(kBlock), sh_mfma, st, q_rot, (const __half *)k_cache, (const __half *)v_cache,
                                          n_head, n_head_kv, n_ctx, pos, T, out, n_head * hd, out_stride, (__half *)out_f16, s_stride);
        else           hipLaunchKernelGGL(attn_chunk_mfma_kernel<64>, grid, dim3(kBlock), sh_mfma, st, q_rot, (const __half *)k_cache, (const __half *)v_cache,
                                          n_head, n_head_kv, n_ctx, pos, T, out, n_head * hd, out_stride, (__half *)out_f16, s_stride);
        return pi::check_launch("pi_k_attn_chunk");
    }
    const size_t sh = sizeof(float) * ((size_t)n_ctx + (size_t)(kBlock / (hd / 8)) * hd);
    if (sh > 60 * 1024) return pi::fail(PI_E_UNSUPPORTED, "pi_k_attn_chunk: context too long for the single-pass kernel (pi_k_attn_chunk_supported)");
    hipLaunchKernelGGL(attn_decode_kernel, dim3(n_head, T), dim3(kBlock), sh, st,
                       q_rot, (const __half *)k_cache, (const __half *)v_cache, n_head, n_head_kv, hd, n_ctx, pos, out, n_head * hd, out_stride, (__half *)out_f16);
    return pi::check_launch("pi_k_attn_chunk");
}

int pi_k_attn_chunk_supported(int hd, int n_ctx, int n_kv_max) {
    if (hd <= 0 || hd % 8 || kBlock % (hd / 8) || PI_WAVE % (hd / 8) || n_ctx <= 0) return 0;
    if (n_kv_max <= 0 || n_kv_max > n_ctx) n_kv_max = n_ctx;
    const int s_stride = ((n_kv_max + 31) & ~31) + 4;
    const size_t sh_mfma = sizeof(float) * 16 * (size_t)s_stride + (size_t)kWavesPerBlock * hd * kAcVtStride * 2;
    if ((hd == 128 || hd == 64) && sh_mfma <= 156 * 1024) return 1;
    return sizeof(float) * ((size_t)n_ctx + (size_t)(kBlock / (hd / 8)) * hd) <= 60 * 1024;
}

// pi_k_attn_chunk for contexts beyond its kernels: RoPE + KV store of the chunk, then every token's cells split over n_parts workgroups
int pi_k_attn_chunk_long(const float * qkv, int qkv_stride, int T, int n_head, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale,
                         const int32_t * pos, int n_ctx, int n_parts, float * scratch, float * q_rot, void * k_cache, void * v_cache,
                         float * out, void * out_f16, pi_stream_t stream) {
    if (!qkv || !pos || !q_rot || !k_cache || !v_cache || !out || !scratch || T <= 0 || T > kChunkMaxT) return pi::fail(PI_E_ARG, "pi_k_attn_chunk_long: bad arguments");
    if (n_head <= 0 || n_head_kv <= 0 || n_head % n_head_kv || (mode != 0 && mode != 2) || hd % 2 || hd / 2 > 1024 || !pi_k_attn_split_supported(hd, n_ctx, n_parts))
        return pi::fail(PI_E_UNSUPPORTED, "pi_k_attn_chunk_long: head size, context per part or part count outside the kernel (pi_k_attn_split_supported)");
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(rope_kv_store_kernel, dim3(n_head + 2 * n_head_kv, T), dim3(hd / 2), 0, st,
                       qkv, n_head, n_head_kv, hd, mode, theta_scale, freq_scale, pos, n_ctx, q_rot, (__half *)k_cache, (__half *)v_cache, qkv_stride, n_head * hd);
    const int s_cap = (n_ctx + n_parts - 1) / n_parts + 1;
    float * acc = scratch;
    float * ml = scratch + (size_t)T * n_head * n_parts * hd;
    hipLaunchKernelGGL(attn_part_kernel<true>, dim3(n_head, n_parts, T), dim3(kAttnPartBlock), attn_part_lds_bytes(hd, s_cap), st, q_rot, (const float2 *)nullptr,
                       (__half *)k_cache, (__half *)v_cache, n_head, n_head_kv, hd, 0, n_ctx, s_cap, pos, acc, ml, n_head * hd, (size_t)0);
    hipLaunchKernelGGL(attn_merge_kernel, dim3(n_head, T), dim3(hd), 0, st, acc, ml, n_parts, hd, out, n_head * hd, (__half *)out_f16);
    return pi::check_launch("pi_k_attn_chunk_long");
}

static size_t attn_ggml_lds(int hd, int n_kv, int T) {
    return sizeof(float) * (size_t)((n_kv + 7) & ~7) + 2 * (size_t)hd * (1 + 2 * (size_t)T) + sizeof(float) * kBlock;
}
int pi_k_attn_ggml_supported(int hd, int n_ctx, int n_kv) {
    return hd > 0 && hd % 8 == 0 && hd <= kBlock && kBlock % hd == 0 && PI_WAVE % (hd / 8) == 0 && n_kv > 0 && n_ctx % 8 == 0 && n_kv <= n_ctx &&
           attn_ggml_lds(hd, n_kv, kBtMaxT) <= 60 * 1024;
}

int pi_k_attn_ggml(const float * q, const float * k, const float * v, const int32_t * pos, int mode, float theta_scale, float freq_scale, float mscale,
                   void * k_cache, void * v_cache, int n_head, int n_head_kv, int hd, int n_ctx, int n_kv, int cell,
                   const float * kq_scale, const float * kq_mask, float * out, pi_stream_t stream) {
    if (!q || !k || !v || !pos || !k_cache || !v_cache || !kq_scale || !kq_mask || !out) return pi::fail(PI_E_ARG, "pi_k_attn_ggml: null pointer");
    if (n_head <= 0 || n_head_kv <= 0 || n_head % n_head_kv || (mode != 0 && mode != 2) || cell < 0 || cell >= n_kv || !pi_k_attn_ggml_supported(hd, n_ctx, n_kv))
        return pi::fail(PI_E_UNSUPPORTED, "pi_k_attn_ggml: head geometry, cell or context outside the kernel (pi_k_attn_ggml_supported)");
    if ((((uintptr_t)k_cache | (uintptr_t)v_cache) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_attn_ggml: the caches must be 16-byte aligned");
    hipLaunchKernelGGL(attn_ggml_kernel, dim3(n_head, 1), dim3(kBlock), attn_ggml_lds(hd, n_kv, 1), (hipStream_t)stream, q, k, v, 0, pos, mode, theta_scale, freq_scale, mscale,
                       (__half *)k_cache, (__half *)v_cache, n_head, n_head_kv, hd, n_ctx, n_kv, 1, cell, kq_scale, kq_mask, 0, out, 0);
    return pi::check_launch("pi_k_attn_ggml");
}

int pi_k_attn_ggml_step(const float * qkv, int qkv_stride, const int32_t * pos, int mode, float theta_scale, float freq_scale, float mscale,
                        void * k_cache, void * v_cache, int n_head, int n_head_kv, int hd, int n_ctx, int n_kv, int T, int cell0,
                        const float * kq_scale, const float * kq_mask, int mask_stride, float * out, int out_stride, pi_stream_t stream) {
    if (!qkv || !pos || !k_cache || !v_cache || !kq_scale || !kq_mask || !out) return pi::fail(PI_E_ARG, "pi_k_attn_ggml_step: null pointer");
    if (n_head <= 0 || n_head_kv <= 0 || n_head % n_head_kv || (mode != 0 && mode != 2) || T < 1 || T > kBtMaxT || cell0 < 0 || cell0 + T > n_kv ||
        qkv_stride < (n_head + 2 * n_head_kv) * hd || mask_stride < n_kv || out_stride < n_head * hd || !pi_k_attn_ggml_supported(hd, n_ctx, n_kv))
        return pi::fail(PI_E_UNSUPPORTED, "pi_k_attn_ggml_step: head geometry, cells, strides or context outside the kernel (pi_k_attn_ggml_supported)");
    if ((((uintptr_t)k_cache | (uintptr_t)v_cache) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_attn_ggml_step: the caches must be 16-byte aligned");
    hipLaunchKernelGGL(attn_ggml_kernel, dim3(n_head, T), dim3(kBlock), attn_ggml_lds(hd, n_kv, T), (hipStream_t)stream, qkv, qkv + (size_t)n_head * hd,
                       qkv + (size_t)(n_head + n_head_kv) * hd, qkv_stride, pos, mode, theta_scale, freq_scale, mscale, (__half *)k_cache, (__half *)v_cache,
                       n_head, n_head_kv, hd, n_ctx, n_kv, T, cell0, kq_scale, kq_mask, mask_stride, out, out_stride);
    return pi::check_launch("pi_k_attn_ggml_step");
}

int pi_k_k_shift(void * k_cache, int rows, int n_ctx, int hd, int mode, float theta_scale, float freq_scale, const int32_t * delta, int n_cells, pi_stream_t stream) {
    if (!k_cache || !delta || rows <= 0 || n_ctx <= 0 || hd <= 0 || hd % 2 || hd / 2 > 1024 || n_cells < 0 || n_cells > n_ctx || (mode != 0 && mode != 2))
        return pi::fail(PI_E_ARG, "pi_k_k_shift: bad arguments");
    if (n_cells == 0) return PI_OK;
    hipLaunchKernelGGL(k_shift_kernel, dim3(n_cells, rows), dim3(hd / 2), 0, (hipStream_t)stream, (__half *)k_cache, n_ctx, hd, mode, theta_scale, freq_scale, delta);
    return pi::check_launch("pi_k_k_shift");
}

int pi_k_k_shift_cells(void * k_cache, int n_layer, int n_cells, int n_head_kv, int hd, int mode, float theta_scale, float freq_scale, const int32_t * delta,
                       pi_stream_t stream) {
    if (!k_cache || !delta || n_layer <= 0 || n_cells <= 0 || n_head_kv <= 0 || hd <= 0 || hd % 2 || hd / 2 > 1024 || (mode != 0 && mode != 2))
        return pi::fail(PI_E_ARG, "pi_k_k_shift_cells: bad arguments");
    hipLaunchKernelGGL(k_shift_cells_kernel, dim3(n_cells, n_layer * n_head_kv), dim3(hd / 2), 0, (hipStream_t)stream, (__half *)k_cache, n_cells, n_head_kv, hd, mode,
                       theta_scale, freq_scale, delta);
    return pi::check_launch("pi_k_k_shift_cells");
}

int pi_k_kv_compact(void * cache, void * stage, int rows, int n_ctx, int hd, const int32_t * map, int n_new, pi_stream_t stream) {
    if (!cache || !stage || !map || rows <= 0 || n_ctx <= 0 || hd <= 0 || hd % 8 || hd / 8 > 1024 || n_new < 0 || n_new > n_ctx)
        return pi::fail(PI_E_ARG, "pi_k_kv_compact: bad arguments");
    if (n_new == 0) return PI_OK;
    hipLaunchKernelGGL(kv_gather_kernel, dim3(n_new, rows), dim3(hd / 8), 0, (hipStream_t)stream, (const __half *)cache, (__half *)stage, map, n_new, n_ctx, hd);
    hipLaunchKernelGGL(kv_place_kernel, dim3(n_new, rows), dim3(hd / 8), 0, (hipStream_t)stream, (__half *)cache, (const __half *)stage, n_new, n_ctx, hd);
    return pi::check_launch("pi_k_kv_compact");
}

}  // extern "C"

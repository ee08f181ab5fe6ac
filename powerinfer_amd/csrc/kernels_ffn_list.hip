// The sparse FFN operator by operator (GGML_OP_MUL_MAT_SPARSE, GGML_OP_AXPY and the predictor in front of them): predictor fc2 with
// threshold and compaction, sparse up/gate over an index list or the mask words, sparse down projection from a compact or a dense h.
// F16 and Q4_0 rows; the route of hybrid buckets, of the ggml boundary and of shapes the fused kernels do not cover.
#include "kernels_common.hpp"

namespace {

// ---------------------------------------------------------------------------------------------------
// Predictor fc2 + activity test + compaction.
// Block = 32 consecutive neurons (8 per wave) -> one 32-bit mask word per block by wave ballot.  The
// block that finishes last (ticket counter) turns the mask words into the ascending active-row list
// with popcount prefix sums.
// ---------------------------------------------------------------------------------------------------
// returns true in every thread of the block that took the last ticket; resets the counter for the next launch
__device__ bool last_block_done(unsigned int * counter, unsigned int n_blocks, int * sflag) {
    __syncthreads();
    if (threadIdx.x == 0) {
        __threadfence();          // cumulative: publishes the whole block's stores, ordered before the ticket
        const unsigned int t = atomicAdd(counter, 1u);
        *sflag = (t == n_blocks - 1);
        if (t == n_blocks - 1) { *counter = 0; __threadfence(); }
    }
    __syncthreads();
    return *sflag != 0;
}

// Block = 32 consecutive neurons (8 per wave); all weight loads of the block are issued before the hidden
// vector is staged.  Emits the logits and one 32-bit activity word per block (wave ballot).  NCH = number of
// 512-column chunks (r <= 512 * NCH); NCH == 0 is the guard-everything variant for other ranks.
template <int NCH>
__global__ __launch_bounds__(kBlock) void pred_fc2_kernel(const __half * __restrict__ W, const float * __restrict__ hidden, int ff, int r,
                                                          float thr, float * __restrict__ logits, uint32_t * __restrict__ words,
                                                          float * zero_fill) {
    extern __shared__ __align__(16) unsigned char smem[];
    float  * xraw = reinterpret_cast<float *>(smem);
    __half * xs   = reinterpret_cast<__half *>(smem + (size_t)r * 4);
    __shared__ float lg[32];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row0 = blockIdx.x * 32 + wave * 8;
    if (zero_fill && threadIdx.x < 32 && (int)(blockIdx.x * 32 + threadIdx.x) < ff) zero_fill[blockIdx.x * 32 + threadIdx.x] = 0.0f;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;

    if constexpr (NCH > 0) {
        for (int base = wave * 256; base < r; base += kWavesPerBlock * 256)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(hidden + base + lane * 4),
                                             (__attribute__((address_space(3))) void *)(xraw + base), 16, 0, 0);
        pi_u32x4 buf[8][NCH];
        const pi_u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int u = 0; u < NCH; ++u)
#pragma unroll
            for (int i = 0; i < 8; ++i)
                buf[i][u] = (row0 + i < ff) ? pi_ld_stream(W + (size_t)(row0 + i) * r + (u * PI_WAVE + lane) * 8) : zero;
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 * NCH) : "memory");
        __syncthreads();
        for (int i = threadIdx.x; i < r; i += kBlock) xs[i] = __float2half_rn(xraw[i]);
        __syncthreads();
#pragma unroll
        for (int u = 0; u < NCH; ++u) {
            float xf[8];
            pi_unpack8(pi_ld16(xs + (u * PI_WAVE + lane) * 8), xf);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = pi_dot8(buf[i][u], xf, acc[i]);
        }
    } else {
        for (int i = threadIdx.x; i < r; i += kBlock) xs[i] = __float2half_rn(hidden[i]);
        __syncthreads();
        for (int c = lane * 8; c < r; c += PI_WAVE * 8) {
            float xf[8];
            pi_unpack8(pi_ld16(xs + c), xf);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (row0 + i < ff) acc[i] = pi_dot8(pi_ld_stream(W + (size_t)(row0 + i) * r + c), xf, acc[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) { const float sum = pi_wave_sum(acc[i]); if (lane == 0) lg[wave * 8 + i] = sum; }
    __syncthreads();
    if (wave == 0) {
        const int row = blockIdx.x * 32 + lane;
        bool act = false;
        if (lane < 32 && row < ff) { const float v = lg[lane]; logits[row] = v; act = !(v < thr); }
        const unsigned long long m = __ballot(act);
        if (lane == 0) words[blockIdx.x] = (uint32_t)m;
    }
}


// ---------------------------------------------------------------------------------------------------
// Predictor fc2 + activity test + sparse up/gate in one kernel (F16, cols == 512*NCH, r == 512*RCH).
// A workgroup owns 32 consecutive neurons.  Phase A: its four waves compute the 32 predictor logits (8 rows
// each, all loads issued at once); while those are in flight every wave loads the FFN input, normalises it
// and keeps it as packed fp16 in registers.  Phase B: the 32 logits meet in LDS, every wave derives the same
// 32-bit activity word, and wave w takes the w-th, (w+4)-th ... set bit, two neurons per round trip (gate row
// + up row each).  The workgroup writes h for all of its 32 neurons (0 where inactive), the activity word and
// the logits; nothing crosses workgroups, so neither a compaction pass nor a second launch sits between
// predictor and FFN.  Neurons fire independently of their index, so a workgroup sees about ff*rate/32*...
// a handful of active rows and finishes phase B in one round trip almost always.
// ---------------------------------------------------------------------------------------------------
template <int NCH, int RCH>
__global__ __launch_bounds__(kBlock) void pred_upgate_f16_kernel(const __half * __restrict__ W2, const float * __restrict__ hidden,
                                                                 const __half * __restrict__ Wup, const __half * __restrict__ Wgate,
                                                                 const float * __restrict__ x, NormArgs na, float thr,
                                                                 float * __restrict__ logits, uint32_t * __restrict__ words, float * __restrict__ h_dense) {
    constexpr int cols = NCH * 512, r = RCH * 512;
    __shared__ float lg[32];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n0 = blockIdx.x * 32;

    // ---- phase A loads: 8 predictor rows per wave, the hidden vector, the FFN input ---------------------
    pi_u32x4 a[8][RCH];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < RCH; ++j) a[i][j] = pi_ld_stream(W2 + (size_t)(n0 + wave * 8 + i) * r + (j * PI_WAVE + lane) * 8);
    float4 hv[RCH][2], xv[NCH][2];
#pragma unroll
    for (int j = 0; j < RCH; ++j) {
        hv[j][0] = *reinterpret_cast<const float4 *>(hidden + j * 512 + lane * 8);
        hv[j][1] = *reinterpret_cast<const float4 *>(hidden + j * 512 + lane * 8 + 4);
    }
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        xv[j][0] = *reinterpret_cast<const float4 *>(x + j * 512 + lane * 8);
        xv[j][1] = *reinterpret_cast<const float4 *>(x + j * 512 + lane * 8 + 4);
    }
    // ---- logits ------------------------------------------------------------------------------------------
    {
        float hf[RCH][8];
#pragma unroll
        for (int j = 0; j < RCH; ++j) {       // the CPU path rounds the hidden vector to fp16 before the dot (ggml.c:9703-9716)
            hf[j][0] = pi_round_f16(hv[j][0].x); hf[j][1] = pi_round_f16(hv[j][0].y); hf[j][2] = pi_round_f16(hv[j][0].z); hf[j][3] = pi_round_f16(hv[j][0].w);
            hf[j][4] = pi_round_f16(hv[j][1].x); hf[j][5] = pi_round_f16(hv[j][1].y); hf[j][6] = pi_round_f16(hv[j][1].z); hf[j][7] = pi_round_f16(hv[j][1].w);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < RCH; ++j) acc = pi_dot8(a[i][j], hf[j], acc);
            acc = pi_wave_sum(acc);
            if (lane == 0) lg[wave * 8 + i] = acc;
        }
    }
    // ---- FFN input: norm, round to fp16, keep in registers --------------------------------------------
    pi_u32x4 xr[NCH];
    {
        const bool has_w = na.kind != 0 && na.w != nullptr;
        float4 wv[NCH][2];
        if (has_w) {
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                wv[j][0] = *reinterpret_cast<const float4 *>(na.w + j * 512 + lane * 8);
                wv[j][1] = *reinterpret_cast<const float4 *>(na.w + j * 512 + lane * 8 + 4);
            }
        }
        float mean = 0.0f, scale = 1.0f;
        if (na.kind == 1) {
            double s = 0.0;
#pragma unroll
            for (int j = 0; j < NCH; ++j)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float4 v = xv[j][h];
                    s += (double)__fmul_rn(v.x, v.x); s += (double)__fmul_rn(v.y, v.y); s += (double)__fmul_rn(v.z, v.z); s += (double)__fmul_rn(v.w, v.w);
                }
            s = pi_wave_sum_f64(s);
            scale = pi_inv_sqrt((float)(s / cols) + na.eps);
        } else if (na.kind == 2) {
            double s = 0.0;
#pragma unroll
            for (int j = 0; j < NCH; ++j)
#pragma unroll
                for (int h = 0; h < 2; ++h) { const float4 v = xv[j][h]; s += (double)v.x; s += (double)v.y; s += (double)v.z; s += (double)v.w; }
            s = pi_wave_sum_f64(s);
            mean = (float)(s / cols);
            double s2 = 0.0;
#pragma unroll
            for (int j = 0; j < NCH; ++j)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float4 v = xv[j][h];
                    const float p = __fsub_rn(v.x, mean), q = __fsub_rn(v.y, mean), c = __fsub_rn(v.z, mean), e = __fsub_rn(v.w, mean);
                    s2 += (double)__fmul_rn(p, p); s2 += (double)__fmul_rn(q, q); s2 += (double)__fmul_rn(c, c); s2 += (double)__fmul_rn(e, e);
                }
            s2 = pi_wave_sum_f64(s2);
            scale = pi_inv_sqrt((float)(s2 / cols) + na.eps);
        }
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            __half2 hh[4];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float4 v = xv[j][h];
                if (na.kind != 0) {
                    if (na.kind == 2) { v.x = __fsub_rn(v.x, mean); v.y = __fsub_rn(v.y, mean); v.z = __fsub_rn(v.z, mean); v.w = __fsub_rn(v.w, mean); }
                    v.x = __fmul_rn(v.x, scale); v.y = __fmul_rn(v.y, scale); v.z = __fmul_rn(v.z, scale); v.w = __fmul_rn(v.w, scale);
                    if (has_w) { const float4 w4 = wv[j][h]; v.x = __fmul_rn(v.x, w4.x); v.y = __fmul_rn(v.y, w4.y); v.z = __fmul_rn(v.z, w4.z); v.w = __fmul_rn(v.w, w4.w); }
                    if (na.b) {
                        const float4 b4 = *reinterpret_cast<const float4 *>(na.b + j * 512 + lane * 8 + 4 * h);
                        v.x = __fadd_rn(v.x, b4.x); v.y = __fadd_rn(v.y, b4.y); v.z = __fadd_rn(v.z, b4.z); v.w = __fadd_rn(v.w, b4.w);
                    }
                }
                hh[2 * h] = __floats2half2_rn(v.x, v.y); hh[2 * h + 1] = __floats2half2_rn(v.z, v.w);
            }
            xr[j] = *reinterpret_cast<const pi_u32x4 *>(hh);
        }
    }
    __syncthreads();
    // ---- activity word (identical in every wave) -----------------------------------------------------
    const float my_logit = lg[lane & 31];
    const bool my_act = !(my_logit < thr);
    const uint32_t mask = (uint32_t)__ballot(my_act);
    if (wave == 0) {
        if (lane < 32) { if (logits) logits[n0 + lane] = my_logit; if (!my_act) h_dense[n0 + lane] = 0.0f; }
        if (lane == 0) words[blockIdx.x] = mask;
    }
    // ---- phase B: two active neurons per wave per round trip ------------------------------------------
    const int n = __popc(mask);
    for (int k = wave; k < n; k += 2 * kWavesPerBlock) {
        const int rowA = n0 + select_nth_bit(mask, k);
        const bool twoB = k + kWavesPerBlock < n;
        const int rowB = twoB ? n0 + select_nth_bit(mask, k + kWavesPerBlock) : rowA;
        pi_u32x4 uA[NCH], gA[NCH], uB[NCH], gB[NCH];
#pragma unroll
        for (int j = 0; j < NCH; ++j) uA[j] = pi_ld_stream(Wup + (size_t)rowA * cols + (j * PI_WAVE + lane) * 8);
        if (Wgate) {
#pragma unroll
            for (int j = 0; j < NCH; ++j) gA[j] = pi_ld_stream(Wgate + (size_t)rowA * cols + (j * PI_WAVE + lane) * 8);
        }
        if (twoB) {
#pragma unroll
            for (int j = 0; j < NCH; ++j) uB[j] = pi_ld_stream(Wup + (size_t)rowB * cols + (j * PI_WAVE + lane) * 8);
            if (Wgate) {
#pragma unroll
                for (int j = 0; j < NCH; ++j) gB[j] = pi_ld_stream(Wgate + (size_t)rowB * cols + (j * PI_WAVE + lane) * 8);
            }
        }
        float au = 0.0f, ag = 0.0f, bu = 0.0f, bg = 0.0f;
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            float xf[8];
            pi_unpack8(xr[j], xf);
            au = pi_dot8(uA[j], xf, au);
            if (Wgate) ag = pi_dot8(gA[j], xf, ag);
        }
        au = pi_wave_sum(au);
        if (Wgate) ag = pi_wave_sum(ag);
        if (lane == 0) h_dense[rowA] = Wgate ? __fmul_rn(fmaxf(ag, 0.0f), au) : fmaxf(au, 0.0f);
        if (twoB) {
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                float xf[8];
                pi_unpack8(xr[j], xf);
                bu = pi_dot8(uB[j], xf, bu);
                if (Wgate) bg = pi_dot8(gB[j], xf, bg);
            }
            bu = pi_wave_sum(bu);
            if (Wgate) bg = pi_wave_sum(bg);
            if (lane == 0) h_dense[rowB] = Wgate ? __fmul_rn(fmaxf(bg, 0.0f), bu) : fmaxf(bu, 0.0f);
        }
    }
}

// compaction of existing mask words into the ascending active-row list (single block)
__global__ __launch_bounds__(1024) void compact_words_kernel(const uint32_t * __restrict__ words, int ff, const int32_t * bucket, int n_bucket,
                                                             int32_t * list, int32_t * n_active) {
    __shared__ int sred[17];
    compact_from_words(words, ff, bucket, n_bucket, list, n_active, sred);
}

// activity test + compaction over existing logits (single block)
__global__ __launch_bounds__(1024) void compact_kernel(const float * __restrict__ logits, int ff, float thr, const int32_t * bucket, int n_bucket,
                                                       uint32_t * words, int32_t * list, int32_t * n_active) {
    __shared__ int sred[17];
    const int lane = threadIdx.x & 63;
    for (int i0 = 0; i0 < ff; i0 += blockDim.x) {
        const int i = i0 + threadIdx.x;
        const bool act = (i < ff) && !(logits[i] < thr);
        const unsigned long long m = __ballot(act);
        if (lane == 0 && i < ff) words[i >> 5] = (uint32_t)m;
        if (lane == 32 && i < ff) words[i >> 5] = (uint32_t)(m >> 32);
    }
    __syncthreads();
    compact_from_words(words, ff, bucket, n_bucket, list, n_active, sred);
}

// ---------------------------------------------------------------------------------------------------
// Sparse up/gate straight from the predictor's mask words (F16).  Every workgroup turns the mask into a
// popcount prefix table in LDS (wave ballot happened in the predictor kernel, the prefix sum happens here),
// so rank k -> neuron row is a binary search + bit select and no separate compaction pass or list read sits
// on the critical path.  Wave w of the grid takes ranks w, w + n_waves, ...: it reads the gate row and the up
// row (2 x cols fp16, 128-bit loads, all issued before the first use), h = relu(g) * u (or relu(u) without a
// gate), and writes h_compact[k] and active_rows[k] = row, so the ascending index list is a by-product.
// ---------------------------------------------------------------------------------------------------
constexpr int kUpBlock = 512;       // 8 waves
constexpr int kUpBlocks = 256;      // about one workgroup per CU: 2048 waves >= the active count of the 7B..40B shapes


template <int NCH>      // cols == 512 * NCH
__global__ __launch_bounds__(kUpBlock) void sparse_upgate_mask_f16_kernel(const __half * __restrict__ Wup, const __half * __restrict__ Wgate,
                                                                          const float * __restrict__ x, NormArgs na, int cols, int ff,
                                                                          const uint32_t * __restrict__ words,
                                                                          int32_t * __restrict__ list, int32_t * __restrict__ n_active,
                                                                          float * __restrict__ h_compact, float * h_dense) {
    extern __shared__ __align__(16) unsigned char smem[];
    float  * lds = reinterpret_cast<float *>(smem);                       // xraw[cols] | wn[cols]
    __half * xs  = reinterpret_cast<__half *>(smem + (size_t)cols * 8);
    int    * prefix = reinterpret_cast<int *>(smem + (size_t)cols * 10);  // [nwords + 1]
    uint32_t * wbits = reinterpret_cast<uint32_t *>(prefix + (ff + 31) / 32 + 1);
    __shared__ double red[16];
    __shared__ int sred[kUpBlock / PI_WAVE + 1];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwords = (ff + 31) / 32;
    constexpr int kWaves = kUpBlock / PI_WAVE;

    // one memory round trip: activations (+ norm weights) by direct-to-LDS loads, mask words by ordinary loads
    stage_fast_issue(lds, x, na, cols);
    int base_cnt = 0;
    for (int w0 = 0; w0 < nwords; w0 += kUpBlock) {
        const int w = w0 + threadIdx.x;
        const uint32_t bits = w < nwords ? words[w] : 0u;
        int tot;
        const int off = base_cnt + block_exclusive_scan_i32(__popc(bits), &tot, sred);
        if (w < nwords) { prefix[w] = off; wbits[w] = bits; }
        base_cnt += tot;
    }
    const int n = base_cnt;
    if (threadIdx.x == 0) { prefix[nwords] = n; if (blockIdx.x == 0) *n_active = n; }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if ((int)(blockIdx.x * kWaves) >= n) return;                           // no rank for this workgroup (uniform)

    stage_fast_finish(xs, lds, na, cols, red);

    for (int k = blockIdx.x * kWaves + wave; k < n; k += gridDim.x * kWaves) {
        // word holding rank k: largest w with prefix[w] <= k
        int lo = 0, hi = nwords - 1;
        while (lo < hi) { const int mid = (lo + hi + 1) >> 1; if (prefix[mid] <= k) lo = mid; else hi = mid - 1; }
        const int row = lo * 32 + select_nth_bit(wbits[lo], k - prefix[lo]);
        const __half * wu = Wup + (size_t)row * cols + lane * 8;
        pi_u32x4 bu[NCH], bg[NCH];
#pragma unroll
        for (int u = 0; u < NCH; ++u) bu[u] = pi_ld_stream(wu + u * (PI_WAVE * 8));
        if (Wgate) {
            const __half * wg = Wgate + (size_t)row * cols + lane * 8;
#pragma unroll
            for (int u = 0; u < NCH; ++u) bg[u] = pi_ld_stream(wg + u * (PI_WAVE * 8));
        }
        float au = 0.0f, ag = 0.0f;
#pragma unroll
        for (int u = 0; u < NCH; ++u) {
            float xf[8];
            pi_unpack8(pi_ld16(xs + (u * PI_WAVE + lane) * 8), xf);
            au = pi_dot8(bu[u], xf, au);
            if (Wgate) ag = pi_dot8(bg[u], xf, ag);
        }
        au = pi_wave_sum(au);
        if (Wgate) ag = pi_wave_sum(ag);
        if (lane == 0) {
            const float h = Wgate ? __fmul_rn(fmaxf(ag, 0.0f), au) : fmaxf(au, 0.0f);
            h_compact[k] = h;
            list[k] = row;
            if (h_dense) h_dense[row] = h;
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Sparse up/gate over the active list.  One wave per active row: reads the gate row and the up row
// (2 x cols fp16) with 128-bit loads, fp32 accumulate, h = relu(g) * u (or relu(u) without a gate).
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void sparse_upgate_f16_kernel(const __half * __restrict__ Wup, const __half * __restrict__ Wgate,
                                                                   const float * __restrict__ x, NormArgs na, int cols,
                                                                   const int32_t * __restrict__ list, const int32_t * __restrict__ n_active,
                                                                   const int32_t * __restrict__ bucket, float * __restrict__ h_compact,
                                                                   float * h_dense, float * up_dense, float * gate_dense) {
    extern __shared__ __align__(16) unsigned char smem[];
    __half * xs = reinterpret_cast<__half *>(smem);
    __shared__ double red[16];
    const int n = *n_active;
    if ((int)(blockIdx.x * kWavesPerBlock) >= n) return;       // whole block idle (uniform)
    stage_x_f16(xs, x, cols, na, red);

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int k = blockIdx.x * kWavesPerBlock + wave; k < n; k += gridDim.x * kWavesPerBlock) {
        const int row = list[k];
        const __half * wu = Wup + (size_t)row * cols;
        const __half * wg = Wgate ? Wgate + (size_t)row * cols : nullptr;
        float au = 0.0f, ag = 0.0f;
#pragma unroll 4
        for (int c = lane * 8; c < cols; c += PI_WAVE * 8) {
            float xf[8];
            pi_unpack8(pi_ld16(xs + c), xf);
            au = pi_dot8(pi_ld_stream(wu + c), xf, au);
            if (wg) ag = pi_dot8(pi_ld_stream(wg + c), xf, ag);
        }
        au = pi_wave_sum(au);
        if (wg) ag = pi_wave_sum(ag);
        if (lane == 0) {
            const float h = wg ? __fmul_rn(fmaxf(ag, 0.0f), au) : fmaxf(au, 0.0f);
            h_compact[k] = h;
            const int neuron = bucket ? bucket[row] : row;
            if (h_dense) h_dense[neuron] = h;
            if (up_dense) up_dense[neuron] = au;
            if (gate_dense && wg) gate_dense[neuron] = ag;
        }
    }
}

__global__ __launch_bounds__(kBlock) void sparse_upgate_q4_kernel(const pi_block_q4_0 * __restrict__ Wup, const pi_block_q4_0 * __restrict__ Wgate,
                                                                  const float * __restrict__ x, NormArgs na, int cols,
                                                                  const int32_t * __restrict__ list, const int32_t * __restrict__ n_active,
                                                                  const int32_t * __restrict__ bucket, float * __restrict__ h_compact,
                                                                  float * h_dense, float * up_dense, float * gate_dense) {
    extern __shared__ __align__(16) unsigned char smem[];
    int8_t * xq   = reinterpret_cast<int8_t *>(smem);
    float  * xd   = reinterpret_cast<float *>(smem + cols);
    float  * xtmp = reinterpret_cast<float *>(smem + cols + (cols / 32) * 4);
    __shared__ double red[16];
    const int n = *n_active;
    if ((int)(blockIdx.x * kWavesPerBlock) >= n) return;
    stage_x_q8(xq, xd, x, cols, na, red, xtmp);

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nb = cols / 32;
    for (int k = blockIdx.x * kWavesPerBlock + wave; k < n; k += gridDim.x * kWavesPerBlock) {
        const int row = list[k];
        const pi_block_q4_0 * wu = Wup + (size_t)row * nb;
        const pi_block_q4_0 * wg = Wgate ? Wgate + (size_t)row * nb : nullptr;
        float au = 0.0f, ag = 0.0f;
        for (int b = lane; b < nb; b += PI_WAVE) {
            const float dx = xd[b];
            au = q4_block_dot(wu + b, xq + b * 32, dx, au);
            if (wg) ag = q4_block_dot(wg + b, xq + b * 32, dx, ag);
        }
        au = pi_wave_sum(au);
        if (wg) ag = pi_wave_sum(ag);
        if (lane == 0) {
            const float h = wg ? __fmul_rn(fmaxf(ag, 0.0f), au) : fmaxf(au, 0.0f);
            h_compact[k] = h;
            const int neuron = bucket ? bucket[row] : row;
            if (h_dense) h_dense[neuron] = h;
            if (up_dense) up_dense[neuron] = au;
            if (gate_dense && wg) gate_dense[neuron] = ag;
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Sparse down projection (axpy).  grid = (column tiles of 512, G row groups).  Wave w of block (t, g)
// takes active rows k = g*4 + w, +4G, ... and accumulates h_k * down_t[row_k][tile] in 8 fp32 registers
// per lane; the four waves merge through LDS; the partial tile goes to scratch; the block that finishes
// last for the tile adds the G partials in order, applies the epilogue and stores.  No float atomics,
// so the sum order -- and the result -- is fixed.  h is rounded to fp16 first and zero rows are skipped
// as on the CPU path (ggml.c:14420-14431).
// ---------------------------------------------------------------------------------------------------
// F16 down projection with the whole reduction inside the workgroup: a workgroup owns 128 output columns
// (lane = 2 columns, one 32-bit load per row) and all active rows; its 16 waves split the rows, accumulate in
// registers and merge through LDS in wave order, so there is no inter-workgroup reduction, no atomics and no
// fence, and the sum order is fixed.  Entries whose fp16-rounded h is zero are dropped by a workgroup-level
// ballot/prefix compaction before any weight is read.
constexpr int kAxBlock = 1024;
constexpr int kAxWaves = kAxBlock / PI_WAVE;
constexpr int kAxCap = 2048;        // compacted entries held in LDS per round
constexpr int kAxUn = 16;           // rows in flight per wave

__global__ __launch_bounds__(kAxBlock) void sparse_axpy_lds_f16_kernel(const __half * __restrict__ Wd, int cols, int n_max,
                                                                       const float * __restrict__ h_compact, const int32_t * __restrict__ list,
                                                                       const int32_t * __restrict__ n_active,
                                                                       int epi, const float * add1, const float * add2, float * __restrict__ out) {
    __shared__ int   crow[kAxCap];
    __shared__ float ca[kAxCap];
    __shared__ float redl[kAxWaves][128];
    __shared__ int   sred[kAxWaves + 1];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int col = blockIdx.x * 128 + lane * 2;
    // the first kAxBlock entries are fetched before the count is known (same round trip); stale slots are masked below
    float a_spec = tid < n_max ? h_compact[tid] : 0.0f;
    int   r_spec = tid < n_max ? list[tid] : 0;
    const int n = *n_active;
    float acc0 = 0.0f, acc1 = 0.0f;
    int k0 = 0;
    while (k0 < n) {
        // ---- compact up to kAxCap non-zero entries starting at k0 -----------------------------------
        int m = 0;
        while (k0 < n && m + kAxBlock <= kAxCap) {
            const int k = k0 + tid;
            float a; int r;
            if (k0 == 0) { a = a_spec; r = r_spec; } else { a = k < n ? h_compact[k] : 0.0f; r = k < n ? list[k] : 0; }
            a = pi_round_f16(a);
            const int nz = (k < n && a != 0.0f) ? 1 : 0;
            int tot;
            const int off = m + block_exclusive_scan_i32(nz, &tot, sred);
            if (nz) { crow[off] = r; ca[off] = a; }
            m += tot;
            k0 += kAxBlock;
        }
        __syncthreads();
        // ---- rows wave, wave + 16, ... of the compacted list ---------------------------------------
        for (int i0 = wave; i0 < m; i0 += kAxWaves * kAxUn) {
            uint32_t w[kAxUn]; float a[kAxUn];
#pragma unroll
            for (int u = 0; u < kAxUn; ++u) {
                const int i = i0 + u * kAxWaves;
                const bool ok = i < m;
                a[u] = ok ? ca[i] : 0.0f;
                w[u] = ok ? __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(Wd + (size_t)crow[i] * cols + col)) : 0u;
            }
#pragma unroll
            for (int u = 0; u < kAxUn; ++u) {
                const float2 f = __half22float2(*reinterpret_cast<const __half2 *>(&w[u]));
                acc0 = fmaf(f.x, a[u], acc0);
                acc1 = fmaf(f.y, a[u], acc1);
            }
        }
        __syncthreads();
    }
    redl[wave][lane * 2] = acc0;
    redl[wave][lane * 2 + 1] = acc1;
    __syncthreads();
    if (tid < 128) {
        float sum = redl[0][tid];
#pragma unroll
        for (int w = 1; w < kAxWaves; ++w) sum += redl[w][tid];
        const int c = blockIdx.x * 128 + tid;
        out[c] = apply_epilogue(sum, epi, add1, add2, c);
    }
}

// ---------------------------------------------------------------------------------------------------
// F16 down projection straight from the dense h vector (0 for inactive neurons).  A workgroup of 16 waves owns
// 64 output columns and all rows.  Every thread fetches its share of h in one go (16 values per 16384
// neurons), rounds to fp16 as the CPU path does and drops zeros (ggml.c:14420-14431); wave ballots give the
// per-(round, wave) counts, one workgroup scan turns them into offsets, and the surviving (row, h) pairs land
// in LDS in ascending row order.  Then one round trip of weight loads: 8 lanes cover the 128-byte segment of
// a row, a wave load instruction covers 8 rows, 8 instructions are in flight per lane.  The 8 row slots of a
// wave merge by shuffles, the 16 waves through LDS in wave order: fixed summation order, no atomics.
// Workgroup 0 also counts the predictor's active neurons from the mask words.
// ---------------------------------------------------------------------------------------------------
constexpr int kAdTile = 64;
constexpr int kAdCap = 4096;         // (row, h) pairs held in LDS per pass
constexpr int kAdRounds = 16;        // h values per thread per super-group of 16384 neurons
constexpr int kAdUn = 8;

__global__ __launch_bounds__(kAxBlock) void sparse_axpy_dense_f16_kernel(const __half * __restrict__ Wd, int cols, int ff,
                                                                         const float * __restrict__ h_dense, const uint32_t * __restrict__ words,
                                                                         int32_t * __restrict__ n_active_out,
                                                                         int epi, const float * add1, const float * add2, float * __restrict__ out) {
    __shared__ int   crow[kAdCap];
    __shared__ float ca[kAdCap];
    __shared__ int   cnt[kAdRounds * kAxWaves];
    __shared__ float redl[kAxWaves][kAdTile];
    __shared__ int   sred[kAxWaves + 1];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int sub = lane >> 3, col = blockIdx.x * kAdTile + (lane & 7) * 8;
    const unsigned long long lt = (1ull << lane) - 1ull;
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.0f;

    for (int base = 0; base < ff; base += kAdRounds * kAxBlock) {
        float hv[kAdRounds];
#pragma unroll
        for (int i = 0; i < kAdRounds; ++i) {
            const int idx = base + i * kAxBlock + tid;
            hv[i] = idx < ff ? h_dense[idx] : 0.0f;
        }
        int lp[kAdRounds];
#pragma unroll
        for (int i = 0; i < kAdRounds; ++i) {
            hv[i] = pi_round_f16(hv[i]);
            const unsigned long long m = __ballot(hv[i] != 0.0f);
            lp[i] = __popcll(m & lt);
            if (lane == 0) cnt[i * kAxWaves + wave] = __popcll(m);
        }
        __syncthreads();
        int tot;
        const int v = tid < kAdRounds * kAxWaves ? cnt[tid] : 0;
        const int off = block_exclusive_scan_i32(v, &tot, sred);
        __syncthreads();
        if (tid < kAdRounds * kAxWaves) cnt[tid] = off;
        __syncthreads();
        for (int c0 = 0; c0 < tot; c0 += kAdCap) {
#pragma unroll
            for (int i = 0; i < kAdRounds; ++i) {
                if (hv[i] != 0.0f) {
                    const int o = cnt[i * kAxWaves + wave] + lp[i] - c0;
                    if (o >= 0 && o < kAdCap) { crow[o] = base + i * kAxBlock + tid; ca[o] = hv[i]; }
                }
            }
            __syncthreads();
            const int m = tot - c0 < kAdCap ? tot - c0 : kAdCap;
            for (int i0 = wave * 8 + sub; i0 < m; i0 += kAxWaves * 8 * kAdUn) {
                pi_u32x4 w[kAdUn]; float a[kAdUn];
#pragma unroll
                for (int u = 0; u < kAdUn; ++u) {
                    const int i = i0 + u * kAxWaves * 8;
                    const bool ok = i < m;
                    a[u] = ok ? ca[i] : 0.0f;
                    w[u] = ok ? pi_ld_stream(Wd + (size_t)crow[i] * cols + col) : pi_u32x4{0u, 0u, 0u, 0u};
                }
#pragma unroll
                for (int u = 0; u < kAdUn; ++u) {
                    float wf[8];
                    pi_unpack8(w[u], wf);
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[j] = fmaf(wf[j], a[u], acc[j]);
                }
            }
            __syncthreads();
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        acc[j] += __shfl_xor(acc[j], 8, PI_WAVE);
        acc[j] += __shfl_xor(acc[j], 16, PI_WAVE);
        acc[j] += __shfl_xor(acc[j], 32, PI_WAVE);
    }
    if (lane < 8) {
#pragma unroll
        for (int j = 0; j < 8; ++j) redl[wave][lane * 8 + j] = acc[j];
    }
    __syncthreads();
    if (tid < kAdTile) {
        float sum = redl[0][tid];
#pragma unroll
        for (int w = 1; w < kAxWaves; ++w) sum += redl[w][tid];
        const int c = blockIdx.x * kAdTile + tid;
        out[c] = apply_epilogue(sum, epi, add1, add2, c);
    }
    if (blockIdx.x == 0 && n_active_out && words) {
        int c = 0;
        for (int w = tid; w < (ff + 31) / 32; w += kAxBlock) c += __popc(words[w]);
        c = pi_wave_sum_i32(c);
        __syncthreads();
        if (lane == 0) sred[wave] = c;
        __syncthreads();
        if (tid == 0) { int t = 0; for (int w = 0; w < kAxWaves; ++w) t += sred[w]; *n_active_out = t; }
    }
}


__device__ void axpy_finish(float * acc, float * lds, float * partial, unsigned int * tile_counter, int cols,
                            int epi, const float * add1, const float * add2, float * out, int * sflag) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int tile = blockIdx.x, g = blockIdx.y, G = gridDim.y;
#pragma unroll
    for (int i = 0; i < 8; ++i) lds[wave * kAxpyTile + lane * 8 + i] = acc[i];
    __syncthreads();
    for (int c = threadIdx.x; c < kAxpyTile; c += blockDim.x) {
        const int col = tile * kAxpyTile + c;
        if (col < cols) {
            float s = lds[c];
            for (int w = 1; w < kWavesPerBlock; ++w) s += lds[w * kAxpyTile + c];
            partial[(size_t)g * cols + col] = s;
        }
    }
    if (last_block_done(&tile_counter[tile], G, sflag)) {
        for (int c = threadIdx.x; c < kAxpyTile; c += blockDim.x) {
            const int col = tile * kAxpyTile + c;
            if (col < cols) {
                float s = partial[col];
                for (int gg = 1; gg < G; ++gg) s += partial[(size_t)gg * cols + col];
                out[col] = apply_epilogue(s, epi, add1, add2, col);
            }
        }
    }
}

__global__ __launch_bounds__(kBlock) void sparse_axpy_f16_kernel(const __half * __restrict__ Wd, int cols, const float * __restrict__ h_compact,
                                                                 const int32_t * __restrict__ list, const int32_t * __restrict__ n_active,
                                                                 float * partial, unsigned int * tile_counter,
                                                                 int epi, const float * add1, const float * add2, float * out) {
    __shared__ float lds[kWavesPerBlock * kAxpyTile];
    __shared__ int sflag;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col = blockIdx.x * kAxpyTile + lane * 8;
    const int n = *n_active;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    if (col < cols) {
        const int stride = gridDim.y * kWavesPerBlock;
#pragma unroll 4
        for (int k = blockIdx.y * kWavesPerBlock + wave; k < n; k += stride) {
            const float a = pi_round_f16(h_compact[k]);
            if (a == 0.0f) continue;
            float wf[8];
            pi_unpack8(pi_ld_stream(Wd + (size_t)list[k] * cols + col), wf);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = fmaf(wf[i], a, acc[i]);
        }
    }
    axpy_finish(acc, lds, partial, tile_counter, cols, epi, add1, add2, out, &sflag);
}

// Q4_0 axpy (ggml_compute_forward_mul_mat_axpy_q4_0, ggml.c:14465-14618; ggml_axpy_q4_0_q8_0, ggml-quants.c:2426):
// h is quantised to Q8_0 over blocks of 32 *neurons* (in the dense [ff] index space on the CPU).  Here the
// caller passes h already quantised per active row: hq[k] (int8) and hd[k] (fp16-rounded block scale).
__global__ __launch_bounds__(kBlock) void sparse_axpy_q4_kernel(const pi_block_q4_0 * __restrict__ Wd, int cols, const int32_t * __restrict__ hq,
                                                                const float * __restrict__ hd,
                                                                const int32_t * __restrict__ list, const int32_t * __restrict__ n_active,
                                                                float * partial, unsigned int * tile_counter,
                                                                int epi, const float * add1, const float * add2, float * out) {
    __shared__ float lds[kWavesPerBlock * kAxpyTile];
    __shared__ int sflag;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // lane covers 8 columns: a quarter of one 32-weight block -> elements (lane&3)*8 .. +8 of block col/32
    const int col = blockIdx.x * kAxpyTile + lane * 8;
    const int nb = cols / 32;
    const int n = *n_active;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    if (col < cols) {
        const int blk = col >> 5, sub = (col >> 3) & 3;          // sub 0,1: low nibbles of qs[0..7], qs[8..15]; sub 2,3: high nibbles
        const int stride = gridDim.y * kWavesPerBlock;
        for (int k = blockIdx.y * kWavesPerBlock + wave; k < n; k += stride) {
            const int alpha = hq[k];
            if (alpha == 0) continue;
            const pi_block_q4_0 * wb = Wd + (size_t)list[k] * nb + blk;
            uint16_t dbits; uint32_t q[2];
            __builtin_memcpy(&dbits, &wb->d, 2);
            __builtin_memcpy(q, wb->qs + (sub & 1) * 8, 8);
            const float d = __fmul_rn(pi_f16_from_bits(dbits), hd[k]);
            const int shift = (sub >> 1) * 4;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int v = (int)((q[i >> 2] >> ((i & 3) * 8 + shift)) & 0xF) - 8;
                acc[i] = __fadd_rn(acc[i], __fmul_rn((float)(v * alpha), d));
            }
        }
    }
    axpy_finish(acc, lds, partial, tile_counter, cols, epi, add1, add2, out, &sflag);
}

// Q8_0 quantisation of h for the Q4_0 axpy.  The CPU path quantises the dense [ff] vector in blocks of 32
// neurons (inactive neurons contribute zeros), so the scale of an active neuron depends on its 31 block
// neighbours.  For each active row this reads the neuron's block from the dense vector and emits the
// int8 value hq[k] and the fp16-rounded block scale hd[k].
__global__ __launch_bounds__(kBlock) void h_q8_gather_kernel(const float * __restrict__ h_dense, const int32_t * __restrict__ list,
                                                             const int32_t * __restrict__ n_active, const int32_t * __restrict__ bucket,
                                                             int32_t * __restrict__ hq, float * __restrict__ hd) {
    const int n = *n_active;
    for (int k = blockIdx.x * blockDim.x + threadIdx.x; k < n; k += gridDim.x * blockDim.x) {
        const int row = list[k];
        const int neuron = bucket ? bucket[row] : row;
        const float * blk = h_dense + (neuron & ~31);
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(blk[j]));
        const float d = pi_div(amax, 127.0f);
        const float id = (amax != 0.0f) ? pi_div(127.0f, amax) : 0.0f;
        hq[k] = (int)rintf(__fmul_rn(h_dense[neuron], id));
        hd[k] = pi_round_f16(d);
    }
}


}  // namespace

extern "C" {

int pi_k_predictor_fc2(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                       const int32_t * bucket, int n_bucket, float * logits,
                       int32_t * active_rows, int32_t * n_active, float * zero_fill, pi_workspace * ws, pi_stream_t stream) {
    if (!fc2_f16 || !hidden || !logits || !ws) return pi::fail(PI_E_ARG, "pi_k_predictor_fc2: null pointer");
    if ((active_rows == nullptr) != (n_active == nullptr)) return pi::fail(PI_E_ARG, "pi_k_predictor_fc2: active_rows and n_active go together");
    if (ff <= 0 || r <= 0 || r % 8 || ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_predictor_fc2: bad shape (r % 8 == 0, ff <= workspace)");
    if (bucket && (n_bucket < 0 || n_bucket > ff)) return pi::fail(PI_E_ARG, "pi_k_predictor_fc2: bad bucket size");
    if (bucket && !active_rows) return pi::fail(PI_E_ARG, "pi_k_predictor_fc2: a bucket needs the explicit row list");
    const int blocks = (ff + 31) / 32;
    hipStream_t st = (hipStream_t)stream;
    const __half * w = (const __half *)fc2_f16;
    const size_t sh = (size_t)r * 6;
    const bool aligned = (((uintptr_t)hidden) & 15) == 0;
    if (r == 1024 && aligned)     hipLaunchKernelGGL(pred_fc2_kernel<2>, dim3(blocks), dim3(kBlock), sh, st, w, hidden, ff, r, threshold, logits, ws->words, zero_fill);
    else if (r == 512 && aligned) hipLaunchKernelGGL(pred_fc2_kernel<1>, dim3(blocks), dim3(kBlock), sh, st, w, hidden, ff, r, threshold, logits, ws->words, zero_fill);
    else                          hipLaunchKernelGGL(pred_fc2_kernel<0>, dim3(blocks), dim3(kBlock), sh, st, w, hidden, ff, r, threshold, logits, ws->words, zero_fill);
    if (active_rows)
        hipLaunchKernelGGL(compact_words_kernel, dim3(1), dim3(1024), 0, st, ws->words, ff, bucket, n_bucket, active_rows, n_active);
    return pi::check_launch("pi_k_predictor_fc2");
}

int pi_k_compact_active(const float * logits, int ff, float threshold, const int32_t * bucket, int n_bucket,
                        int32_t * active_rows, int32_t * n_active, pi_workspace * ws, pi_stream_t stream) {
    if (!logits || !active_rows || !n_active || !ws || ff <= 0 || ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_compact_active: bad arguments");
    if (bucket && (n_bucket < 0 || n_bucket > ff)) return pi::fail(PI_E_ARG, "pi_k_compact_active: bad bucket size");
    hipLaunchKernelGGL(compact_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, logits, ff, threshold, bucket, n_bucket, ws->words, active_rows, n_active);
    return pi::check_launch("pi_k_compact_active");
}

int pi_k_sparse_upgate(int wtype, const void * up, const void * gate, int cols, int ff, const float * x, const pi_norm * norm,
                       int from_mask, int32_t * active_rows, int32_t * n_active, const int32_t * bucket,
                       float * h_compact, float * h_dense, float * up_dense, float * gate_dense, pi_workspace * ws, pi_stream_t stream) {
    if (!up || !x || !active_rows || !n_active || !h_compact || cols <= 0) return pi::fail(PI_E_ARG, "pi_k_sparse_upgate: null pointer or empty shape");
    const NormArgs na = to_norm(norm);
    hipStream_t st = (hipStream_t)stream;
    if (from_mask) {
        if (!ws || ff <= 0 || ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_sparse_upgate: the mask lives in the workspace (ff <= workspace)");
        if (bucket) return pi::fail(PI_E_ARG, "pi_k_sparse_upgate: a bucket needs the explicit row list (from_mask = 0)");
        const size_t sh = (size_t)cols * 10 + (size_t)((ff + 31) / 32) * 8 + 16;
        const bool aligned = ((((uintptr_t)x) | (uintptr_t)na.w) & 15) == 0;
        const bool fast = wtype == PI_TYPE_F16 && cols % 512 == 0 && cols / 512 <= 8 && sh <= 64 * 1024 && aligned && !up_dense && !gate_dense;
        if (fast) {
            const __half * u = (const __half *)up; const __half * g = (const __half *)gate;
            const int nch = cols / 512;
#define PI_UP_CASE(N) case N: hipLaunchKernelGGL(sparse_upgate_mask_f16_kernel<N>, dim3(kUpBlocks), dim3(kUpBlock), sh, st, u, g, x, na, cols, ff, ws->words, active_rows, n_active, h_compact, h_dense); break;
            switch (nch) { PI_UP_CASE(1) PI_UP_CASE(2) PI_UP_CASE(4) PI_UP_CASE(8)
                default: hipLaunchKernelGGL(compact_words_kernel, dim3(1), dim3(1024), 0, st, ws->words, ff, nullptr, 0, active_rows, n_active); goto list_mode; }
#undef PI_UP_CASE
            return pi::check_launch("pi_k_sparse_upgate");
        }
        // shapes the fused kernel does not cover: materialise the list first
        hipLaunchKernelGGL(compact_words_kernel, dim3(1), dim3(1024), 0, st, ws->words, ff, nullptr, 0, active_rows, n_active);
    }
list_mode:
    {
        const int blocks = 1024;       // fixed grid: the active count lives on the device; idle blocks exit at once
        if (wtype == PI_TYPE_F16) {
            if (cols % 8 || (size_t)cols * 2 > 60 * 1024) return pi::fail(PI_E_ARG, "pi_k_sparse_upgate: bad cols for F16");
            hipLaunchKernelGGL(sparse_upgate_f16_kernel, dim3(blocks), dim3(kBlock), (size_t)cols * 2, st,
                               (const __half *)up, (const __half *)gate, x, na, cols, active_rows, n_active, bucket, h_compact, h_dense, up_dense, gate_dense);
        } else if (wtype == PI_TYPE_Q4_0) {
            const size_t sh = (size_t)cols + (size_t)(cols / 32) * 4 + (size_t)cols * 4;
            if (cols % 32 || sh > 60 * 1024) return pi::fail(PI_E_ARG, "pi_k_sparse_upgate: bad cols for Q4_0");
            hipLaunchKernelGGL(sparse_upgate_q4_kernel, dim3(blocks), dim3(kBlock), sh, st,
                               (const pi_block_q4_0 *)up, (const pi_block_q4_0 *)gate, x, na, cols, active_rows, n_active, bucket, h_compact, h_dense, up_dense, gate_dense);
        } else {
            return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_upgate: weight type must be F16 or Q4_0");
        }
    }
    return pi::check_launch("pi_k_sparse_upgate");
}

int pi_k_sparse_axpy(int wtype, const void * down_t, int cols, int n_rows, const float * h_compact, const float * h_dense, const int32_t * bucket,
                     const int32_t * active_rows, const int32_t * n_active,
                     int epilogue, const float * add1, const float * add2, float * out,
                     pi_workspace * ws, pi_stream_t stream) {
    if (!down_t || !h_compact || !active_rows || !n_active || !out || !ws) return pi::fail(PI_E_ARG, "pi_k_sparse_axpy: null pointer");
    if (cols <= 0 || cols > ws->max_d || n_rows <= 0) return pi::fail(PI_E_ARG, "pi_k_sparse_axpy: cols exceeds the workspace or n_rows <= 0");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || epilogue == PI_EPI_RELU || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_sparse_axpy: bad epilogue arguments");
    const int tiles = (cols + kAxpyTile - 1) / kAxpyTile;
    const dim3 grid(tiles, kAxpyGroups);
    hipStream_t st = (hipStream_t)stream;
    if (wtype == PI_TYPE_F16) {
        if (cols % 8) return pi::fail(PI_E_ARG, "pi_k_sparse_axpy: F16 needs cols % 8 == 0");
        if (cols % 128 == 0)
            hipLaunchKernelGGL(sparse_axpy_lds_f16_kernel, dim3(cols / 128), dim3(kAxBlock), 0, st,
                               (const __half *)down_t, cols, n_rows, h_compact, active_rows, n_active, epilogue, add1, add2, out);
        else
            hipLaunchKernelGGL(sparse_axpy_f16_kernel, grid, dim3(kBlock), 0, st,
                               (const __half *)down_t, cols, h_compact, active_rows, n_active, ws->partial, ws->counters + 1, epilogue, add1, add2, out);
    } else if (wtype == PI_TYPE_Q4_0) {
        if (cols % 32) return pi::fail(PI_E_ARG, "pi_k_sparse_axpy: Q4_0 needs cols % 32 == 0");
        if (!h_dense) return pi::fail(PI_E_ARG, "pi_k_sparse_axpy: Q4_0 needs the dense h vector (block scales span 32 neurons)");
        hipLaunchKernelGGL(h_q8_gather_kernel, dim3(64), dim3(kBlock), 0, st, h_dense, active_rows, n_active, bucket, ws->hq, ws->hd);
        hipLaunchKernelGGL(sparse_axpy_q4_kernel, grid, dim3(kBlock), 0, st,
                           (const pi_block_q4_0 *)down_t, cols, ws->hq, ws->hd, active_rows, n_active, ws->partial, ws->counters + 1, epilogue, add1, add2, out);
    } else {
        return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_axpy: weight type must be F16 or Q4_0");
    }
    return pi::check_launch("pi_k_sparse_axpy");
}

int pi_k_pred_upgate(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                     const void * up_f16, const void * gate_f16, int cols, const float * x, const pi_norm * norm,
                     float * logits, float * h_dense, pi_workspace * ws, pi_stream_t stream) {
    if (!fc2_f16 || !hidden || !up_f16 || !x || !h_dense || !ws) return pi::fail(PI_E_ARG, "pi_k_pred_upgate: null pointer");
    if (!pi_k_pred_upgate_supported(ff, r, cols)) return pi::fail(PI_E_UNSUPPORTED, "pi_k_pred_upgate: shape outside the fused kernel (cols 4096, r 1024, ff % 32 == 0)");
    if (ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_pred_upgate: ff exceeds the workspace");
    const NormArgs na = to_norm(norm);
    if ((((uintptr_t)hidden | (uintptr_t)x | (uintptr_t)na.w | (uintptr_t)na.b) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_pred_upgate: vectors must be 16-byte aligned");
    hipLaunchKernelGGL((pred_upgate_f16_kernel<8, 2>), dim3(ff / 32), dim3(kBlock), 0, (hipStream_t)stream,
                       (const __half *)fc2_f16, hidden, (const __half *)up_f16, (const __half *)gate_f16, x, na, threshold, logits, ws->words, h_dense);
    return pi::check_launch("pi_k_pred_upgate");
}

int pi_k_pred_upgate_supported(int ff, int r, int cols) { return cols == 4096 && r == 1024 && ff > 0 && ff % 32 == 0; }

int pi_k_sparse_axpy_dense(const void * down_t_f16, int cols, int ff, const float * h_dense, int32_t * n_active,
                           int epilogue, const float * add1, const float * add2, float * out, pi_workspace * ws, pi_stream_t stream) {
    if (!down_t_f16 || !h_dense || !out || !ws) return pi::fail(PI_E_ARG, "pi_k_sparse_axpy_dense: null pointer");
    if (cols <= 0 || cols % kAdTile || ff <= 0 || ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_sparse_axpy_dense: cols % 64 == 0 and ff <= workspace required");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || epilogue == PI_EPI_RELU || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_sparse_axpy_dense: bad epilogue arguments");
    hipLaunchKernelGGL(sparse_axpy_dense_f16_kernel, dim3(cols / kAdTile), dim3(kAxBlock), 0, (hipStream_t)stream,
                       (const __half *)down_t_f16, cols, ff, h_dense, ws->words, n_active, epilogue, add1, add2, out);
    return pi::check_launch("pi_k_sparse_axpy_dense");
}

}  // extern "C"

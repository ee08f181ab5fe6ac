// The sparse FFN of one token as one launch plus a reduction (F16: one workgroup per compute unit or per 32 neurons; Q4_0: per 32
// neurons, one Q8_0 block of h), the two-phase forms of hybrid layers with their hand-over kernels, and the entry point that allocates
// nothing.
#include "kernels_common.hpp"

namespace {

// ---------------------------------------------------------------------------------------------------
// The whole sparse FFN of one token behind fc1, in one launch plus a small reduction (F16, cols == 4096).
// A workgroup of 8 waves owns 32 consecutive neurons.
//   A  wave w computes 4 of the 32 predictor logits (fc2 rows, r == 512*RCH) and, meanwhile, loads ITS eighth
//      of the FFN input and of the norm weights (columns [512w, 512w+512): 8 values per lane); the sum of squares
//      (and the mean for LayerNorm) crosses the waves through LDS, after which each wave holds its slice of
//      fp16(norm(x)) in four registers.  Nobody reads the whole vector.
//   B  the 32 logits meet in LDS, every wave derives the same activity word, and for up to 8 active neurons
//      at a time wave w loads ITS 512-column slice of the gate, up and down rows (one 16-byte load per lane and
//      row, all issued together), so the work is balanced whatever the number of active neurons.  The partial
//      gate/up dots cross the waves through LDS in wave order; h = relu(g)*u (relu(u) without a gate).
//   C  out_partial[workgroup][512w + 8*lane ..] += fp16(h) * down slice: the wave owns its columns, so the
//      workgroup's contribution needs no further merge and is stored once.
// ffn_reduce_kernel then adds the per-workgroup partial vectors in workgroup order plus the residual(s).
// Two dependent memory round trips (A, B+C) instead of four kernels; summation order fixed, no atomics.
// ---------------------------------------------------------------------------------------------------
constexpr int kPfBlock = 512;
constexpr int kPfWaves = kPfBlock / PI_WAVE;      // 8 column slices of 512
constexpr int kPfChunk = 8;                       // active neurons per round trip


// HYB: a hot/cold split layer.  Only the GPU-resident neurons are computed (mask & hot word; weight row = hot prefix + rank among
// the hot bits: the compact matrices of the bucket), the activity words of that share go to words_hot, and workgroup 0 hands the
// fp16-rounded normalised input to the host share (xn_out; like logits it may be pinned host memory).
// PHASE 1 / 2 (G == 1) cut the launch in two for a hybrid layer whose host share should start behind the predictor: 1 stops after the
// logits (to `logits` and `logits2`), the mask words and the fp16 input for the host; 2 reads the logits back from `logits2`.
// a hand-over to the host announced by the first lane of a launch (see host_signal_kernel): device counter and word 0 of the pinned flags
struct HostAnnounce { uint32_t * seq; uint32_t * flags; uint32_t * words_out = nullptr; };    // words_out: a second copy of the activity words (pinned memory) for the logits-only launch

template <int CPW, int RCH, bool GATE, int G, bool HYB, int PHASE = 0>      // cols == 8 waves * CPW chunks * 512; r == RCH * 512; G groups of 32 neurons
__global__ __launch_bounds__(kPfBlock, 2) void pred_ffn_f16_kernel(const __half * __restrict__ W2, const float * __restrict__ hidden,
                                                                   const __half * __restrict__ Wup, const __half * __restrict__ Wgate,
                                                                   const __half * __restrict__ Wdown,
                                                                   const float * __restrict__ x, NormArgs na, float thr,
                                                                   float * __restrict__ logits, uint32_t * __restrict__ words, float * __restrict__ h_dense,
                                                                   float * __restrict__ partial,
                                                                   const uint32_t * __restrict__ hot_words, const int32_t * __restrict__ hot_prefix,
                                                                   uint32_t * __restrict__ words_hot, __half * __restrict__ xn_out,
                                                                   float * __restrict__ logits2, HostAnnounce ann) {
    static_assert(PHASE == 0 || G == 1, "the two-phase form takes one group per workgroup");
    if (PHASE == 2 && ann.flags && blockIdx.x == 0 && threadIdx.x == 0) {
        // what was queued before this launch is complete and visible to the host: a new hand-over starts here, without a launch of its own
        const uint32_t sq = *ann.seq + 1u;
        *ann.seq = sq;
        __hip_atomic_store(ann.flags, sq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    constexpr int cols = kPfWaves * CPW * 512, r = RCH * 512;
    constexpr int CH = kPfChunk / CPW;                 // active neurons per round trip: 3*CPW*CH (2*CPW*CH) loads in flight per lane
    __shared__ float  lg[2][32];
    __shared__ double red[2][kPfWaves];
    __shared__ float  part[kPfWaves][CH][2];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int n0 = blockIdx.x * 32 * G;
    const int cbase = wave * CPW * 512 + lane * 8;     // chunk c of this lane starts at column cbase + 512*c

    // ---- A: loads ------------------------------------------------------------------------------------------
    pi_u32x4 a[4][RCH];
    float4 hv[RCH][2];
    float logit_in = 0.0f;
    if (PHASE != 2) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < RCH; ++j) a[i][j] = pi_ld_stream(W2 + (size_t)(n0 + wave * 4 + i) * r + (j * PI_WAVE + lane) * 8);
#pragma unroll
        for (int j = 0; j < RCH; ++j) {
            hv[j][0] = *reinterpret_cast<const float4 *>(hidden + j * 512 + lane * 8);
            hv[j][1] = *reinterpret_cast<const float4 *>(hidden + j * 512 + lane * 8 + 4);
        }
    } else {
        logit_in = logits2[n0 + (lane & 31)];
    }
    float xs[CPW][8], ws[CPW][8], bs[CPW][8];
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
        const int o = cbase + c * 512;
        const float4 x0 = *reinterpret_cast<const float4 *>(x + o), x1 = *reinterpret_cast<const float4 *>(x + o + 4);
        xs[c][0] = x0.x; xs[c][1] = x0.y; xs[c][2] = x0.z; xs[c][3] = x0.w; xs[c][4] = x1.x; xs[c][5] = x1.y; xs[c][6] = x1.z; xs[c][7] = x1.w;
        if (na.kind != 0 && na.w) {
            const float4 w0 = *reinterpret_cast<const float4 *>(na.w + o), w1 = *reinterpret_cast<const float4 *>(na.w + o + 4);
            ws[c][0] = w0.x; ws[c][1] = w0.y; ws[c][2] = w0.z; ws[c][3] = w0.w; ws[c][4] = w1.x; ws[c][5] = w1.y; ws[c][6] = w1.z; ws[c][7] = w1.w;
        }
        if (na.kind != 0 && na.b) {
            const float4 b0 = *reinterpret_cast<const float4 *>(na.b + o), b1 = *reinterpret_cast<const float4 *>(na.b + o + 4);
            bs[c][0] = b0.x; bs[c][1] = b0.y; bs[c][2] = b0.z; bs[c][3] = b0.w; bs[c][4] = b1.x; bs[c][5] = b1.y; bs[c][6] = b1.z; bs[c][7] = b1.w;
        }
    }
    // ---- A: logits (the CPU path rounds the hidden vector to fp16 before the dot, ggml.c:9703-9716) ------------
    pi_u32x4 hr[RCH];
    if (PHASE != 2) {
#pragma unroll
        for (int j = 0; j < RCH; ++j) {
            __half2 hh[4] = {__floats2half2_rn(hv[j][0].x, hv[j][0].y), __floats2half2_rn(hv[j][0].z, hv[j][0].w),
                             __floats2half2_rn(hv[j][1].x, hv[j][1].y), __floats2half2_rn(hv[j][1].z, hv[j][1].w)};
            hr[j] = *reinterpret_cast<const pi_u32x4 *>(hh);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < RCH; ++j) acc = pi_dot8h(a[i][j], hr[j], acc);
            acc = pi_wave_sum(acc);
            if (lane == 0) lg[0][wave * 4 + i] = acc;
        }
    }
    if (G > 1) {       // the next group's predictor rows travel while this group's FFN rows are fetched and used
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < RCH; ++j) a[i][j] = pi_ld_stream(W2 + (size_t)(n0 + 32 + wave * 4 + i) * r + (j * PI_WAVE + lane) * 8);
    }
    // ---- A: norm statistics across the 8 slices ---------------------------------------------------------------
    float mean = 0.0f, scale = 1.0f;
    if (na.kind == 1) {
        double sq = 0.0;
#pragma unroll
        for (int c = 0; c < CPW; ++c)
#pragma unroll
            for (int k = 0; k < 8; ++k) sq += (double)__fmul_rn(xs[c][k], xs[c][k]);
        sq = pi_wave_sum_f64(sq);
        if (lane == 0) red[0][wave] = sq;
        __syncthreads();
        double t = 0.0;
#pragma unroll
        for (int w = 0; w < kPfWaves; ++w) t += red[0][w];
        scale = pi_inv_sqrt((float)(t / cols) + na.eps);
    } else if (na.kind == 2) {
        double sm = 0.0;
#pragma unroll
        for (int c = 0; c < CPW; ++c)
#pragma unroll
            for (int k = 0; k < 8; ++k) sm += (double)xs[c][k];
        sm = pi_wave_sum_f64(sm);
        if (lane == 0) red[0][wave] = sm;
        __syncthreads();
        double t = 0.0;
#pragma unroll
        for (int w = 0; w < kPfWaves; ++w) t += red[0][w];
        mean = (float)(t / cols);
        double sq = 0.0;
#pragma unroll
        for (int c = 0; c < CPW; ++c)
#pragma unroll
            for (int k = 0; k < 8; ++k) { const float v = __fsub_rn(xs[c][k], mean); sq += (double)__fmul_rn(v, v); }
        sq = pi_wave_sum_f64(sq);
        if (lane == 0) red[1][wave] = sq;
        __syncthreads();
        double t2 = 0.0;
#pragma unroll
        for (int w = 0; w < kPfWaves; ++w) t2 += red[1][w];
        scale = pi_inv_sqrt((float)(t2 / cols) + na.eps);
    } else {
        __syncthreads();
    }
    pi_u32x4 xr[CPW];
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            float v = xs[c][k];
            if (na.kind != 0) {
                v = __fmul_rn(na.kind == 2 ? __fsub_rn(v, mean) : v, scale);
                if (na.w) v = __fmul_rn(v, ws[c][k]);
                if (na.b) v = __fadd_rn(v, bs[c][k]);
            }
            xs[c][k] = v;
        }
        __half2 hh[4] = {__floats2half2_rn(xs[c][0], xs[c][1]), __floats2half2_rn(xs[c][2], xs[c][3]),
                         __floats2half2_rn(xs[c][4], xs[c][5]), __floats2half2_rn(xs[c][6], xs[c][7])};
        xr[c] = *reinterpret_cast<const pi_u32x4 *>(hh);
        if (HYB && blockIdx.x == 0 && xn_out) *reinterpret_cast<pi_u32x4 *>(xn_out + cbase + c * 512) = xr[c];
    }
    float acc[CPW][8];
#pragma unroll
    for (int c = 0; c < CPW; ++c)
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[c][k] = 0.0f;
#pragma unroll 1
    for (int g = 0; g < G; ++g, n0 += 32) {
    if (g > 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float lacc = 0.0f;
#pragma unroll
            for (int j = 0; j < RCH; ++j) lacc = pi_dot8h(a[i][j], hr[j], lacc);
            lacc = pi_wave_sum(lacc);
            if (lane == 0) lg[g & 1][wave * 4 + i] = lacc;
        }
        if (g + 1 < G) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < RCH; ++j) a[i][j] = pi_ld_stream(W2 + (size_t)(n0 + 32 + wave * 4 + i) * r + (j * PI_WAVE + lane) * 8);
        }
        __syncthreads();
    }
    // ---- activity word (identical in every wave; lg[g & 1] is complete after the barrier above) ----------------
    const float my_logit = PHASE == 2 ? logit_in : lg[g & 1][lane & 31];
    const bool my_act = !(my_logit < thr);
    const uint32_t all = (uint32_t)__ballot(my_act);
    const uint32_t hot = HYB ? hot_words[blockIdx.x * G + g] : 0xFFFFFFFFu;
    const int base_row = HYB ? hot_prefix[blockIdx.x * G + g] : n0;
    const uint32_t mask = all & hot;
    if (wave == 0) {
        if (lane < 32) {
            if (PHASE != 2 && logits) logits[n0 + lane] = my_logit;
            if (PHASE == 1) logits2[n0 + lane] = my_logit;
            if (PHASE != 1 && h_dense && !((mask >> lane) & 1u)) h_dense[n0 + lane] = 0.0f;
        }
        if (lane == 0) { words[blockIdx.x * G + g] = all; if (HYB) words_hot[blockIdx.x * G + g] = mask; if (PHASE == 1 && ann.words_out) ann.words_out[blockIdx.x * G + g] = all; }
    }
    if (PHASE == 1) return;
    // ---- B + C ---------------------------------------------------------------------------------------------
    const int n = __popc(mask);
    for (int c0 = 0; c0 < n; c0 += CH) {
        const int nn = n - c0 < CH ? n - c0 : CH;
        int rows[CH];
        pi_u32x4 gu[CH][CPW], uu[CH][CPW], dd[CH][CPW];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (j < nn) {
                const int bit = select_nth_bit(mask, c0 + j);
                rows[j] = n0 + bit;
                const size_t off = (size_t)(HYB ? base_row + __popc(hot & ((1u << bit) - 1u)) : rows[j]) * cols + cbase;
#pragma unroll
                for (int c = 0; c < CPW; ++c) {
                    uu[j][c] = pi_ld_stream(Wup + off + c * 512);
                    if (GATE) gu[j][c] = pi_ld_stream(Wgate + off + c * 512);
                    dd[j][c] = pi_ld_stream(Wdown + off + c * 512);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (j < nn) {
                float pu = 0.0f, pg = 0.0f;
#pragma unroll
                for (int c = 0; c < CPW; ++c) { pu = pi_dot8h(uu[j][c], xr[c], pu); if (GATE) pg = pi_dot8h(gu[j][c], xr[c], pg); }
                pu = pi_wave_sum(pu);
                if (GATE) pg = pi_wave_sum(pg);
                if (lane == 0) { part[wave][j][0] = pu; part[wave][j][1] = pg; }
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (j < nn) {
                float u = 0.0f, g = 0.0f;
#pragma unroll
                for (int w = 0; w < kPfWaves; ++w) { u += part[w][j][0]; if (GATE) g += part[w][j][1]; }
                const float h = GATE ? __fmul_rn(fmaxf(g, 0.0f), u) : fmaxf(u, 0.0f);
                if (h_dense && threadIdx.x == 0) h_dense[rows[j]] = h;
                const float hq = pi_round_f16(h);                 // the CPU axpy rounds h to fp16 (ggml.c:14420-14431)
#pragma unroll
                for (int c = 0; c < CPW; ++c) {
                    float wf[8];
                    pi_unpack8(dd[j][c], wf);
#pragma unroll
                    for (int k = 0; k < 8; ++k) acc[c][k] = fmaf(wf[k], hq, acc[c][k]);
                }
            }
        }
        if (c0 + CH < n) __syncthreads();                         // part[] is reused by the next chunk
    }
    }   // groups: the barrier behind the next group's logits also orders this group's last reads of part[] and lg[]
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
        float4 * po = reinterpret_cast<float4 *>(partial + (size_t)blockIdx.x * cols + cbase + c * 512);
        po[0] = make_float4(acc[c][0], acc[c][1], acc[c][2], acc[c][3]);
        po[1] = make_float4(acc[c][4], acc[c][5], acc[c][6], acc[c][7]);
    }
}

// ---------------------------------------------------------------------------------------------------
// The same block with the neurons spread evenly over the compute units (F16, cols == 4096, every neuron on the device).
// What bounds a launch of this kind is the compute unit that has to pull the most bytes: a unit sustains about 1/256 of the
// chip's HBM rate whatever it has in flight, so with ff / 32 workgroups of 32 neurons (344 on 256 units at ff 11008) the 88
// units that hold two workgroups set the pace and the others idle.  Here the grid is one workgroup per unit and workgroup b
// owns neurons [ff * b / n, ff * (b + 1) / n): up to 64 of them, so that one 64-lane ballot yields the activity mask.
//   A  wave w computes the predictor logits of neurons w, w + 8, ... of the range (fc2 rows, r == 512 * RCH) and loads its
//      eighth of the FFN input and norm weights; statistics and logits cross the waves through LDS.
//   B  every wave derives the same 64-bit mask and loads ITS 512-column slice of the gate, up and down rows of up to
//      kCuChunk active neurons at once; partial gate / up dots cross the waves through LDS; h = relu(g) * u.
//   C  partial[b][512 w + 8 lane ..] += fp16(h) * down slice; one store per workgroup; ffn_reduce_kernel adds the n vectors.
// A workgroup may use the whole register file of its unit (one workgroup per unit), which is what lets twelve active
// neurons travel at once.  Logits and sums are those of pred_ffn_f16_kernel for the same rows.
// What is left on the table is the spread of the active neurons over the ranges: 1107 active of 11008 are 4.3 per workgroup on
// average and up to 12, and the launch takes 16.2 us against 13.2 us for the same number spread evenly (5 at most).  Dealing them out
// evenly needs every range's mask first, i.e. a launch boundary: the predictor part as a launch of its own (6.1 us) followed by the
// rows of the active neurons in equal shares, each workgroup deriving its share from all the mask words (12.6 us), was slower.
// ---------------------------------------------------------------------------------------------------
constexpr int kCuChunk = 12;

__device__ __forceinline__ int select_nth_bit64(uint64_t bits, int n) {      // index of the n-th (0-based) set bit
    for (int i = 0; i < n; ++i) bits &= bits - 1;
    return __ffsll((unsigned long long)bits) - 1;
}

// KIND: 0 no norm, 1 RMSNorm * w, 2 LayerNorm * w + b (the launcher checks that the operands are there).  Every load of phase A is
// unconditional - a wave without an ROWS-th row of its own requests the range's last row again, which its unit already has on the way -
// because the compiler counts outstanding loads conservatively across branches and would otherwise hold the norm statistics back
// until the last predictor row has landed.
// NW waves of 512 columns each (8: 4096 columns, 10: 5120); R = predictor rank, a multiple of 256 (a last half chunk of 512 is read by
// half the lanes, the others re-read the row's start against a zero of the hidden vector).  Ten waves are three on two of the four
// SIMDs, which leaves each 168 registers: eight active neurons travel at once instead of twelve.
template <int NW, int R, bool GATE, int ROWS, int KIND>      // ROWS fc2 rows per wave: at most NW * ROWS neurons per workgroup
__global__ __launch_bounds__(NW * 64, 1) void ffn_cu_f16_kernel(const __half * __restrict__ W2, const float * __restrict__ hidden,
                                                                 const __half * __restrict__ Wup, const __half * __restrict__ Wgate,
                                                                 const __half * __restrict__ Wdown,
                                                                 const float * __restrict__ x, const float * __restrict__ nw, const float * __restrict__ nb, float eps,
                                                                 float thr, int ff,
                                                                 float * __restrict__ logits, uint32_t * __restrict__ words, float * __restrict__ h_dense,
                                                                 float * __restrict__ partial) {
    constexpr int cols = NW * 512, r = R, RCH = (R + 511) / 512, CH = NW == 8 ? kCuChunk : 8;
    static_assert(R % 256 == 0 && NW * ROWS <= 64 + NW - 1, "rank in half chunks; one 64-bit mask per workgroup");
    __shared__ float  lg[64];
    __shared__ double red[2][NW];
    __shared__ float  part[NW][CH][2];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n0 = (int)((long long)ff * blockIdx.x / gridDim.x);
    const int np = (int)((long long)ff * (blockIdx.x + 1) / gridDim.x) - n0;       // <= NW * ROWS and <= 64 (the launcher's test)
    const int cbase = wave * 512 + lane * 8;

    // ---- A: loads.  Memory returns a wave's loads in the order it issued them: the small operands go first, so that the norm
    // statistics, their exchange and the division run while the predictor rows are still on their way, and only the dot products
    // and one barrier lie between the last predictor row and the first gate / up / down request. ------------------------------
    float xs[8], ws[8], bs[8];
    {
        const float4 x0 = *reinterpret_cast<const float4 *>(x + cbase), x1 = *reinterpret_cast<const float4 *>(x + cbase + 4);
        xs[0] = x0.x; xs[1] = x0.y; xs[2] = x0.z; xs[3] = x0.w; xs[4] = x1.x; xs[5] = x1.y; xs[6] = x1.z; xs[7] = x1.w;
        if (KIND >= 1) {
            const float4 w0 = *reinterpret_cast<const float4 *>(nw + cbase), w1 = *reinterpret_cast<const float4 *>(nw + cbase + 4);
            ws[0] = w0.x; ws[1] = w0.y; ws[2] = w0.z; ws[3] = w0.w; ws[4] = w1.x; ws[5] = w1.y; ws[6] = w1.z; ws[7] = w1.w;
        }
        if (KIND == 2) {
            const float4 b0 = *reinterpret_cast<const float4 *>(nb + cbase), b1 = *reinterpret_cast<const float4 *>(nb + cbase + 4);
            bs[0] = b0.x; bs[1] = b0.y; bs[2] = b0.z; bs[3] = b0.w; bs[4] = b1.x; bs[5] = b1.y; bs[6] = b1.z; bs[7] = b1.w;
        }
    }
    float4 hv[RCH][2];
    int roff[RCH];
#pragma unroll
    for (int j = 0; j < RCH; ++j) {
        const bool in = (j + 1) * 512 <= R || (j * PI_WAVE + lane) * 8 < R;          // the last chunk may be half a chunk
        roff[j] = in ? (j * PI_WAVE + lane) * 8 : 0;
        hv[j][0] = *reinterpret_cast<const float4 *>(hidden + roff[j]);
        hv[j][1] = *reinterpret_cast<const float4 *>(hidden + roff[j] + 4);
        if (!in) hv[j][0] = hv[j][1] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    pi_u32x4 a[ROWS][RCH];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const int row = wave + NW * i < np ? wave + NW * i : np - 1;
#pragma unroll
        for (int j = 0; j < RCH; ++j) a[i][j] = pi_ld_stream(W2 + (size_t)(n0 + row) * r + roff[j]);
    }
    // ---- A: norm statistics across the NW slices ---------------------------------------------------------------
    float mean = 0.0f, scale = 1.0f;
    if (KIND == 1) {
        double sq = 0.0;
#pragma unroll
        for (int k = 0; k < 8; ++k) sq += (double)__fmul_rn(xs[k], xs[k]);
        sq = pi_wave_sum_f64(sq);
        if (lane == 0) red[0][wave] = sq;
        __syncthreads();
        double t = 0.0;
#pragma unroll
        for (int w = 0; w < NW; ++w) t += red[0][w];
        scale = pi_inv_sqrt((float)(t / cols) + eps);
    } else if (KIND == 2) {
        double sm = 0.0;
#pragma unroll
        for (int k = 0; k < 8; ++k) sm += (double)xs[k];
        sm = pi_wave_sum_f64(sm);
        if (lane == 0) red[0][wave] = sm;
        __syncthreads();
        double t = 0.0;
#pragma unroll
        for (int w = 0; w < NW; ++w) t += red[0][w];
        mean = (float)(t / cols);
        double sq = 0.0;
#pragma unroll
        for (int k = 0; k < 8; ++k) { const float v = __fsub_rn(xs[k], mean); sq += (double)__fmul_rn(v, v); }
        sq = pi_wave_sum_f64(sq);
        if (lane == 0) red[1][wave] = sq;
        __syncthreads();
        double t2 = 0.0;
#pragma unroll
        for (int w = 0; w < NW; ++w) t2 += red[1][w];
        scale = pi_inv_sqrt((float)(t2 / cols) + eps);
    }
    pi_u32x4 xr;
    {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            float v = xs[k];
            if (KIND >= 1) v = __fmul_rn(__fmul_rn(KIND == 2 ? __fsub_rn(v, mean) : v, scale), ws[k]);
            if (KIND == 2) v = __fadd_rn(v, bs[k]);
            xs[k] = v;
        }
        __half2 hh[4] = {__floats2half2_rn(xs[0], xs[1]), __floats2half2_rn(xs[2], xs[3]),
                         __floats2half2_rn(xs[4], xs[5]), __floats2half2_rn(xs[6], xs[7])};
        xr = *reinterpret_cast<const pi_u32x4 *>(hh);
    }
    // ---- A: logits (the CPU path rounds the hidden vector to fp16 before the dot, ggml.c:9703-9716) ------------
    {
        pi_u32x4 hr[RCH];
#pragma unroll
        for (int j = 0; j < RCH; ++j) {
            __half2 hh[4] = {__floats2half2_rn(hv[j][0].x, hv[j][0].y), __floats2half2_rn(hv[j][0].z, hv[j][0].w),
                             __floats2half2_rn(hv[j][1].x, hv[j][1].y), __floats2half2_rn(hv[j][1].z, hv[j][1].w)};
            hr[j] = *reinterpret_cast<const pi_u32x4 *>(hh);
        }
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < RCH; ++j) acc = pi_dot8h(a[i][j], hr[j], acc);
            acc = pi_wave_sum(acc);
            if (lane == 0 && wave + NW * i < np) lg[wave + NW * i] = acc;
        }
    }
    __syncthreads();
    // ---- activity mask (identical in every wave; lg[] is complete after the barrier above) -----------------------
    const float my_logit = lane < np ? lg[lane] : 0.0f;
    const bool my_act = lane < np && !(my_logit < thr);
    const uint64_t mask = (uint64_t)__ballot(my_act);
    if (wave == 0) {
        if (lane < np) {
            if (logits) logits[n0 + lane] = my_logit;
            if (h_dense && !my_act) h_dense[n0 + lane] = 0.0f;
        }
        if (lane == 0) { words[2 * blockIdx.x] = (uint32_t)mask; words[2 * blockIdx.x + 1] = (uint32_t)(mask >> 32); }
    }
    // ---- B + C ---------------------------------------------------------------------------------------------
    float acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = 0.0f;
    const int n = __popcll((unsigned long long)mask);
    for (int c0 = 0; c0 < n; c0 += CH) {
        const int nn = n - c0 < CH ? n - c0 : CH;
        int rows[CH];
        pi_u32x4 gu[CH], uu[CH], dd[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (j < nn) {
                rows[j] = n0 + select_nth_bit64(mask, c0 + j);
                const size_t off = (size_t)rows[j] * cols + cbase;
                uu[j] = pi_ld_stream(Wup + off);
                if (GATE) gu[j] = pi_ld_stream(Wgate + off);
                dd[j] = pi_ld_stream(Wdown + off);
            }
        }
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (j < nn) {
                float pu = pi_dot8h(uu[j], xr, 0.0f), pg = 0.0f;
                if (GATE) pg = pi_dot8h(gu[j], xr, 0.0f);
                pu = pi_wave_sum(pu);
                if (GATE) pg = pi_wave_sum(pg);
                if (lane == 0) { part[wave][j][0] = pu; part[wave][j][1] = pg; }
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (j < nn) {
                float u = 0.0f, g = 0.0f;
#pragma unroll
                for (int w = 0; w < NW; ++w) { u += part[w][j][0]; if (GATE) g += part[w][j][1]; }
                const float h = GATE ? __fmul_rn(fmaxf(g, 0.0f), u) : fmaxf(u, 0.0f);
                if (h_dense && threadIdx.x == 0) h_dense[rows[j]] = h;
                const float hq = pi_round_f16(h);                 // the CPU axpy rounds h to fp16 (ggml.c:14420-14431)
                float wf[8];
                pi_unpack8(dd[j], wf);
#pragma unroll
                for (int k = 0; k < 8; ++k) acc[k] = fmaf(wf[k], hq, acc[k]);
            }
        }
        if (c0 + CH < n) __syncthreads();                         // part[] is reused by the next chunk
    }
    float4 * po = reinterpret_cast<float4 *>(partial + (size_t)blockIdx.x * cols + cbase);
    po[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    po[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
}

// out[c] = epi( sum over workgroups b (within a fixed tree) of partial[b][c] ).  A workgroup of 8 waves owns kFrCols = 32
// columns, one 128-byte line of every partial vector: 8 lanes x float4 cover them, the eight 8-lane groups of a wave and the
// 8 waves split the rows of the partial matrix (64 rows per pass, all of a thread's rows requested at once); groups merge by
// shuffles, waves through LDS in wave order.  cols / 32 workgroups: a compute unit sustains only about 1/256 of the chip's
// HBM rate, so the partial matrix has to be spread over as many units as 128-byte lines allow.  Workgroup 0 also counts the
// predictor's active neurons from the mask words.
constexpr int kFrUn = 6, kFrCols = 32;
__global__ __launch_bounds__(kPfBlock) void ffn_reduce_kernel(const float * __restrict__ partial, int n_part, int cols,
                                                              const uint32_t * __restrict__ words, int n_words, int32_t * __restrict__ n_active_out,
                                                              int epi, const float * __restrict__ add1, const float * __restrict__ add2, float * __restrict__ out) {
    __shared__ float redl[kPfWaves][kFrCols];
    __shared__ int   sred[kPfWaves];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int sub = lane >> 3, col = blockIdx.x * kFrCols + (lane & 7) * 4;
    // the residual operands and the mask words do not depend on anything computed here: fetch them first
    float r1 = 0.0f, r2 = 0.0f;
    if (tid < kFrCols) {
        if (epi >= PI_EPI_ADD) r1 = add1[blockIdx.x * kFrCols + tid];
        if (epi == PI_EPI_ADD2) r2 = add2[blockIdx.x * kFrCols + tid];
    }
    int cnt = 0;
    if (blockIdx.x == 0 && n_active_out)
        for (int w = tid; w < n_words; w += kPfBlock) cnt += __popc(words[w]);
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (int b0 = wave * 8 + sub; b0 < n_part; b0 += kPfWaves * 8 * kFrUn) {
        float4 v[kFrUn];
#pragma unroll
        for (int u = 0; u < kFrUn; ++u) {
            const int b = b0 + u * kPfWaves * 8;
            v[u] = b < n_part ? *reinterpret_cast<const float4 *>(partial + (size_t)b * cols + col) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
#pragma unroll
        for (int u = 0; u < kFrUn; ++u) { acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w; }
    }
#pragma unroll
    for (int o = 8; o < 64; o <<= 1) {
        acc.x += __shfl_xor(acc.x, o, PI_WAVE); acc.y += __shfl_xor(acc.y, o, PI_WAVE); acc.z += __shfl_xor(acc.z, o, PI_WAVE); acc.w += __shfl_xor(acc.w, o, PI_WAVE);
    }
    if (lane < 8) { redl[wave][lane * 4] = acc.x; redl[wave][lane * 4 + 1] = acc.y; redl[wave][lane * 4 + 2] = acc.z; redl[wave][lane * 4 + 3] = acc.w; }
    if (blockIdx.x == 0 && n_active_out) { cnt = pi_wave_sum_i32(cnt); if (lane == 0) sred[wave] = cnt; }
    __syncthreads();
    if (tid < kFrCols) {
        float sum = redl[0][tid];
#pragma unroll
        for (int w = 1; w < kPfWaves; ++w) sum += redl[w][tid];
        if (epi == PI_EPI_ADD) sum = __fadd_rn(sum, r1);
        else if (epi == PI_EPI_ADD2) sum = __fadd_rn(__fadd_rn(sum, r1), r2);
        out[blockIdx.x * kFrCols + tid] = sum;
    }
    if (blockIdx.x == 0 && n_active_out && tid == 0) { int t = 0; for (int w = 0; w < kPfWaves; ++w) t += sred[w]; *n_active_out = t; }
}

// ---------------------------------------------------------------------------------------------------
// Q4_0 weights (cols == 4096): the predictor's second layer, the mask and the up/gate rows of the GPU-resident
// neurons in one launch, in the layout of pred_ffn_f16_kernel: a workgroup of 8 waves owns 32 neurons, wave w owns
// columns [512w, 512w + 512), lane l eight of them, i.e. a quarter of one 32-weight block (sub = l & 3: low nibbles of
// qs[0..7], of qs[8..15], then the high nibbles of the same bytes).
//   A  four fc2 rows per wave; the wave's slice of the FFN input is normalised and quantised to Q8_0 in registers:
//      the four lanes of a block agree on amax by two quad permutations, d = amax/127 kept as fp16, q = rint(x*127/amax)
//      (x86 path of quantize_row_q8_0, ggml-quants.c:702-760).  Workgroup 0 also stores the Q8_0 blocks ({fp16 d, 32 x int8},
//      34 bytes each) for a host that computes the other neurons from the same quantised input.
//   B  active neurons that live on the GPU (mask & hot word): row = hot_prefix + rank among the hot bits; every wave loads
//      its 8 bytes + scale of up to 8 up and gate rows at once; exact int32 block sums (two more quad permutations)
//      times d_w * d_x (vec_dot_q4_0_q8_0, ggml-quants.c:2512-2650), summed per wave and across waves through LDS.
// h_dense gets h for those neurons and 0 for every other neuron of the group; the pointers handed in for logits,
// h_dense and the Q8_0 blocks may be pinned host memory (a hybrid layer's host share reads them after the launch).
// ---------------------------------------------------------------------------------------------------
struct __attribute__((packed)) pi_q8_host_block { uint16_t d; int8_t qs[32]; };
constexpr int kAqChunkFused = 8;           // down rows in flight per wave in the fused form

// SPLIT: the neurons outside the hot words are computed here too, from a second pair of matrices that holds exactly those
// neurons' rows in ascending order (rows in pinned host memory, fetched over the host link by the loads below).
// PHASE 1 / 2 cut the launch in two for a hybrid layer whose host share should start as early as possible: 1 stops behind the
// logits (to `logits` and `logits2`), the mask words and the Q8_0 blocks of the input; 2 reads the logits back from `logits2`
// instead of computing them, and writes h only for the neurons of the hot words (h or 0): the other entries of that vector
// belong to the host.
// FUSE: the workgroup's 32 neurons are exactly one Q8_0 block of h, so when every active neuron is computed here (all of them resident,
// or SPLIT) the launch goes on with the down projection: h of the group is quantised as the CPU path quantises the dense vector
// (ggml.c:14465-14618), and each wave adds its 512-column slice of the down rows of the neurons with a non-zero quant, in ascending
// order and with axpy_q4_groups_kernel's arithmetic; the workgroup's partial output vector goes to `partial` for ffn_reduce_kernel.
template <int RCH, bool GATE, bool SPLIT, int PHASE = 0, bool FUSE = false>
__global__ __launch_bounds__(kPfBlock, 2) void pred_upgate_q4_kernel(const __half * __restrict__ W2, const float * __restrict__ hidden,
                                                                     const pi_block_q4_0 * __restrict__ Wup, const pi_block_q4_0 * __restrict__ Wgate,
                                                                     const pi_block_q4_0 * __restrict__ Wup_rest, const pi_block_q4_0 * __restrict__ Wgate_rest,
                                                                     const float * __restrict__ x, NormArgs na, float thr,
                                                                     const uint32_t * __restrict__ hot_words, const int32_t * __restrict__ hot_prefix,
                                                                     float * __restrict__ logits, uint32_t * __restrict__ words, uint32_t * __restrict__ words_hot,
                                                                     float * __restrict__ h_dense, pi_q8_host_block * __restrict__ xq_out,
                                                                     float * __restrict__ logits2,
                                                                     const pi_block_q4_0 * __restrict__ Wd, const pi_block_q4_0 * __restrict__ Wd_rest,
                                                                     float * __restrict__ partial, HostAnnounce ann) {
    static_assert(!FUSE || PHASE == 0, "the two-phase form of a hybrid layer leaves the down projection to its own launch");
    if (PHASE == 2 && ann.flags && blockIdx.x == 0 && threadIdx.x == 0) {
        // what was queued before this launch is complete and visible to the host (the kernel boundary released at system scope):
        // a new hand-over starts here, without a launch of its own
        const uint32_t sq = *ann.seq + 1u;
        *ann.seq = sq;
        __hip_atomic_store(ann.flags, sq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    constexpr int cols = 4096, r = RCH * 512, nb = cols / 32, CH = kPfChunk;
    __shared__ float  hs[32];
    __shared__ float  lg[32];
    __shared__ double red[2][kPfWaves];
    __shared__ float  part[kPfWaves][CH][2];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n0 = blockIdx.x * 32;
    const int cbase = wave * 512 + lane * 8;
    const int blk = cbase >> 5, sub = lane & 3;

    // ---- A: loads ------------------------------------------------------------------------------------------
    pi_u32x4 a[4][RCH];
    float4 hv[RCH][2];
    float logit_in = 0.0f;
    if (PHASE != 2) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < RCH; ++j) a[i][j] = pi_ld_stream(W2 + (size_t)(n0 + wave * 4 + i) * r + (j * PI_WAVE + lane) * 8);
#pragma unroll
        for (int j = 0; j < RCH; ++j) {
            hv[j][0] = *reinterpret_cast<const float4 *>(hidden + j * 512 + lane * 8);
            hv[j][1] = *reinterpret_cast<const float4 *>(hidden + j * 512 + lane * 8 + 4);
        }
    } else {
        logit_in = logits2[n0 + (lane & 31)];
    }
    const uint32_t hot = hot_words ? hot_words[blockIdx.x] : 0xFFFFFFFFu;
    const int base_row = hot_prefix ? hot_prefix[blockIdx.x] : n0;
    float xs[8], wn[8], bn[8];
    {
        const float4 x0 = *reinterpret_cast<const float4 *>(x + cbase), x1 = *reinterpret_cast<const float4 *>(x + cbase + 4);
        xs[0] = x0.x; xs[1] = x0.y; xs[2] = x0.z; xs[3] = x0.w; xs[4] = x1.x; xs[5] = x1.y; xs[6] = x1.z; xs[7] = x1.w;
        if (na.kind != 0 && na.w) {
            const float4 w0 = *reinterpret_cast<const float4 *>(na.w + cbase), w1 = *reinterpret_cast<const float4 *>(na.w + cbase + 4);
            wn[0] = w0.x; wn[1] = w0.y; wn[2] = w0.z; wn[3] = w0.w; wn[4] = w1.x; wn[5] = w1.y; wn[6] = w1.z; wn[7] = w1.w;
        }
        if (na.kind != 0 && na.b) {
            const float4 b0 = *reinterpret_cast<const float4 *>(na.b + cbase), b1 = *reinterpret_cast<const float4 *>(na.b + cbase + 4);
            bn[0] = b0.x; bn[1] = b0.y; bn[2] = b0.z; bn[3] = b0.w; bn[4] = b1.x; bn[5] = b1.y; bn[6] = b1.z; bn[7] = b1.w;
        }
    }
    // ---- A: logits (the CPU path rounds the hidden vector to fp16 before the dot, ggml.c:9703-9716) ------------
    if (PHASE != 2) {
        pi_u32x4 hr[RCH];
#pragma unroll
        for (int j = 0; j < RCH; ++j) {
            __half2 hh[4] = {__floats2half2_rn(hv[j][0].x, hv[j][0].y), __floats2half2_rn(hv[j][0].z, hv[j][0].w),
                             __floats2half2_rn(hv[j][1].x, hv[j][1].y), __floats2half2_rn(hv[j][1].z, hv[j][1].w)};
            hr[j] = *reinterpret_cast<const pi_u32x4 *>(hh);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < RCH; ++j) acc = pi_dot8h(a[i][j], hr[j], acc);
            acc = pi_wave_sum(acc);
            if (lane == 0) lg[wave * 4 + i] = acc;
        }
    }
    // ---- A: norm statistics across the 8 slices ---------------------------------------------------------------
    float mean = 0.0f, scale = 1.0f;
    if (na.kind == 1) {
        double sq = 0.0;
#pragma unroll
        for (int k = 0; k < 8; ++k) sq += (double)__fmul_rn(xs[k], xs[k]);
        sq = pi_wave_sum_f64(sq);
        if (lane == 0) red[0][wave] = sq;
        __syncthreads();
        double t = 0.0;
#pragma unroll
        for (int w = 0; w < kPfWaves; ++w) t += red[0][w];
        scale = pi_inv_sqrt((float)(t / cols) + na.eps);
    } else if (na.kind == 2) {
        double sm = 0.0;
#pragma unroll
        for (int k = 0; k < 8; ++k) sm += (double)xs[k];
        sm = pi_wave_sum_f64(sm);
        if (lane == 0) red[0][wave] = sm;
        __syncthreads();
        double t = 0.0;
#pragma unroll
        for (int w = 0; w < kPfWaves; ++w) t += red[0][w];
        mean = (float)(t / cols);
        double sq = 0.0;
#pragma unroll
        for (int k = 0; k < 8; ++k) { const float v = __fsub_rn(xs[k], mean); sq += (double)__fmul_rn(v, v); }
        sq = pi_wave_sum_f64(sq);
        if (lane == 0) red[1][wave] = sq;
        __syncthreads();
        double t2 = 0.0;
#pragma unroll
        for (int w = 0; w < kPfWaves; ++w) t2 += red[1][w];
        scale = pi_inv_sqrt((float)(t2 / cols) + na.eps);
    } else {
        __syncthreads();
    }
    // ---- A: Q8_0 of the normalised slice -----------------------------------------------------------------------
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        float v = xs[k];
        if (na.kind != 0) {
            v = __fmul_rn(na.kind == 2 ? __fsub_rn(v, mean) : v, scale);
            if (na.w) v = __fmul_rn(v, wn[k]);
            if (na.b) v = __fadd_rn(v, bn[k]);
        }
        xs[k] = v;
        amax = fmaxf(amax, fabsf(v));
    }
    amax = fmaxf(amax, pi_dpp_f32<PI_DPP_XOR1, 0xF>(amax));
    amax = fmaxf(amax, pi_dpp_f32<PI_DPP_XOR2, 0xF>(amax));
    const float dq = pi_div(amax, 127.0f), idq = (amax != 0.0f) ? pi_div(127.0f, amax) : 0.0f;
    const float dx = pi_round_f16(dq);
    int xq0 = 0, xq1 = 0, sx = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int q = (int)rintf(__fmul_rn(xs[k], idq));
        sx += q;
        if (k < 4) xq0 |= (q & 0xFF) << (8 * k); else xq1 |= (q & 0xFF) << (8 * (k - 4));
    }
    if (blockIdx.x == 0 && xq_out) {
        pi_q8_host_block * ob = xq_out + blk;
        const int q2[2] = {xq0, xq1};
        __builtin_memcpy(ob->qs + sub * 8, q2, 8);
        if (sub == 0) { const uint16_t db = pi_f16_bits(dq); __builtin_memcpy(&ob->d, &db, 2); }
    }
    // ---- activity word (identical in every wave; lg is complete after the barrier above) -----------------------
    const float my_logit = PHASE == 2 ? logit_in : lg[lane & 31];
    const bool my_act = !(my_logit < thr);
    const uint32_t mask = (uint32_t)__ballot(my_act);
    const uint32_t sel = SPLIT ? mask : mask & hot;
    if (wave == 0) {
        if (lane < 32) {
            if (PHASE != 2 && logits) logits[n0 + lane] = my_logit;
            if (PHASE == 1) logits2[n0 + lane] = my_logit;
            if (PHASE == 0 && !((sel >> lane) & 1u)) h_dense[n0 + lane] = 0.0f;
            if (PHASE == 2 && ((hot >> lane) & 1u) && !((sel >> lane) & 1u)) h_dense[n0 + lane] = 0.0f;
            if (FUSE) hs[lane] = 0.0f;             // ordered before the h values below by the barrier inside the first chunk
        }
        if (lane == 0) { words[blockIdx.x] = mask; if (words_hot) words_hot[blockIdx.x] = sel; }
    }
    if (PHASE == 1) return;
    // ---- B -------------------------------------------------------------------------------------------------
    const int n = __popc(sel);
    const int shift = (sub >> 1) * 4, qoff = (sub & 1) * 8;
    for (int c0 = 0; c0 < n; c0 += CH) {
        const int nn = n - c0 < CH ? n - c0 : CH;
        int nrn[CH];
        uint32_t qu[CH][2], qg[CH][2];
        uint16_t du[CH], dg[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (j < nn) {
                const int bit = select_nth_bit(sel, c0 + j);
                nrn[j] = n0 + bit;
                const int below = __popc(hot & ((1u << bit) - 1u));
                const bool rest = SPLIT && !((hot >> bit) & 1u);      // n0 - base_row neurons outside the hot set lie before this group
                const size_t row = rest ? (size_t)(n0 - base_row + bit - below) : (size_t)(base_row + below);
                const pi_block_q4_0 * wu = (rest ? Wup_rest : Wup) + row * nb + blk;
                __builtin_memcpy(&du[j], &wu->d, 2);
                __builtin_memcpy(qu[j], wu->qs + qoff, 8);
                if (GATE) {
                    const pi_block_q4_0 * wg = (rest ? Wgate_rest : Wgate) + row * nb + blk;
                    __builtin_memcpy(&dg[j], &wg->d, 2);
                    __builtin_memcpy(qg[j], wg->qs + qoff, 8);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (j < nn) {
                int su = __builtin_amdgcn_sdot4((int)((qu[j][0] >> shift) & 0x0F0F0F0Fu), xq0, 0, false);
                su = __builtin_amdgcn_sdot4((int)((qu[j][1] >> shift) & 0x0F0F0F0Fu), xq1, su, false) - 8 * sx;
                su += pi_dpp_i32<PI_DPP_XOR1, 0xF>(su);
                su += pi_dpp_i32<PI_DPP_XOR2, 0xF>(su);
                float pu = sub == 0 ? __fmul_rn(__fmul_rn(pi_f16_from_bits(du[j]), dx), (float)su) : 0.0f, pg = 0.0f;
                if (GATE) {
                    int sg = __builtin_amdgcn_sdot4((int)((qg[j][0] >> shift) & 0x0F0F0F0Fu), xq0, 0, false);
                    sg = __builtin_amdgcn_sdot4((int)((qg[j][1] >> shift) & 0x0F0F0F0Fu), xq1, sg, false) - 8 * sx;
                    sg += pi_dpp_i32<PI_DPP_XOR1, 0xF>(sg);
                    sg += pi_dpp_i32<PI_DPP_XOR2, 0xF>(sg);
                    pg = sub == 0 ? __fmul_rn(__fmul_rn(pi_f16_from_bits(dg[j]), dx), (float)sg) : 0.0f;
                    pg = pi_wave_sum(pg);
                }
                pu = pi_wave_sum(pu);
                if (lane == 0) { part[wave][j][0] = pu; part[wave][j][1] = pg; }
            }
        }
        __syncthreads();
        if (threadIdx.x < CH && (int)threadIdx.x < nn) {
            const int j = threadIdx.x;
            float u = 0.0f, g = 0.0f;
#pragma unroll
            for (int w = 0; w < kPfWaves; ++w) { u += part[w][j][0]; if (GATE) g += part[w][j][1]; }
            int nj = 0;
#pragma unroll
            for (int jj = 0; jj < CH; ++jj) if (jj == j) nj = nrn[jj];
            const float hval = GATE ? __fmul_rn(fmaxf(g, 0.0f), u) : fmaxf(u, 0.0f);
            h_dense[nj] = hval;
            if (FUSE) hs[nj - n0] = hval;
        }
        if (c0 + CH < n) __syncthreads();                         // part[] is reused by the next chunk
    }
    if (FUSE) {
        // ---- C: Q8_0 of the group's h, then the down rows ------------------------------------------------------------
        __syncthreads();
        const float hvv = hs[lane & 31];
        float hmax = fabsf(hvv);
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) hmax = fmaxf(hmax, __shfl_xor(hmax, o, PI_WAVE));
        const float dh = pi_round_f16(pi_div(hmax, 127.0f)), idh = (hmax != 0.0f) ? pi_div(127.0f, hmax) : 0.0f;
        const int qh = (int)rintf(__fmul_rn(hvv, idh));
        // neurons that add something, ascending
        const uint32_t nz = (uint32_t)__ballot(qh != 0) & sel;
        const int nrows = __popc(nz);
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
        for (int k0 = 0; k0 < nrows; k0 += kAqChunkFused) {
            uint32_t q[kAqChunkFused][2];
            uint16_t dw[kAqChunkFused];
            int alpha[kAqChunkFused];
#pragma unroll
            for (int j = 0; j < kAqChunkFused; ++j) {
                if (k0 + j < nrows) {
                    const int bit = select_nth_bit(nz, k0 + j);
                    alpha[j] = __builtin_amdgcn_readlane(qh, bit);
                    const int below = __popc(hot & ((1u << bit) - 1u));
                    const bool rest = SPLIT && !((hot >> bit) & 1u);
                    const size_t row = rest ? (size_t)(n0 - base_row + bit - below) : (size_t)(base_row + below);
                    const pi_block_q4_0 * wb = (rest ? Wd_rest : Wd) + row * nb + blk;
                    __builtin_memcpy(&dw[j], &wb->d, 2);
                    __builtin_memcpy(q[j], wb->qs + qoff, 8);
                }
            }
#pragma unroll
            for (int j = 0; j < kAqChunkFused; ++j) {
                if (k0 + j < nrows) {
                    const float d = __fmul_rn(pi_f16_from_bits(dw[j]), dh);
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const int v = (int)((q[j][i >> 2] >> ((i & 3) * 8 + shift)) & 0xF) - 8;
                        acc[i] = __fadd_rn(acc[i], __fmul_rn((float)(v * alpha[j]), d));
                    }
                }
            }
        }
        float4 * po = reinterpret_cast<float4 *>(partial + (size_t)blockIdx.x * cols + cbase);
        po[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
        po[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
    }
}

// Q4_0 down projection behind pred_upgate_q4_kernel (cols == 4096).  A workgroup owns kAqGroups x 32 consecutive neurons.
// Their h (hot and host-computed values merged by the caller; `h` may be pinned host memory, only wave 0 touches it) is
// quantised to Q8_0 over the 32-neuron blocks exactly as the CPU path does on the dense vector (ggml.c:14465-14618):
// d = amax/127 as fp16, q = rint(h*127/amax).  Neurons with q != 0 that live on the GPU are compacted into LDS, and the 8
// waves each add their 512-column slice of those rows: acc += float((nibble - 8) * q) * (d_w * d_h), one fp32 multiply and
// one fp32 add per element (ggml_axpy_q4_0_q8_0, ggml-quants.c:2426-2509), rows in ascending order.  One partial vector per
// workgroup goes to `partial`; ffn_reduce_kernel adds them in workgroup order.
constexpr int kAqGroups = 1;               // the launch is all latency: more, smaller workgroups finish sooner (4 -> 1: 12.8 us -> about 9 per 7B layer)
constexpr int kAqN = kAqGroups * 32;       // neurons per workgroup
constexpr int kAqChunk = 16;               // rows in flight per wave

// SPLIT: rows of the neurons outside the hot words come from Wd_rest (those neurons' rows in ascending order, pinned host memory).
constexpr int kAqRestFlag = 1 << 30;
template <bool SPLIT>
__global__ __launch_bounds__(kPfBlock, 2) void axpy_q4_groups_kernel(const pi_block_q4_0 * __restrict__ Wd, const pi_block_q4_0 * __restrict__ Wd_rest,
                                                                     const float * h, int ff,
                                                                     const uint32_t * __restrict__ hot_words, const int32_t * __restrict__ hot_prefix,
                                                                     float * __restrict__ partial) {
    constexpr int cols = 4096, nb = cols / 32;
    __shared__ int   lrow[kAqN];
    __shared__ int   lq[kAqN];
    __shared__ float ld[kAqN];
    __shared__ int   ln;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int cbase = wave * 512 + lane * 8, blk = cbase >> 5, sub = lane & 3;
    const int n0 = blockIdx.x * kAqN;
    if (wave == 0) {
        int cnt = 0;
#pragma unroll
        for (int i = 0; i < (kAqN + 63) / 64; ++i) {
            const bool mine = i * 64 + lane < kAqN;                  // kAqN == 32: the upper half of the wave idles
            const int nrn = mine ? n0 + i * 64 + lane : ff;
            const float hvv = nrn < ff ? h[nrn] : 0.0f;
            float amax = fabsf(hvv);
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, PI_WAVE));
            const float d = pi_div(amax, 127.0f), id = (amax != 0.0f) ? pi_div(127.0f, amax) : 0.0f;
            const int q = (int)rintf(__fmul_rn(hvv, id));
            const int g = nrn >> 5;
            const uint32_t hot = (nrn < ff) ? (hot_words ? hot_words[g] : 0xFFFFFFFFu) : 0u;
            const bool is_hot = (hot >> (lane & 31)) & 1u;
            const bool take = q != 0 && (is_hot || (SPLIT && nrn < ff));
            const unsigned long long b = __ballot(take);
            if (take) {
                const int pos = cnt + __popcll(b & ((1ull << lane) - 1ull));
                const int base = hot_prefix ? hot_prefix[g] : (nrn & ~31), below = __popc(hot & ((1u << (lane & 31)) - 1u));
                lrow[pos] = is_hot ? base + below : (((nrn & ~31) - base + (lane & 31) - below) | kAqRestFlag);
                lq[pos] = q;
                ld[pos] = pi_round_f16(d);
            }
            cnt += __popcll(b);
        }
        if (lane == 0) ln = cnt;
    }
    __syncthreads();
    const int n = ln;
    const int shift = (sub >> 1) * 4, qoff = (sub & 1) * 8;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    for (int k0 = 0; k0 < n; k0 += kAqChunk) {
        uint32_t q[kAqChunk][2];
        uint16_t dw[kAqChunk];
#pragma unroll
        for (int j = 0; j < kAqChunk; ++j) {
            if (k0 + j < n) {
                const int lr = lrow[k0 + j];
                const pi_block_q4_0 * wb = ((SPLIT && (lr & kAqRestFlag)) ? Wd_rest + (size_t)(lr & ~kAqRestFlag) * nb : Wd + (size_t)lr * nb) + blk;
                __builtin_memcpy(&dw[j], &wb->d, 2);
                __builtin_memcpy(q[j], wb->qs + qoff, 8);
            }
        }
#pragma unroll
        for (int j = 0; j < kAqChunk; ++j) {
            if (k0 + j < n) {
                const int alpha = lq[k0 + j];
                const float d = __fmul_rn(pi_f16_from_bits(dw[j]), ld[k0 + j]);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int v = (int)((q[j][i >> 2] >> ((i & 3) * 8 + shift)) & 0xF) - 8;
                    acc[i] = __fadd_rn(acc[i], __fmul_rn((float)(v * alpha), d));
                }
            }
        }
    }
    float4 * po = reinterpret_cast<float4 *>(partial + (size_t)blockIdx.x * cols + cbase);
    po[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    po[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
}

// Hand-over points between the device and host threads that compute a share of a layer (hybrid layers).  Both sides count the
// hand-overs; the device's count lives in *seq.  `flags` is pinned host memory: word 0 is written by the device, words 16 and 32
// (their own cache lines) by the host, word 48 is the host's stop word; word 8 is a second device-written word.
//   host_signal_kernel: everything queued before it on the stream is complete and visible to the host (a kernel boundary releases
//                       at system scope): publish *seq in flags[word] (word 0 or 8), after advancing it when a new hand-over starts.
//   host_wait_kernel:   (publishes *seq in flags[signal_word] first when signal_word >= 0: a signal and a wait in one launch;)
//                       returns once flags[slot] has reached *seq.  The wait is bounded: after `limit` ticks of the 100 MHz clock, or
//                       when the host has set its stop word, the kernel records the failure in *status and returns, so the stream
//                       always drains; later waits then return at once.
__global__ void host_signal_kernel(uint32_t * __restrict__ seq, uint32_t * __restrict__ flags, int word, int advance) {
    if (threadIdx.x == 0) {
        uint32_t s = *seq;
        if (advance) { s += 1u; *seq = s; }
        __hip_atomic_store(flags + word, s, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}
__global__ void host_wait_kernel(const uint32_t * __restrict__ seq, uint32_t * __restrict__ flags, int slot, uint32_t * __restrict__ status,
                                 unsigned long long limit, int signal_word) {
    if (threadIdx.x != 0) return;
    const uint32_t want = *seq;
    if (signal_word >= 0) __hip_atomic_store(flags + signal_word, want, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);     // host_signal_kernel without advance
    if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0u) return;
    const unsigned long long t0 = wall_clock64();
    for (;;) {
        const uint32_t v = __hip_atomic_load(flags + slot, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM);
        if ((int32_t)(v - want) >= 0) return;
        if (__hip_atomic_load(flags + 48, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0u || wall_clock64() - t0 > limit) {
            __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            return;
        }
        __builtin_amdgcn_s_sleep(4);
    }
}

}  // namespace

extern "C" {

int pi_k_pred_upgate_q4_supported(int ff, int r, int cols) {
    return cols == 4096 && (r == 512 || r == 1024) && ff > 0 && ff % 32 == 0;
}

int pi_k_pred_upgate_q4(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                        const void * up_q4, const void * gate_q4, int cols, const float * x, const pi_norm * norm,
                        const uint32_t * hot_words, const int32_t * hot_prefix,
                        float * logits, float * h_dense, void * xq8_out, pi_workspace * ws, pi_stream_t stream) {
    return pi_k_pred_upgate_q4_split(fc2_f16, ff, r, hidden, threshold, up_q4, gate_q4, nullptr, nullptr, cols, x, norm, hot_words, hot_prefix,
                                     logits, h_dense, xq8_out, ws, stream);
}

int pi_k_pred_upgate_q4_split(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                              const void * up_q4, const void * gate_q4, const void * up_rest_q4, const void * gate_rest_q4,
                              int cols, const float * x, const pi_norm * norm,
                              const uint32_t * hot_words, const int32_t * hot_prefix,
                              float * logits, float * h_dense, void * xq8_out, pi_workspace * ws, pi_stream_t stream) {
    if (!fc2_f16 || !hidden || !up_q4 || !x || !h_dense || !ws) return pi::fail(PI_E_ARG, "pi_k_pred_upgate_q4: null pointer");
    if (up_rest_q4 && (!hot_words || (gate_q4 != nullptr) != (gate_rest_q4 != nullptr)))
        return pi::fail(PI_E_ARG, "pi_k_pred_upgate_q4_split: the second matrices need hot_words / hot_prefix and a gate on both sides or on neither");
    if (!pi_k_pred_upgate_q4_supported(ff, r, cols)) return pi::fail(PI_E_UNSUPPORTED, "pi_k_pred_upgate_q4: shape outside the fused kernel (cols 4096, r 512 or 1024, ff % 32 == 0)");
    if (ff > ws->max_ff || cols > ws->max_d) return pi::fail(PI_E_ARG, "pi_k_pred_upgate_q4: shape exceeds the workspace");
    if ((hot_words == nullptr) != (hot_prefix == nullptr)) return pi::fail(PI_E_ARG, "pi_k_pred_upgate_q4: hot_words and hot_prefix go together");
    const NormArgs na = to_norm(norm);
    if ((((uintptr_t)hidden | (uintptr_t)x | (uintptr_t)na.w | (uintptr_t)na.b) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_pred_upgate_q4: vectors must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const __half * w2 = (const __half *)fc2_f16;
    const pi_block_q4_0 * u = (const pi_block_q4_0 *)up_q4; const pi_block_q4_0 * g = (const pi_block_q4_0 *)gate_q4;
    const dim3 grid(ff / 32), block(kPfBlock);
    const pi_block_q4_0 * ur = (const pi_block_q4_0 *)up_rest_q4; const pi_block_q4_0 * gr = (const pi_block_q4_0 *)gate_rest_q4;
#define PI_PQ_LAUNCH(RCH, GATE, SPLIT) hipLaunchKernelGGL((pred_upgate_q4_kernel<RCH, GATE, SPLIT>), grid, block, 0, st, w2, hidden, u, g, ur, gr, x, na, threshold, hot_words, hot_prefix, logits, ws->words, ws->words_hot, h_dense, (pi_q8_host_block *)xq8_out, nullptr, nullptr, nullptr, nullptr, HostAnnounce{nullptr, nullptr})
#define PI_PQ_LAUNCH_S(RCH, GATE) do { if (ur) PI_PQ_LAUNCH(RCH, GATE, true); else PI_PQ_LAUNCH(RCH, GATE, false); } while (0)
    if (r == 1024) { if (g) PI_PQ_LAUNCH_S(2, true); else PI_PQ_LAUNCH_S(2, false); }
    else           { if (g) PI_PQ_LAUNCH_S(1, true); else PI_PQ_LAUNCH_S(1, false); }
#undef PI_PQ_LAUNCH_S
#undef PI_PQ_LAUNCH
    return pi::check_launch("pi_k_pred_upgate_q4");
}

int pi_k_sparse_ffn_q4_partials(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                                const void * up_q4, const void * gate_q4, const void * down_t_q4,
                                const void * up_rest_q4, const void * gate_rest_q4, const void * down_t_rest_q4,
                                int cols, const float * x, const pi_norm * norm, const uint32_t * hot_words, const int32_t * hot_prefix,
                                float * logits, float * h_dense, pi_workspace * ws, pi_stream_t stream) {
    if (!fc2_f16 || !hidden || !up_q4 || !down_t_q4 || !x || !h_dense || !ws) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_q4_partials: null pointer");
    const bool split = up_rest_q4 != nullptr;
    if (split != (down_t_rest_q4 != nullptr) || (split && (!hot_words || !hot_prefix || (gate_q4 != nullptr) != (gate_rest_q4 != nullptr))) || (!split && hot_words))
        return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_q4_partials: either every neuron's rows are in the first matrices (no hot words), or the second matrices and hot_words / hot_prefix come together");
    if (!pi_k_pred_upgate_q4_supported(ff, r, cols) || ff > ws->max_ff || cols > ws->max_d) return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_ffn_q4_partials: shape outside the fused kernel (cols 4096, r 512 or 1024, ff % 32 == 0) or the workspace");
    const NormArgs na = to_norm(norm);
    if ((((uintptr_t)hidden | (uintptr_t)x | (uintptr_t)na.w | (uintptr_t)na.b) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_q4_partials: vectors must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const __half * w2 = (const __half *)fc2_f16;
    const pi_block_q4_0 * u = (const pi_block_q4_0 *)up_q4; const pi_block_q4_0 * g = (const pi_block_q4_0 *)gate_q4; const pi_block_q4_0 * dn = (const pi_block_q4_0 *)down_t_q4;
    const pi_block_q4_0 * ur = (const pi_block_q4_0 *)up_rest_q4; const pi_block_q4_0 * gr = (const pi_block_q4_0 *)gate_rest_q4; const pi_block_q4_0 * dr = (const pi_block_q4_0 *)down_t_rest_q4;
    const dim3 grid(ff / 32), block(kPfBlock);
#define PI_PQF(RCH, GATE, SPLIT) hipLaunchKernelGGL((pred_upgate_q4_kernel<RCH, GATE, SPLIT, 0, true>), grid, block, 0, st, w2, hidden, u, g, ur, gr, x, na, threshold, hot_words, hot_prefix, logits, ws->words, (uint32_t *)nullptr, h_dense, (pi_q8_host_block *)nullptr, (float *)nullptr, dn, dr, ws->ffn_partial, HostAnnounce{nullptr, nullptr})
#define PI_PQF_S(RCH, GATE) do { if (split) PI_PQF(RCH, GATE, true); else PI_PQF(RCH, GATE, false); } while (0)
    if (r == 1024) { if (g) PI_PQF_S(2, true); else PI_PQF_S(2, false); }
    else           { if (g) PI_PQF_S(1, true); else PI_PQF_S(1, false); }
#undef PI_PQF_S
#undef PI_PQF
    return pi::check_launch("pi_k_sparse_ffn_q4_partials");
}

int pi_k_sparse_ffn_q4_reduce(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out, int32_t * n_active,
                              pi_workspace * ws, pi_stream_t stream) {
    if (!out || !ws || cols != 4096 || ff <= 0 || ff % 32 || ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_q4_reduce: bad arguments");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || epilogue == PI_EPI_RELU || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_q4_reduce: bad epilogue arguments");
    hipLaunchKernelGGL(ffn_reduce_kernel, dim3(cols / kFrCols), dim3(kPfBlock), 0, (hipStream_t)stream, ws->ffn_partial, ff / 32, cols,
                       ws->words, ff / 32, n_active, epilogue, add1, add2, out);
    return pi::check_launch("pi_k_sparse_ffn_q4_reduce");
}

int pi_k_pred_q4_logits(const void * fc2_f16, int ff, int r, const float * hidden, float threshold, int cols, const float * x, const pi_norm * norm,
                        float * logits, float * logits_dev, void * xq8_out, uint32_t * words_out, pi_workspace * ws, pi_stream_t stream) {
    if (!fc2_f16 || !hidden || !x || !logits_dev || !ws) return pi::fail(PI_E_ARG, "pi_k_pred_q4_logits: null pointer");
    if (!pi_k_pred_upgate_q4_supported(ff, r, cols) || ff > ws->max_ff || cols > ws->max_d) return pi::fail(PI_E_UNSUPPORTED, "pi_k_pred_q4_logits: shape outside the fused kernel or the workspace");
    const NormArgs na = to_norm(norm);
    if ((((uintptr_t)hidden | (uintptr_t)x | (uintptr_t)na.w | (uintptr_t)na.b) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_pred_q4_logits: vectors must be 16-byte aligned");
    const dim3 grid(ff / 32), block(kPfBlock);
    const pi_block_q4_0 * none = nullptr;
#define PI_PQ1(RCH) hipLaunchKernelGGL((pred_upgate_q4_kernel<RCH, false, false, 1>), grid, block, 0, (hipStream_t)stream, (const __half *)fc2_f16, hidden, none, none, none, none, x, na, threshold, (const uint32_t *)nullptr, (const int32_t *)nullptr, logits, ws->words, words_out, (float *)nullptr, (pi_q8_host_block *)xq8_out, logits_dev, none, none, (float *)nullptr, HostAnnounce{nullptr, nullptr})
    if (r == 1024) PI_PQ1(2); else PI_PQ1(1);
#undef PI_PQ1
    return pi::check_launch("pi_k_pred_q4_logits");
}

int pi_k_upgate_q4_hot_rows(int ff, float threshold, const void * up_q4, const void * gate_q4, int cols, const float * x, const pi_norm * norm,
                            const uint32_t * hot_words, const int32_t * hot_prefix, const float * logits_dev, float * h_dense,
                            uint32_t * announce_seq, uint32_t * announce_flags, pi_workspace * ws, pi_stream_t stream) {
    if (!up_q4 || !x || !hot_words || !hot_prefix || !logits_dev || !h_dense || !ws) return pi::fail(PI_E_ARG, "pi_k_upgate_q4_hot_rows: null pointer");
    if ((announce_seq == nullptr) != (announce_flags == nullptr)) return pi::fail(PI_E_ARG, "pi_k_upgate_q4_hot_rows: announce_seq and announce_flags go together");
    if (cols != 4096 || ff <= 0 || ff % 32 || ff > ws->max_ff || cols > ws->max_d) return pi::fail(PI_E_UNSUPPORTED, "pi_k_upgate_q4_hot_rows: cols must be 4096, ff % 32 == 0, within the workspace");
    const NormArgs na = to_norm(norm);
    if ((((uintptr_t)x | (uintptr_t)na.w | (uintptr_t)na.b) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_upgate_q4_hot_rows: vectors must be 16-byte aligned");
    const dim3 grid(ff / 32), block(kPfBlock);
    const pi_block_q4_0 * none = nullptr;
    const pi_block_q4_0 * u = (const pi_block_q4_0 *)up_q4; const pi_block_q4_0 * g = (const pi_block_q4_0 *)gate_q4;
#define PI_PQ2(GATE) hipLaunchKernelGGL((pred_upgate_q4_kernel<1, GATE, false, 2>), grid, block, 0, (hipStream_t)stream, (const __half *)nullptr, (const float *)nullptr, u, g, none, none, x, na, threshold, hot_words, hot_prefix, (float *)nullptr, ws->words, ws->words_hot, h_dense, (pi_q8_host_block *)nullptr, const_cast<float *>(logits_dev), none, none, (float *)nullptr, HostAnnounce{announce_seq, announce_flags})
    if (g) PI_PQ2(true); else PI_PQ2(false);
#undef PI_PQ2
    return pi::check_launch("pi_k_upgate_q4_hot_rows");
}

int pi_k_axpy_q4_partials(const void * down_t_q4, int cols, int ff, const float * h, const uint32_t * hot_words, const int32_t * hot_prefix,
                          pi_workspace * ws, pi_stream_t stream) {
    return pi_k_axpy_q4_partials_split(down_t_q4, nullptr, cols, ff, h, hot_words, hot_prefix, ws, stream);
}

int pi_k_axpy_q4_partials_split(const void * down_t_q4, const void * down_t_rest_q4, int cols, int ff, const float * h,
                                const uint32_t * hot_words, const int32_t * hot_prefix, pi_workspace * ws, pi_stream_t stream) {
    if (!down_t_q4 || !h || !ws) return pi::fail(PI_E_ARG, "pi_k_axpy_q4_partials: null pointer");
    if (down_t_rest_q4 && !hot_words) return pi::fail(PI_E_ARG, "pi_k_axpy_q4_partials_split: the second matrix needs hot_words / hot_prefix");
    if (cols != 4096 || ff <= 0 || ff % 32 || ff > ws->max_ff || cols > ws->max_d) return pi::fail(PI_E_UNSUPPORTED, "pi_k_axpy_q4_partials: cols must be 4096, ff % 32 == 0, within the workspace");
    if ((hot_words == nullptr) != (hot_prefix == nullptr)) return pi::fail(PI_E_ARG, "pi_k_axpy_q4_partials: hot_words and hot_prefix go together");
    if (down_t_rest_q4)
        hipLaunchKernelGGL(axpy_q4_groups_kernel<true>, dim3((ff + kAqN - 1) / kAqN), dim3(kPfBlock), 0, (hipStream_t)stream,
                           (const pi_block_q4_0 *)down_t_q4, (const pi_block_q4_0 *)down_t_rest_q4, h, ff, hot_words, hot_prefix, ws->ffn_partial);
    else
        hipLaunchKernelGGL(axpy_q4_groups_kernel<false>, dim3((ff + kAqN - 1) / kAqN), dim3(kPfBlock), 0, (hipStream_t)stream,
                           (const pi_block_q4_0 *)down_t_q4, (const pi_block_q4_0 *)nullptr, h, ff, hot_words, hot_prefix, ws->ffn_partial);
    return pi::check_launch("pi_k_axpy_q4_partials");
}

int pi_k_axpy_q4_reduce(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out, int32_t * n_active,
                        pi_workspace * ws, pi_stream_t stream) {
    if (!out || !ws || cols != 4096 || ff <= 0 || ff % 32 || ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_axpy_q4_reduce: bad arguments");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || epilogue == PI_EPI_RELU || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_axpy_q4_reduce: bad epilogue arguments");
    hipLaunchKernelGGL(ffn_reduce_kernel, dim3(cols / kFrCols), dim3(kPfBlock), 0, (hipStream_t)stream, ws->ffn_partial, (ff + kAqN - 1) / kAqN, cols,
                       ws->words_hot, ff / 32, n_active, epilogue, add1, add2, out);
    return pi::check_launch("pi_k_axpy_q4_reduce");
}

static int pf_cu_workgroups(int ff, int r, int cols);
// the grouped form (a workgroup per 32 G neurons) and the two-phase forms of hybrid layers
static bool pf_grouped_shape(int ff, int r, int cols) { return (cols == 4096 || cols == 8192) && (r == 1024 || r == 512) && ff > 0 && ff % 32 == 0; }
// 5120 columns with a predictor of rank 1280 (the 13B shape) exist in the one-workgroup-per-unit form only: every neuron resident,
// at most 60 neurons per compute unit
int pi_k_sparse_ffn_supported(int ff, int r, int cols) { return pf_grouped_shape(ff, r, cols) || pf_cu_workgroups(ff, r, cols) > 0; }
static int pf_parts(int ff, int r, int cols, bool hyb);
int pi_k_sparse_ffn_workgroups(int ff, int r, int cols) { return pi_k_sparse_ffn_supported(ff, r, cols) ? pf_parts(ff, r, cols, false) : 0; }

// Groups of 32 neurons per workgroup of the fused sparse FFN.  Wide rows: a workgroup takes four groups in turn (the next
// group's predictor rows travel during the current group's FFN rows) and stores one partial vector for all of them, which
// quarters the partial-sum traffic (it grows with cols; at 32768 x 8192 it was 67 MB of 220 MB per layer).
static int pf_groups(int ff, int cols) {
    if (cols != 8192) return 1;                    // at 4096 columns one group per workgroup measured fastest
    return (ff % 128 == 0 && ff / 128 >= 256) ? 4 : 1;
}

// Workgroups of the one-per-compute-unit form (ffn_cu_f16_kernel), or 0 where the grouped form runs: 4096 columns, every neuron on
// the device, and more than 32 but at most 64 neurons per unit (with 32 or fewer the groups of 32 already have a unit each).
static int pf_cu_workgroups(int ff, int r, int cols) {
    const bool wide = cols == 5120 && r == 1280;
    if (!wide && !(cols == 4096 && (r == 1024 || r == 512))) return 0;
    const int n_cu = pi::compute_units();
    if (n_cu <= 0 || ff <= 32 * n_cu || (ff + n_cu - 1) / n_cu > (wide ? 60 : 64)) return 0;
    return n_cu;
}
// partial vectors the fused launch leaves for the reduction when nothing about the call rules the one-per-unit form out
static int pf_parts(int ff, int r, int cols, bool hyb) { const int n = hyb ? 0 : pf_cu_workgroups(ff, r, cols); return n ? n : ff / (32 * pf_groups(ff, cols)); }

static int sparse_ffn_partials_impl(const char * who, const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                                    const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols, const float * x, const pi_norm * norm,
                                    float * logits, float * h_dense, const uint32_t * hot_words, const int32_t * hot_prefix, void * xn_f16_out,
                                    pi_workspace * ws, pi_stream_t stream) {
    if (!fc2_f16 || !hidden || !up_f16 || !down_t_f16 || !x || !ws) return pi::fail(PI_E_ARG, who);
    if (!pi_k_sparse_ffn_supported(ff, r, cols)) return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_ffn: shape outside the fused kernels (cols 4096 or 8192 with r 512 or 1024 and ff % 32 == 0; cols 5120 with r 1280 and 33..60 neurons per compute unit)");
    if (ff > ws->max_ff || cols > ws->max_d) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn: shape exceeds the workspace");
    if ((hot_words == nullptr) != (hot_prefix == nullptr)) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn: hot_words and hot_prefix go together");
    const NormArgs na = to_norm(norm);
    if ((((uintptr_t)hidden | (uintptr_t)x | (uintptr_t)na.w | (uintptr_t)na.b | (uintptr_t)xn_f16_out) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn: vectors must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const __half * w2 = (const __half *)fc2_f16; const __half * u = (const __half *)up_f16; const __half * g = (const __half *)gate_f16;
    const __half * dn = (const __half *)down_t_f16;
    const bool hyb = hot_words != nullptr;
    // the one-workgroup-per-unit form takes the norm as a template parameter: it must carry what its kind needs
    const bool cu_norm = na.kind == 0 || (na.kind == 1 && na.w && !na.b) || (na.kind == 2 && na.w && na.b);
    if (const int n_wg = (hyb || !cu_norm) ? 0 : pf_cu_workgroups(ff, r, cols)) {
        const int nw = cols / 512;
        const int rows = ((ff + n_wg - 1) / n_wg + nw - 1) / nw;         // fc2 rows per wave
#define PI_CU_LAUNCH(NW, R, GATE, ROWS, KIND) hipLaunchKernelGGL((ffn_cu_f16_kernel<NW, R, GATE, ROWS, KIND>), dim3(n_wg), dim3(NW * 64), 0, st, w2, hidden, u, g, dn, x, na.w, na.b, na.eps, threshold, ff, logits, ws->words, h_dense, ws->ffn_partial)
#define PI_CU_KIND(NW, R, GATE, ROWS) do { if (na.kind == 0) PI_CU_LAUNCH(NW, R, GATE, ROWS, 0); else if (na.kind == 1) PI_CU_LAUNCH(NW, R, GATE, ROWS, 1); else PI_CU_LAUNCH(NW, R, GATE, ROWS, 2); } while (0)
#define PI_CU_ROWS(NW, R, GATE) do { if (rows <= 6) PI_CU_KIND(NW, R, GATE, 6); else PI_CU_KIND(NW, R, GATE, 8); } while (0)
        if (cols == 5120)   { if (g) PI_CU_KIND(10, 1280, true, 6); else PI_CU_KIND(10, 1280, false, 6); }
        else if (r == 1024) { if (g) PI_CU_ROWS(8, 1024, true); else PI_CU_ROWS(8, 1024, false); }
        else                { if (g) PI_CU_ROWS(8, 512, true); else PI_CU_ROWS(8, 512, false); }
#undef PI_CU_ROWS
#undef PI_CU_KIND
#undef PI_CU_LAUNCH
        ws->pf_parts = n_wg; ws->pf_words = 2 * n_wg;
        return pi::check_launch(who);
    }
    if (!pf_grouped_shape(ff, r, cols)) return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_ffn: this shape runs only with every neuron resident and a norm the kernel carries (5120 columns, rank 1280)");
    ws->pf_parts = ff / (32 * pf_groups(ff, cols)); ws->pf_words = ff / 32;
    const int G = pf_groups(ff, cols);
    const dim3 grid(ff / (32 * G)), block(kPfBlock);
#define PI_PF_LAUNCH2(CPW, RCH, GATE, GG, HYB) hipLaunchKernelGGL((pred_ffn_f16_kernel<CPW, RCH, GATE, GG, HYB>), grid, block, 0, st, w2, hidden, u, g, dn, x, na, threshold, logits, ws->words, h_dense, ws->ffn_partial, hot_words, hot_prefix, ws->words_hot, (__half *)xn_f16_out, nullptr, HostAnnounce{nullptr, nullptr})
#define PI_PF_LAUNCH(CPW, RCH, GATE, GG) do { if (hyb) PI_PF_LAUNCH2(CPW, RCH, GATE, GG, true); else PI_PF_LAUNCH2(CPW, RCH, GATE, GG, false); } while (0)
#define PI_PF_WIDE(RCH, GATE) do { if (G == 4) PI_PF_LAUNCH(2, RCH, GATE, 4); else if (G == 2) PI_PF_LAUNCH(2, RCH, GATE, 2); else PI_PF_LAUNCH(2, RCH, GATE, 1); } while (0)
    const int cpw = cols / 4096, rch = r / 512;
    if (cpw == 1 && rch == 2) { if (g) PI_PF_LAUNCH(1, 2, true, 1); else PI_PF_LAUNCH(1, 2, false, 1); }
    else if (cpw == 1)        { if (g) PI_PF_LAUNCH(1, 1, true, 1); else PI_PF_LAUNCH(1, 1, false, 1); }
    else if (rch == 2)        { if (g) PI_PF_WIDE(2, true); else PI_PF_WIDE(2, false); }
    else                      { if (g) PI_PF_WIDE(1, true); else PI_PF_WIDE(1, false); }
#undef PI_PF_WIDE
#undef PI_PF_LAUNCH
#undef PI_PF_LAUNCH2
    return pi::check_launch(who);
}

int pi_k_sparse_ffn_partials(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                             const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols, const float * x, const pi_norm * norm,
                             float * logits, float * h_dense, pi_workspace * ws, pi_stream_t stream) {
    return sparse_ffn_partials_impl("pi_k_sparse_ffn_partials", fc2_f16, ff, r, hidden, threshold, up_f16, gate_f16, down_t_f16, cols, x, norm, logits, h_dense,
                                    nullptr, nullptr, nullptr, ws, stream);
}

int pi_k_sparse_ffn_partials_hot(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                                 const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols, const float * x, const pi_norm * norm,
                                 const uint32_t * hot_words, const int32_t * hot_prefix, float * logits, float * h_dense, void * xn_f16_out,
                                 pi_workspace * ws, pi_stream_t stream) {
    if (!hot_words || !hot_prefix) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_partials_hot: hot words and prefix are required");
    if (!pf_grouped_shape(ff, r, cols)) return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_ffn_partials_hot: shape outside the fused kernel of hybrid layers (pi_k_sparse_ffn_hot_supported)");
    return sparse_ffn_partials_impl("pi_k_sparse_ffn_partials_hot", fc2_f16, ff, r, hidden, threshold, up_f16, gate_f16, down_t_f16, cols, x, norm, logits, h_dense,
                                    hot_words, hot_prefix, xn_f16_out, ws, stream);
}

int pi_k_sparse_ffn_hot_supported(int ff, int r, int cols) { return pf_grouped_shape(ff, r, cols); }
int pi_k_sparse_ffn_two_phase_supported(int ff, int r, int cols) { return pf_grouped_shape(ff, r, cols) && cols == 4096; }

int pi_k_sparse_ffn_logits_hot(const void * fc2_f16, int ff, int r, const float * hidden, float threshold, int cols, const float * x, const pi_norm * norm,
                               const uint32_t * hot_words, const int32_t * hot_prefix, float * logits, float * logits_dev, void * xn_f16_out,
                               uint32_t * words_out, pi_workspace * ws, pi_stream_t stream) {
    if (!fc2_f16 || !hidden || !x || !hot_words || !hot_prefix || !logits_dev || !ws) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_logits_hot: null pointer");
    if (!pi_k_sparse_ffn_two_phase_supported(ff, r, cols) || ff > ws->max_ff || cols > ws->max_d) return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_ffn_logits_hot: cols must be 4096, r 512 or 1024, ff % 32 == 0, within the workspace");
    const NormArgs na = to_norm(norm);
    if ((((uintptr_t)hidden | (uintptr_t)x | (uintptr_t)na.w | (uintptr_t)na.b | (uintptr_t)xn_f16_out) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_logits_hot: vectors must be 16-byte aligned");
    const dim3 grid(ff / 32), block(kPfBlock);
    const __half * none = nullptr;
#define PI_PF1(RCH) hipLaunchKernelGGL((pred_ffn_f16_kernel<1, RCH, false, 1, true, 1>), grid, block, 0, (hipStream_t)stream, (const __half *)fc2_f16, hidden, none, none, none, x, na, threshold, logits, ws->words, (float *)nullptr, (float *)nullptr, hot_words, hot_prefix, ws->words_hot, (__half *)xn_f16_out, logits_dev, HostAnnounce{nullptr, nullptr, words_out})
    if (r == 1024) PI_PF1(2); else PI_PF1(1);
#undef PI_PF1
    ws->pf_parts = ff / 32; ws->pf_words = ff / 32;
    return pi::check_launch("pi_k_sparse_ffn_logits_hot");
}

int pi_k_sparse_ffn_rows_hot(int ff, float threshold, const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols, const float * x,
                             const pi_norm * norm, const uint32_t * hot_words, const int32_t * hot_prefix, const float * logits_dev, float * h_dense,
                             uint32_t * announce_seq, uint32_t * announce_flags, pi_workspace * ws, pi_stream_t stream) {
    if (!up_f16 || !down_t_f16 || !x || !hot_words || !hot_prefix || !logits_dev || !ws) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_rows_hot: null pointer");
    if ((announce_seq == nullptr) != (announce_flags == nullptr)) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_rows_hot: announce_seq and announce_flags go together");
    if (cols != 4096 || ff <= 0 || ff % 32 || ff > ws->max_ff || cols > ws->max_d) return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_ffn_rows_hot: cols must be 4096, ff % 32 == 0, within the workspace");
    const NormArgs na = to_norm(norm);
    if ((((uintptr_t)x | (uintptr_t)na.w | (uintptr_t)na.b) & 15) != 0) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_rows_hot: vectors must be 16-byte aligned");
    const dim3 grid(ff / 32), block(kPfBlock);
    const __half * u = (const __half *)up_f16; const __half * g = (const __half *)gate_f16; const __half * dn = (const __half *)down_t_f16;
#define PI_PF2(GATE) hipLaunchKernelGGL((pred_ffn_f16_kernel<1, 1, GATE, 1, true, 2>), grid, block, 0, (hipStream_t)stream, (const __half *)nullptr, (const float *)nullptr, u, g, dn, x, na, threshold, (float *)nullptr, ws->words, h_dense, ws->ffn_partial, hot_words, hot_prefix, ws->words_hot, (__half *)nullptr, const_cast<float *>(logits_dev), HostAnnounce{announce_seq, announce_flags})
    if (g) PI_PF2(true); else PI_PF2(false);
#undef PI_PF2
    ws->pf_parts = ff / 32; ws->pf_words = ff / 32;
    return pi::check_launch("pi_k_sparse_ffn_rows_hot");
}

static int sparse_ffn_reduce_impl(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out, int32_t * n_active,
                                  bool hot, pi_workspace * ws, pi_stream_t stream);

int pi_k_sparse_ffn_reduce(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out, int32_t * n_active,
                           pi_workspace * ws, pi_stream_t stream) {
    return sparse_ffn_reduce_impl(ff, cols, epilogue, add1, add2, out, n_active, false, ws, stream);
}

int pi_k_sparse_ffn_reduce_hot(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out, int32_t * n_active,
                               pi_workspace * ws, pi_stream_t stream) {
    return sparse_ffn_reduce_impl(ff, cols, epilogue, add1, add2, out, n_active, true, ws, stream);
}

static int sparse_ffn_reduce_impl(int ff, int cols, int epilogue, const float * add1, const float * add2, float * out, int32_t * n_active,
                                  bool hot, pi_workspace * ws, pi_stream_t stream) {
    if (!out || !ws || ff <= 0 || ff % 32 || ff > ws->max_ff || cols <= 0 || cols % 64 || cols > ws->max_d) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_reduce: bad arguments");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || epilogue == PI_EPI_RELU || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_sparse_ffn_reduce: bad epilogue arguments");
    if (ws->pf_parts <= 0 || ws->pf_words <= 0 || ws->pf_words > ws->max_ff / 32 + 2048)
        return pi::fail(PI_E_STATE, "pi_k_sparse_ffn_reduce: no fused launch has filled this workspace");
    hipLaunchKernelGGL(ffn_reduce_kernel, dim3(cols / kFrCols), dim3(kPfBlock), 0, (hipStream_t)stream, ws->ffn_partial, ws->pf_parts, cols, hot ? ws->words_hot : ws->words,
                       ws->pf_words, n_active, epilogue, add1, add2, out);
    return pi::check_launch("pi_k_sparse_ffn_reduce");
}

int pi_k_sparse_ffn(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                    const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols, const float * x, const pi_norm * norm,
                    int epilogue, const float * add1, const float * add2, float * out,
                    float * logits, float * h_dense, int32_t * n_active, pi_workspace * ws, pi_stream_t stream) {
    if (!out) return pi::fail(PI_E_ARG, "pi_k_sparse_ffn: null pointer");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || epilogue == PI_EPI_RELU || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_sparse_ffn: bad epilogue arguments");
    const int rc = pi_k_sparse_ffn_partials(fc2_f16, ff, r, hidden, threshold, up_f16, gate_f16, down_t_f16, cols, x, norm, logits, h_dense, ws, stream);
    if (rc != PI_OK) return rc;
    return pi_k_sparse_ffn_reduce(ff, cols, epilogue, add1, add2, out, n_active, ws, stream);
}

// ---- the fused sparse FFN for callers that may not allocate ------------------------------------------------
// The block's scratch (per-workgroup partial outputs, activity words) lives in a file-scope device array instead of a
// pi_workspace, so the call reaches no allocator.  Every call on a device shares that device's array.
}  // extern "C"

constexpr size_t kNaPartialBytes = (size_t)8 << 20;      // per-workgroup partial vectors: n_parts * cols floats
constexpr int    kNaMaxWords     = 4096;                 // activity words: ff / 32
constexpr size_t kNaScratchBytes = kNaPartialBytes + 2 * sizeof(uint32_t) * kNaMaxWords;
static __device__ __align__(256) unsigned char scratch[kNaScratchBytes];

namespace {
constexpr int kNaMaxDevices = 16;
unsigned char * g_na_ptr[kNaMaxDevices] = {};            // device address of `scratch` on each device (the name itself is not one)
}

// the scratch array's address on the current device.  pi_init resolves it once per device (resolve = true: taking a symbol's address
// may load the code object, which allocates); the entry point itself only looks it up, so that a call never reaches an allocator.
static int noalloc_setup_current_device(unsigned char ** out, bool resolve) {
    int dev = -1;
    PI_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kNaMaxDevices) return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_ffn_noalloc: device index beyond 15");
    if (!g_na_ptr[dev] && !resolve) return pi::fail(PI_E_STATE, "pi_k_sparse_ffn_noalloc: call pi_init on this device first (it resolves the scratch array's address)");
    if (!g_na_ptr[dev]) {
        unsigned char * p = nullptr;
        PI_HIP_TRY(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
        if (!p) return pi::fail(PI_E_HIP, "pi_k_sparse_ffn_noalloc: the scratch array has no device address");
        g_na_ptr[dev] = p;
    }
    if (out) *out = g_na_ptr[dev];
    return PI_OK;
}

namespace pi {
int noalloc_setup() { return noalloc_setup_current_device(nullptr, true); }      // called by pi_init with the device current
}

extern "C" {

size_t pi_k_sparse_ffn_noalloc_scratch_bytes(void) { return kNaScratchBytes; }

int pi_k_sparse_ffn_noalloc_supported(int ff, int r, int cols) {
    if (!pi_k_sparse_ffn_supported(ff, r, cols)) return 0;
    const size_t parts = (size_t)pf_parts(ff, r, cols, false);
    return ff / 32 <= kNaMaxWords && 2 * parts <= (size_t)kNaMaxWords && parts * (size_t)cols * sizeof(float) <= kNaPartialBytes;
}

int pi_k_sparse_ffn_noalloc(const void * fc2_f16, int ff, int r, const float * hidden, float threshold,
                            const void * up_f16, const void * gate_f16, const void * down_t_f16, int cols, const float * x, const pi_norm * norm,
                            int epilogue, const float * add1, const float * add2, float * out,
                            float * logits, float * h_dense, int32_t * n_active, pi_stream_t stream) {
    if (!pi_k_sparse_ffn_supported(ff, r, cols)) return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_ffn_noalloc: shape outside the fused kernel (cols 4096 or 8192, r 512 or 1024, ff % 32 == 0)");
    if (!pi_k_sparse_ffn_noalloc_supported(ff, r, cols))
        return pi::fail(PI_E_UNSUPPORTED, "pi_k_sparse_ffn_noalloc: shape exceeds the static scratch (at most 8 MiB of partial vectors = (ff / 32 or ff / 128) * cols floats, ff <= 131072)");
    unsigned char * base = nullptr;
    const int rc = noalloc_setup_current_device(&base, false);
    if (rc != PI_OK) return rc;
    // a workspace view of the static array: only the members the fused route touches
    pi_workspace ws{};
    ws.max_ff = kNaMaxWords * 32; ws.max_d = cols;
    ws.ffn_partial = reinterpret_cast<float *>(base);
    ws.words       = reinterpret_cast<uint32_t *>(base + kNaPartialBytes);
    ws.words_hot   = ws.words + kNaMaxWords;
    return pi_k_sparse_ffn(fc2_f16, ff, r, hidden, threshold, up_f16, gate_f16, down_t_f16, cols, x, norm, epilogue, add1, add2, out,
                           logits, h_dense, n_active, &ws, stream);
}

int pi_k_host_signal(uint32_t * seq, uint32_t * flags_pinned, int word, int advance, pi_stream_t stream) {
    if (!seq || !flags_pinned || (word != 0 && word != 8)) return pi::fail(PI_E_ARG, "pi_k_host_signal: bad arguments (word 0 or 8)");
    hipLaunchKernelGGL(host_signal_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, seq, flags_pinned, word, advance);
    return pi::check_launch("pi_k_host_signal");
}
int pi_k_host_wait(const uint32_t * seq, const uint32_t * flags_pinned, int slot, uint32_t * status_pinned, double limit_seconds, pi_stream_t stream) {
    return pi_k_host_signal_wait(seq, const_cast<uint32_t *>(flags_pinned), -1, slot, status_pinned, limit_seconds, stream);
}
int pi_k_host_signal_wait(const uint32_t * seq, uint32_t * flags_pinned, int signal_word, int slot, uint32_t * status_pinned, double limit_seconds, pi_stream_t stream) {
    if (!seq || !flags_pinned || !status_pinned || (slot != 16 && slot != 32) || !(limit_seconds > 0.0) || limit_seconds > 60.0)
        return pi::fail(PI_E_ARG, "pi_k_host_wait: bad arguments (slot 16 or 32, 0 < limit <= 60 s)");
    if (signal_word != -1 && signal_word != 0 && signal_word != 8) return pi::fail(PI_E_ARG, "pi_k_host_signal_wait: signal word 0 or 8, or -1 for none");
    hipLaunchKernelGGL(host_wait_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, seq, flags_pinned, slot, status_pinned,
                       (unsigned long long)(limit_seconds * 1e8), signal_word);
    return pi::check_launch("pi_k_host_wait");
}

}  // extern "C"

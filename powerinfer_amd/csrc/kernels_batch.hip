// Steps of several tokens: 2..16 sequences in lockstep or a prompt chunk of one sequence.  Dense and sparse mat-muls on the matrix
// cores, the union of the tokens' active rows, norm + rounding passes, Q4_0 expansion and row assembly for prompt chunks.
#include "kernels_common.hpp"
#include <type_traits>

namespace {

// =====================================================================================================
// Batched decode (2..16 tokens per step, one per sequence).  Weights are still streamed once per step, so the
// roofline stays HBM, but 16 dot products per weight would make the VALU the limit: the dense mat-muls and the
// sparse gate/up run on the matrix cores (v_mfma_f32_16x16x32_f16: a tile of 16 weight rows x 16 tokens x 32
// columns per instruction, fp32 accumulate).  Lane l holds, for row (token) l % 16, the 8 columns
// 8 * (l / 16) .. + 8 of the 32-column slab of both operands, i.e. one 16-byte load each; the accumulator lane l
// holds rows 4 * (l / 16) .. + 4 of column (token) l % 16.
// Activations are normalised and rounded to fp16 once per mat-mul input by norm_round_f16_kernel (the CPU path rounds
// them to fp16 before every dot, ggml.c:9703-9716) and read by every tile from L2.
// =====================================================================================================

// the value a Q8_0 block keeps of v: q * fp16(amax / 127) with q = rint(v * 127 / amax) and amax over the 32 consecutive elements
// the 32 lanes of a half-wave hold (quantize_row_q8_0, x86 path, ggml-quants.c:702-760), rounded to fp16 for a mat-mul input
__device__ __forceinline__ float q8_block_value(float v) {
    float amax = fabsf(v);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, PI_WAVE));
    const float d = pi_round_f16(pi_div(amax, 127.0f)), id = (amax != 0.0f) ? pi_div(127.0f, amax) : 0.0f;
    return __fmul_rn((float)(int)rintf(__fmul_rn(v, id)), d);
}

// q8 != 0 (cols % 32 == 0, cols <= 8192): the normalised row goes through Q8_0 blocks of 32 before the fp16 rounding, which is what
// a Q4_0 mat-mul of the CPU path multiplies with (ggml_vec_dot_q4_0_q8_0, ggml-quants.c:2512-2650)
// ol != 0: both outputs in the operand layout of the 16-token mat-muls (pi_ol_index) instead of [token][cols].
__global__ __launch_bounds__(1024) void norm_round_f16_kernel(const float * __restrict__ x, int cols, NormArgs na, __half * __restrict__ out,
                                                              __half * __restrict__ out_plain, int q8, int ol) {
    __shared__ double red[16];
    const float * xt = x + (size_t)blockIdx.x * cols;
    auto at = [&](int i) -> size_t { return ol ? pi_ol_index(blockIdx.x, i) : (size_t)blockIdx.x * cols + i; };
    float mean = 0.0f, scale = 1.0f;
    if (cols <= 8 * 1024) {
        // one memory round trip: the row, the norm weights and the bias are requested together and stay in registers
        float xv[8], wv[8], bv[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int i = threadIdx.x + k * 1024;
            xv[k] = i < cols ? xt[i] : 0.0f;
            wv[k] = (na.kind != 0 && na.w && i < cols) ? na.w[i] : 1.0f;
            bv[k] = (na.kind != 0 && na.b && i < cols) ? na.b[i] : 0.0f;
        }
        if (na.kind == 1) {
            double s = 0.0;
#pragma unroll
            for (int k = 0; k < 8; ++k) s += (double)__fmul_rn(xv[k], xv[k]);
            s = block_sum_f64(s, red);
            scale = pi_inv_sqrt((float)(s / cols) + na.eps);
        } else if (na.kind == 2) {
            double s = 0.0;
#pragma unroll
            for (int k = 0; k < 8; ++k) s += (double)xv[k];
            s = block_sum_f64(s, red);
            mean = (float)(s / cols);
            double s2 = 0.0;
#pragma unroll
            for (int k = 0; k < 8; ++k) { const int i = threadIdx.x + k * 1024; const float v = __fsub_rn(xv[k], mean); if (i < cols) s2 += (double)__fmul_rn(v, v); }
            s2 = block_sum_f64(s2, red);
            scale = pi_inv_sqrt((float)(s2 / cols) + na.eps);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int i = threadIdx.x + k * 1024;
            float v = xv[k];
            if (i < cols && out_plain) out_plain[at(i)] = __float2half_rn(v);
            if (na.kind != 0) {
                v = __fmul_rn(na.kind == 2 ? __fsub_rn(v, mean) : v, scale);
                if (na.w) v = __fmul_rn(v, wv[k]);
                if (na.b) v = __fadd_rn(v, bv[k]);
            }
            if (q8) v = q8_block_value(i < cols ? v : 0.0f);          // every lane takes part in the block's maximum
            if (i < cols) out[at(i)] = __float2half_rn(v);
        }
        return;
    }
    if (na.kind == 1) {
        double s = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float v = xt[i]; s += (double)__fmul_rn(v, v); }
        s = block_sum_f64(s, red);
        scale = pi_inv_sqrt((float)(s / cols) + na.eps);
    } else if (na.kind == 2) {
        double s = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) s += (double)xt[i];
        s = block_sum_f64(s, red);
        mean = (float)(s / cols);
        double s2 = 0.0;
        for (int i = threadIdx.x; i < cols; i += blockDim.x) { const float v = __fsub_rn(xt[i], mean); s2 += (double)__fmul_rn(v, v); }
        s2 = block_sum_f64(s2, red);
        scale = pi_inv_sqrt((float)(s2 / cols) + na.eps);
    }
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        float v = xt[i];
        if (out_plain) out_plain[at(i)] = __float2half_rn(v);
        if (na.kind != 0) {
            v = __fmul_rn(na.kind == 2 ? __fsub_rn(v, mean) : v, scale);
            if (na.w) v = __fmul_rn(v, na.w[i]);
            if (na.b) v = __fadd_rn(v, na.b[i]);
        }
        out[at(i)] = __float2half_rn(v);
    }
}

// y[t][row] = epi( W[row] . xn[t] ), t < T <= 16.  A workgroup owns 16*RT rows; its four waves split the columns in
// quarters (cols % 128 == 0) and merge their 16 x 16 accumulator tiles through LDS in wave order.  A wave loads each
// activation fragment once per 32-column step and uses it for its RT row tiles (the activations of a step are 16 x cols
// fp16, as many bytes per row tile as the weights, so re-reading them per tile would double the L2 -> CU traffic);
// 16 weight loads of 16 B per lane are in flight.
template <int RT>
__global__ __launch_bounds__(kBlock) void gemm_t16_f16_kernel(const __half * __restrict__ W, const __half * __restrict__ xn, int T, int rows, int cols,
                                                              int epi, const float * __restrict__ add1, const float * __restrict__ add2, float * __restrict__ y,
                                                              __half * __restrict__ y16, float thr, unsigned char * __restrict__ row_any, int lay) {
    // lay bit 0: xn in the operand layout (pi_ol_index); bit 1: y16 in the operand layout (the next mat-mul's input)
    __shared__ float cs[kWavesPerBlock][16][17];
    constexpr int SU = 16 / RT;                     // steps per batch of loads
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int i = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.x * 16 * RT;
    const int tok = i < T ? i : T - 1;
    const int kw = cols / kWavesPerBlock;
    const __half * ap[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = row0 + rt * 16 + i < rows ? row0 + rt * 16 + i : rows - 1;
        ap[rt] = W + (size_t)row * cols + wave * kw + g * 8;
    }
    const __half * bp = (lay & 1) ? xn + ((size_t)(wave * kw / 32) * 64 + g * 16 + i) * 8 : xn + (size_t)tok * cols + wave * kw + g * 8;
    const int bstep = (lay & 1) ? 512 : 32;        // halves from one 32-column step's fragment to the next
    pi_f4 acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc[rt] = pi_f4{0.0f, 0.0f, 0.0f, 0.0f};
    const int steps = kw / 32;
    for (int s0 = 0; s0 < steps; s0 += SU) {
        pi_u32x4 a[SU][RT], b[SU];
#pragma unroll
        for (int u = 0; u < SU; ++u)
            if (s0 + u < steps) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) a[u][rt] = pi_ld_stream(ap[rt] + (s0 + u) * 32);
                b[u] = pi_ld16(bp + (s0 + u) * bstep);
            }
#pragma unroll
        for (int u = 0; u < SU; ++u)
            if (s0 + u < steps) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, a[u][rt]), __builtin_bit_cast(pi_h8, b[u]), acc[rt], 0, 0, 0);
            }
    }
    const int rr = threadIdx.x >> 4, t = threadIdx.x & 15;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (rt > 0) __syncthreads();
#pragma unroll
        for (int r = 0; r < 4; ++r) cs[wave][4 * g + r][i] = acc[rt][r];
        __syncthreads();
        const int row = row0 + rt * 16 + rr;
        bool act = false;
        if (row < rows && t < T) {
            float sum = cs[0][rr][t];
#pragma unroll
            for (int w = 1; w < kWavesPerBlock; ++w) sum += cs[w][rr][t];
            const size_t o = (size_t)t * rows + row;
            if (epi == PI_EPI_RELU) sum = fmaxf(sum, 0.0f);
            else if (epi == PI_EPI_ADD) sum = __fadd_rn(sum, add1[o]);
            else if (epi == PI_EPI_ADD2) sum = __fadd_rn(__fadd_rn(sum, add1[o]), add2[o]);
            y[o] = sum;
            if (y16) y16[(lay & 2) ? pi_ol_index(t, row) : o] = __float2half_rn(sum);
            act = !(sum < thr);
        }
        if (row_any) {      // predictor logits: is the row active for at least one token of the step?  (16 lanes = 16 tokens of a row)
            const unsigned long long m = __ballot(act);
            if (t == 0 && row < rows) row_any[row] = ((m >> (16 * (lane >> 4))) & 0xffffull) ? 1 : 0;
        }
    }
}

// The same mat-mul with row-contiguous global reads (cols % 256 == 0).  The MFMA operand layout wants lane l to hold
// row l % 16, which makes a direct load instruction touch 16 rows x 64 B; here a wave instead reads 2 rows x 512 B per
// instruction (8 instructions = its 16 rows x 256 columns), drops the tile into a wave-private LDS buffer with a padded
// row stride (conflict-free both ways) and reads it back in operand layout.  No workgroup barrier is involved: the
// buffer belongs to one wave and LDS operations of a wave complete in order.  Two 256-column tiles of loads are in flight.
constexpr int kGlStride = 512 + 16;               // bytes per LDS row: 256 fp16 + one 16-byte pad
template <int RT, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_t16_lds_f16_kernel(const __half * __restrict__ W, const __half * __restrict__ xn, int T, int rows, int cols,
                                                                  int epi, const float * __restrict__ add1, const float * __restrict__ add2, float * __restrict__ y,
                                                                  __half * __restrict__ y16, float thr, unsigned char * __restrict__ row_any, int lay) {
    __shared__ __align__(16) unsigned char tile[NW][16 * kGlStride];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int i = lane & 15, g = lane >> 4;
    const int lr = lane >> 5, lc = lane & 31;           // load role: row within the pair, 16-byte chunk within the 512-byte row piece
    const int row0 = blockIdx.x * 16 * RT;
    const int tok = i < T ? i : T - 1;
    // the 256-column super-steps of a row are dealt round-robin to the NW waves: wave w takes steps w, w + NW, ...
    const __half * bp = (lay & 1) ? xn + (g * 16 + i) * 8 : xn + (size_t)tok * cols + g * 8;
    const int bstep = (lay & 1) ? 512 : 32;        // halves from one 32-column step's fragment to the next
    unsigned char * mytile = tile[wave];
    pi_f4 acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc[rt] = pi_f4{0.0f, 0.0f, 0.0f, 0.0f};
    const int n_ss = (cols / 256 - wave + NW - 1) / NW;      // super-steps of this wave
    pi_u32x4 ld[2][RT][8];
    auto issue = [&](int buf, int ss) {
        if (ss < n_ss) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    int r = row0 + rt * 16 + 2 * j + lr;
                    r = r < rows ? r : rows - 1;
                    ld[buf][rt][j] = pi_ld_stream(W + (size_t)r * cols + (wave + ss * NW) * 256 + lc * 8);
                }
        }
    };
    issue(0, 0);
    issue(1, 1);
    for (int ss = 0; ss < n_ss; ss += 2) {
#pragma unroll
        for (int buf = 0; buf < 2; ++buf) {
            const int cur = ss + buf;
            if (cur < n_ss) {
                pi_u32x4 b[8];
#pragma unroll
                for (int st = 0; st < 8; ++st) b[st] = pi_ld16(bp + ((wave + cur * NW) * 8 + st) * bstep);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) *reinterpret_cast<pi_u32x4 *>(mytile + (2 * j + lr) * kGlStride + lc * 16) = ld[buf][rt][j];
#pragma unroll
                    for (int st = 0; st < 8; ++st) {
                        const pi_u32x4 a = *reinterpret_cast<const pi_u32x4 *>(mytile + i * kGlStride + (4 * st + g) * 16);
                        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, a), __builtin_bit_cast(pi_h8, b[st]), acc[rt], 0, 0, 0);
                    }
                }
            }
            issue(buf, cur + 2);
        }
    }
    // the waves' accumulator tiles meet in LDS, each in the front of its wave's own (now idle) staging buffer
    auto cs = [&](int w, int r, int c) -> float & { return reinterpret_cast<float *>(tile[w])[r * 17 + c]; };
    const int rr = threadIdx.x >> 4, t = threadIdx.x & 15;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (rt > 0) __syncthreads();
#pragma unroll
        for (int r = 0; r < 4; ++r) cs(wave, 4 * g + r, i) = acc[rt][r];
        __syncthreads();
        if (threadIdx.x >= 256) continue;         // 16 rows x 16 tokens: the first four waves write the tile out
        const int row = row0 + rt * 16 + rr;
        bool act = false;
        if (row < rows && t < T) {
            float sum = cs(0, rr, t);
#pragma unroll
            for (int w = 1; w < NW; ++w) sum += cs(w, rr, t);
            const size_t o = (size_t)t * rows + row;
            if (epi == PI_EPI_RELU) sum = fmaxf(sum, 0.0f);
            else if (epi == PI_EPI_ADD) sum = __fadd_rn(sum, add1[o]);
            else if (epi == PI_EPI_ADD2) sum = __fadd_rn(__fadd_rn(sum, add1[o]), add2[o]);
            y[o] = sum;
            if (y16) y16[(lay & 2) ? pi_ol_index(t, row) : o] = __float2half_rn(sum);
            act = !(sum < thr);
        }
        if (row_any) {
            const unsigned long long m = __ballot(act);
            if (t == 0 && row < rows) row_any[row] = ((m >> (16 * (lane >> 4))) & 0xffffull) ? 1 : 0;
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Prompt chunks of any length on the matrix cores with both operands staged in LDS: y[t][row] = epi(W[row] . xn[t]).
// A workgroup of four waves owns BM weight rows x BN tokens; the reduction dimension advances 64 columns at a time through two
// LDS stages, and two more stages travel in registers as 16-byte global loads (one stage of MFMAs lasts about 0.2 us, less than a
// trip to HBM); one barrier per stage.  Both operands are stored row by row with the reduction dimension contiguous, which is
// the matrix cores' operand layout (eight consecutive columns per lane), so a fragment is one ds_read_b128.  A row is 128 bytes;
// its eight 16-byte pieces are stored at piece ^ (row & 7), so that the 16 rows a quarter wave reads the same piece of, and the
// eight pieces of a row that eight neighbouring lanes write, fall on different banks (the bank-conflict counter reads 0; with
// rows padded to 144 bytes instead it read a third of the LDS cycles).  A wave computes (BM/2) x (BN/2) outputs as 16 x 16
// tiles; per 32-column step it reads BM/32 + BN/32 fragments for (BM/32) * (BN/32) MFMAs.  Workgroups are numbered so that the
// token tiles of one row tile run on the same XCD back to back: the row tile's weights cross HBM once and are re-read from that
// XCD's L2.  cols % 64 == 0; rows and T need not fill the tiles (requests past the edge re-read the last row, results are not
// stored).
// ---------------------------------------------------------------------------------------------------
constexpr int kGtBK = 64;                        // columns per stage
constexpr int kGtRow = kGtBK * 2;                // bytes per LDS row
template <int BM, int BN, int WGM = 2, int WGN = 2>      // output tile and the waves' grid over it (WGM x WGN waves)
__global__ __launch_bounds__(64 * WGM * WGN, (WGM * WGN > 4 ? 1 : BM + BN <= 192 ? 3 : 2)) void gemm_tile_f16_kernel(const __half * __restrict__ W, const __half * __restrict__ xn, int T, int rows, int cols,
                                                                  int nx, int ny, int epi, const float * __restrict__ add1, const float * __restrict__ add2,
                                                                  float * __restrict__ y, __half * __restrict__ y16) {
    constexpr int kThreads = 64 * WGM * WGN;
    constexpr int WM = BM / WGM, WN = BN / WGN, MT = WM / 16, NT = WN / 16;
    constexpr int ACH = BM * kGtBK * 2 / 16 / kThreads, BCH = BN * kGtBK * 2 / 16 / kThreads;  // 16-byte chunks per thread and stage
    static_assert(WM % 16 == 0 && WN % 16 == 0 && ACH * kThreads * 16 == BM * kGtBK * 2 && BCH * kThreads * 16 == BN * kGtBK * 2, "tile does not divide among the waves");
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char * sa = smem;                                     // [2][BM][kGtRow]
    unsigned char * sb = smem + 2 * BM * kGtRow;                   // [2][BN][kGtRow]
    // workgroup -> (row tile, token tile): XCD x takes row tiles x, x + 8, ... and walks each one's token tiles in turn
    const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
    const int tx = (slot / ny) * 8 + xcd, ty = slot % ny;
    if (tx >= nx) return;
    const int row0 = tx * BM, tok0 = ty * BN;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, i = lane & 15, g = lane >> 4;
    const int wm = wave % WGM, wn = wave / WGM;
    auto lds_off = [](int r, int kc) { return r * kGtRow + ((kc ^ (r & 7)) * 16); };
    const __half * ga[ACH]; const __half * gb[BCH];
    int la[ACH], lb[BCH];
#pragma unroll
    for (int j = 0; j < ACH; ++j) {
        const int kc = tid % 8, r = j * (kThreads / 8) + tid / 8;
        const int rr = row0 + r < rows ? row0 + r : rows - 1;
        ga[j] = W + (size_t)rr * cols + kc * 8; la[j] = lds_off(r, kc);
    }
#pragma unroll
    for (int j = 0; j < BCH; ++j) {
        const int kc = tid % 8, r = j * (kThreads / 8) + tid / 8;
        const int tt = tok0 + r < T ? tok0 + r : T - 1;
        gb[j] = xn + (size_t)tt * cols + kc * 8; lb[j] = lds_off(r, kc);
    }
    pi_f4 acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = pi_f4{0.0f, 0.0f, 0.0f, 0.0f};
    // Two column stages travel in registers while a third is being multiplied: stage kt sits in LDS half kt & 1, stages kt + 1 and
    // kt + 2 are in flight (one stage of MFMAs is about 0.2 us, less than a trip to HBM).
    pi_u32x4 ra[2][ACH], rb[2][BCH];
    const int nk = cols / kGtBK;
    auto fetch = [&](auto slot, int kt) {
        constexpr int S = decltype(slot)::value;
#pragma unroll
        for (int j = 0; j < ACH; ++j) ra[S][j] = pi_ld16(ga[j] + (size_t)kt * kGtBK);
#pragma unroll
        for (int j = 0; j < BCH; ++j) rb[S][j] = pi_ld16(gb[j] + (size_t)kt * kGtBK);
    };
    auto stash = [&](auto slot) {              // registers of slot S -> LDS half S
        constexpr int S = decltype(slot)::value;
        unsigned char * na = sa + S * BM * kGtRow; unsigned char * nb = sb + S * BN * kGtRow;
#pragma unroll
        for (int j = 0; j < ACH; ++j) *reinterpret_cast<pi_u32x4 *>(na + la[j]) = ra[S][j];
#pragma unroll
        for (int j = 0; j < BCH; ++j) *reinterpret_cast<pi_u32x4 *>(nb + lb[j]) = rb[S][j];
    };
    const std::integral_constant<int, 0> c0; const std::integral_constant<int, 1> c1;
    // every fetch and stash below is unconditional (past the last stage the last one is fetched again and stashed where nobody
    // reads): the count of loads in flight is then the same on every path, and the waits name exactly the loads they need
    const int last = nk - 1;
    fetch(c0, 0);
    fetch(c1, min(1, last));
    stash(c0);
    fetch(c0, min(2, last));
    __syncthreads();
    // the lane's two pieces (columns 8g.. of each 32-column step) of fragment row i: every 16-row tile starts on a multiple of 8
    const int koff[2] = {(g ^ (i & 7)) * 16, ((4 + g) ^ (i & 7)) * 16};
    const int frag_a = (wm * WM + i) * kGtRow, frag_b = (wn * WN + i) * kGtRow;
    // The fragments of a stage's first 32 columns are read while the previous stage's second 32 are multiplied, those of its second
    // 32 while its first are: every LDS read has a block of MFMAs between its issue and its use.
    pi_u32x4 f0a[MT], f0b[NT], f1a[MT], f1b[NT];
    auto frags = [&](auto par, auto half, pi_u32x4 * fa, pi_u32x4 * fb) {
        constexpr int P = decltype(par)::value, KS = decltype(half)::value;
        const unsigned char * ca = sa + P * BM * kGtRow + frag_a + koff[KS];
        const unsigned char * cb = sb + P * BN * kGtRow + frag_b + koff[KS];
#pragma unroll
        for (int m = 0; m < MT; ++m) fa[m] = *reinterpret_cast<const pi_u32x4 *>(ca + m * 16 * kGtRow);
#pragma unroll
        for (int n = 0; n < NT; ++n) fb[n] = *reinterpret_cast<const pi_u32x4 *>(cb + n * 16 * kGtRow);
    };
    auto mfmas = [&](const pi_u32x4 * fa, const pi_u32x4 * fb) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, fa[m]), __builtin_bit_cast(pi_h8, fb[n]), acc[m][n], 0, 0, 0);
    };
    frags(c0, c0, f0a, f0b);
    auto step = [&](auto par, int kt) {
        constexpr int P = decltype(par)::value;
        const std::integral_constant<int, P ^ 1> other;
        frags(par, c1, f1a, f1b);
        __builtin_amdgcn_sched_barrier(0);
        mfmas(f0a, f0b);
        stash(other);
        fetch(other, min(kt + 3, last));
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        frags(other, c0, f0a, f0b);           // past the last stage: the re-stashed last stage, read and not used
        __builtin_amdgcn_sched_barrier(0);
        mfmas(f1a, f1b);
        __builtin_amdgcn_sched_barrier(0);
    };
    int kt = 0;
    for (; kt + 1 < nk; kt += 2) { step(c0, kt); step(c1, kt + 1); }
    if (kt < nk) step(c0, kt);
    // acc[m][n][r] = y[token tok0 + wn*WN + n*16 + i][row row0 + wm*WM + m*16 + 4g + r]: four consecutive rows per lane
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            const int row = row0 + wm * WM + m * 16 + 4 * g, tok = tok0 + wn * WN + n * 16 + i;
            if (tok >= T || row >= rows) continue;
            const size_t o = (size_t)tok * rows + row;
            float v[4] = {acc[m][n][0], acc[m][n][1], acc[m][n][2], acc[m][n][3]};
            if (row + 4 <= rows && (rows & 3) == 0) {
                if (epi == PI_EPI_RELU) { for (int r = 0; r < 4; ++r) v[r] = fmaxf(v[r], 0.0f); }
                else if (epi >= PI_EPI_ADD) {
                    const float4 a1 = *reinterpret_cast<const float4 *>(add1 + o);
                    v[0] = __fadd_rn(v[0], a1.x); v[1] = __fadd_rn(v[1], a1.y); v[2] = __fadd_rn(v[2], a1.z); v[3] = __fadd_rn(v[3], a1.w);
                    if (epi == PI_EPI_ADD2) {
                        const float4 a2 = *reinterpret_cast<const float4 *>(add2 + o);
                        v[0] = __fadd_rn(v[0], a2.x); v[1] = __fadd_rn(v[1], a2.y); v[2] = __fadd_rn(v[2], a2.z); v[3] = __fadd_rn(v[3], a2.w);
                    }
                }
                *reinterpret_cast<float4 *>(y + o) = make_float4(v[0], v[1], v[2], v[3]);
                if (y16) {
                    __half2 h2[2] = {__floats2half2_rn(v[0], v[1]), __floats2half2_rn(v[2], v[3])};
                    *reinterpret_cast<uint2 *>(y16 + o) = *reinterpret_cast<const uint2 *>(h2);
                }
            } else {
                for (int r = 0; r < 4 && row + r < rows; ++r) {
                    float s = v[r];
                    if (epi == PI_EPI_RELU) s = fmaxf(s, 0.0f);
                    else if (epi == PI_EPI_ADD) s = __fadd_rn(s, add1[o + r]);
                    else if (epi == PI_EPI_ADD2) s = __fadd_rn(__fadd_rn(s, add1[o + r]), add2[o + r]);
                    y[o + r] = s;
                    if (y16) y16[o + r] = __float2half_rn(s);
                }
            }
        }
}

// h16[t][n] = fp16( !(logit[t][n] < thr) ? relu(gate[t][n]) * up[t][n] : 0 )   (relu(up) without a gate): the FFN's hidden vector of a
// prompt chunk from the dense gate/up products; inactive neurons become exact zeros, which add nothing in the down projection
// q8 != 0 (n % 64 == 0 and n_ff % 32 == 0): h goes through Q8_0 blocks of 32 neurons first, as the CPU path's Q4_0 down projection quantises it
// (ggml.c:14465-14618)
__global__ void ffn_h_f16_kernel(const float * __restrict__ up, const float * __restrict__ gate, const float * __restrict__ logits, float thr,
                                 size_t n, __half * __restrict__ h16, int q8) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        float h = 0.0f;
        if (!(logits[i] < thr)) h = gate ? __fmul_rn(fmaxf(gate[i], 0.0f), up[i]) : fmaxf(up[i], 0.0f);
        if (q8) h = q8_block_value(h);
        h16[i] = __float2half_rn(h);
    }
}
// out[c][r] = in[r][c] for an fp16 matrix [rows][cols] (32 x 32 tiles through LDS)
__global__ void transpose_f16_kernel(const __half * __restrict__ in, int rows, int cols, __half * __restrict__ out) {
    __shared__ __half t[32][33];
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    for (int j = threadIdx.y; j < 32; j += blockDim.y) {
        const int r = r0 + j, c = c0 + threadIdx.x;
        if (r < rows && c < cols) t[j][threadIdx.x] = in[(size_t)r * cols + c];
    }
    __syncthreads();
    for (int j = threadIdx.y; j < 32; j += blockDim.y) {
        const int c = c0 + j, r = r0 + threadIdx.x;
        if (r < rows && c < cols) out[(size_t)c * rows + r] = t[threadIdx.x][j];
    }
}

// the operator boundary hands over the predictor's output instead of running the predictor: row_any[n] = some token has !(idx[t][n] < thr)
__global__ void batch_flag_any_kernel(const float * __restrict__ idx, int T, int ff, float thr, unsigned char * __restrict__ row_any) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= ff) return;
    bool any = false;
    for (int t = 0; t < T; ++t) any = any || !(idx[(size_t)t * ff + n] < thr);
    row_any[n] = any ? 1 : 0;
}
// hc[t][u] = fp16(h[t][row_u]) where the row is active for token t, 0 elsewhere and in the padding up to the next multiple of 16
__global__ void batch_gather_h_kernel(const float * __restrict__ h, const float * __restrict__ idx, int T, int ff, float thr,
                                      const int32_t * __restrict__ list, const int32_t * __restrict__ n_union, __half * __restrict__ hc, int hstride) {
    const int n = *n_union, n_pad = (n + 15) & ~15;
    const int t = blockIdx.y;
    for (int u = blockIdx.x * blockDim.x + threadIdx.x; u < n_pad; u += gridDim.x * blockDim.x) {
        float v = 0.0f;
        if (u < n && t < T) { const int row = list[u]; if (!(idx[(size_t)t * ff + row] < thr)) v = h[(size_t)t * ff + row]; }
        hc[(size_t)t * hstride + u] = __float2half_rn(v);
    }
}
__global__ void zero_f32_kernel(float * __restrict__ p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0.0f;
}

// union over the tokens of the step of the predictor's active sets: ascending list of the neurons whose flag the
// predictor's mat-mul epilogue raised (single workgroup: wave ballot per 64 neurons, popcount prefix over the mask words)
__global__ __launch_bounds__(1024) void union_active_kernel(const unsigned char * __restrict__ row_any, int ff,
                                                            uint32_t * __restrict__ words, int32_t * __restrict__ list, int32_t * __restrict__ n_union) {
    __shared__ int sred[17];
    const int lane = threadIdx.x & 63;
    if ((ff & 31) == 0) {
        // a thread takes 16 neurons (one 16-byte load); 16384 neurons per pass
        int base = 0;
        for (int i0 = 0; i0 < ff; i0 += 16 * 1024) {
            const int i = i0 + threadIdx.x * 16;
            uint32_t m = 0;
            if (i < ff) {
                const pi_u32x4 v = *reinterpret_cast<const pi_u32x4 *>(row_any + i);
                const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int k = 0; k < 16; ++k) m |= (((d[k >> 2] >> ((k & 3) * 8)) & 0xFFu) != 0u ? 1u : 0u) << k;
            }
            const uint32_t hi = (uint32_t)__shfl_down((int)m, 1, PI_WAVE);
            if ((threadIdx.x & 1) == 0 && i < ff) words[i >> 5] = m | (hi << 16);
            int tot;
            int off = base + block_exclusive_scan_i32(__popc(m), &tot, sred);
            while (m) { const int b = __ffs(m) - 1; m &= m - 1; list[off++] = i + b; }
            base += tot;
            __syncthreads();
        }
        if (threadIdx.x == 0) *n_union = base;
        return;
    }
    for (int i0 = 0; i0 < ff; i0 += blockDim.x) {
        const int i = i0 + threadIdx.x;
        const bool act = i < ff && row_any[i] != 0;
        const unsigned long long m = __ballot(act);
        if (lane == 0 && i < ff) words[i >> 5] = (uint32_t)m;
        if (lane == 32 && i < ff) words[i >> 5] = (uint32_t)(m >> 32);
    }
    __syncthreads();
    compact_from_words(words, ff, nullptr, 0, list, n_union, sred);
}

// sparse gate/up for the union rows: a workgroup gathers 16 rows of the union list into one MFMA tile (lane l reads
// the row of list entry 16 * tile + l % 16), the four waves split the columns, then
// hc[u][t] = active(t, row_u) ? relu(gate . x_t) * (up . x_t) : 0  (relu(up . x_t) without a gate).
__global__ __launch_bounds__(kBlock) void batch_upgate_f16_kernel(const __half * __restrict__ Wup, const __half * __restrict__ Wgate, int cols,
                                                                  const __half * __restrict__ xn, int T, const float * __restrict__ logits, int ff, float thr,
                                                                  const int32_t * __restrict__ list, const int32_t * __restrict__ n_union,
                                                                  __half * __restrict__ hc, int hstride) {
    // hc[t][u] (token-major, stride hstride) holds h already rounded to fp16: the CPU axpy rounds h before use (ggml.c:14420-14431)
    __shared__ float cu[kWavesPerBlock][16][17], cg[kWavesPerBlock][16][17];
    const int n = *n_union;
    const int u0 = blockIdx.x * 16;
    if (u0 >= n) return;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int i = lane & 15, g = lane >> 4;
    const int row = list[u0 + i < n ? u0 + i : n - 1];
    const int tok = i < T ? i : T - 1;
    const int kw = cols / kWavesPerBlock;
    const size_t aoff = (size_t)row * cols + wave * kw + g * 8;
    const __half * bp = xn + (size_t)tok * cols + wave * kw + g * 8;
    pi_f4 au = {0.0f, 0.0f, 0.0f, 0.0f}, ag = {0.0f, 0.0f, 0.0f, 0.0f};
    const int steps = kw / 32;
    constexpr int UN = 4;
    for (int s0 = 0; s0 < steps; s0 += UN) {
        pi_u32x4 a[UN], c[UN], b[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (s0 + u < steps) {
                a[u] = pi_ld_stream(Wup + aoff + (s0 + u) * 32);
                if (Wgate) c[u] = pi_ld_stream(Wgate + aoff + (s0 + u) * 32);
                b[u] = pi_ld16(bp + (s0 + u) * 32);
            }
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (s0 + u < steps) {
                au = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, a[u]), __builtin_bit_cast(pi_h8, b[u]), au, 0, 0, 0);
                if (Wgate) ag = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, c[u]), __builtin_bit_cast(pi_h8, b[u]), ag, 0, 0, 0);
            }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) { cu[wave][4 * g + r][i] = au[r]; cg[wave][4 * g + r][i] = ag[r]; }
    __syncthreads();
    const int rr = threadIdx.x >> 4, t = threadIdx.x & 15;
    float h = 0.0f;
    if (u0 + rr < n && t < T) {
        const int rrow = list[u0 + rr];
        if (!(logits[(size_t)t * ff + rrow] < thr)) {
            float su = cu[0][rr][t], sg = cg[0][rr][t];
#pragma unroll
            for (int w = 1; w < kWavesPerBlock; ++w) { su += cu[w][rr][t]; sg += cg[w][rr][t]; }
            h = Wgate ? __fmul_rn(fmaxf(sg, 0.0f), su) : fmaxf(su, 0.0f);
        }
    }
    hc[(size_t)t * hstride + u0 + rr] = __float2half_rn(h);
}

// sparse gate/up with row-contiguous reads (cols % 256 == 0): the loader of gemm_t16_lds_f16_kernel applied to the gathered
// rows of the union list; the gate tile and the up tile of a 256-column step pass through the same wave-private LDS buffer.
__global__ __launch_bounds__(kBlock) void batch_upgate_lds_f16_kernel(const __half * __restrict__ Wup, const __half * __restrict__ Wgate, int cols,
                                                                      const __half * __restrict__ xn, int T, const float * __restrict__ logits, int ff, float thr,
                                                                      const int32_t * __restrict__ list, const int32_t * __restrict__ n_union,
                                                                      __half * __restrict__ hc, int hstride, float * __restrict__ raw) {
    // raw != nullptr: the plain product of ONE matrix (Wgate == nullptr) for the operator boundary: raw[t][row] = Wup[row] . xn[t] for
    // the tokens the row is active for and 0 for the others (rows outside the union list are zeroed by the caller); hc is not written
    __shared__ __align__(16) unsigned char tile[kWavesPerBlock][16 * kGlStride];
    __shared__ float cu[kWavesPerBlock][16][17], cg[kWavesPerBlock][16][17];
    const int n = *n_union;
    const int u0 = blockIdx.x * 16;
    if (u0 >= n) return;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int i = lane & 15, g = lane >> 4;
    const int lr = lane >> 5, lc = lane & 31;
    const int tok = i < T ? i : T - 1;
    const __half * bp = xn + (size_t)tok * cols + g * 8;       // super-steps w, w + 4, ... of the row belong to wave w
    unsigned char * mytile = tile[wave];
    size_t roff[8];                                       // row offsets of the 8 load instructions of this lane
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int u = u0 + 2 * j + lr;
        roff[j] = (size_t)list[u < n ? u : n - 1] * cols + wave * 256 + lc * 8;
    }
    const bool has_gate = Wgate != nullptr;
    pi_f4 au = {0.0f, 0.0f, 0.0f, 0.0f}, ag = {0.0f, 0.0f, 0.0f, 0.0f};
    const int n_ss = (cols / 256 - wave + kWavesPerBlock - 1) / kWavesPerBlock;
    pi_u32x4 lu[2][8], lg[2][8];
    auto issue = [&](int buf, int ss) {
        if (ss < n_ss) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                lu[buf][j] = pi_ld_stream(Wup + roff[j] + ss * kWavesPerBlock * 256);
                if (has_gate) lg[buf][j] = pi_ld_stream(Wgate + roff[j] + ss * kWavesPerBlock * 256);
            }
        }
    };
    issue(0, 0);
    issue(1, 1);
    for (int ss = 0; ss < n_ss; ss += 2) {
#pragma unroll
        for (int buf = 0; buf < 2; ++buf) {
            const int cur = ss + buf;
            if (cur < n_ss) {
                pi_u32x4 b[8];
#pragma unroll
                for (int st = 0; st < 8; ++st) b[st] = pi_ld16(bp + (wave + cur * kWavesPerBlock) * 256 + st * 32);
#pragma unroll
                for (int j = 0; j < 8; ++j) *reinterpret_cast<pi_u32x4 *>(mytile + (2 * j + lr) * kGlStride + lc * 16) = lu[buf][j];
#pragma unroll
                for (int st = 0; st < 8; ++st) {
                    const pi_u32x4 a = *reinterpret_cast<const pi_u32x4 *>(mytile + i * kGlStride + (4 * st + g) * 16);
                    au = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, a), __builtin_bit_cast(pi_h8, b[st]), au, 0, 0, 0);
                }
                if (has_gate) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) *reinterpret_cast<pi_u32x4 *>(mytile + (2 * j + lr) * kGlStride + lc * 16) = lg[buf][j];
#pragma unroll
                    for (int st = 0; st < 8; ++st) {
                        const pi_u32x4 a = *reinterpret_cast<const pi_u32x4 *>(mytile + i * kGlStride + (4 * st + g) * 16);
                        ag = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, a), __builtin_bit_cast(pi_h8, b[st]), ag, 0, 0, 0);
                    }
                }
            }
            issue(buf, cur + 2);
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) { cu[wave][4 * g + r][i] = au[r]; cg[wave][4 * g + r][i] = ag[r]; }
    __syncthreads();
    const int rr = threadIdx.x >> 4, t = threadIdx.x & 15;
    float h = 0.0f, su = 0.0f;
    int rrow = -1;
    if (u0 + rr < n && t < T) {
        rrow = list[u0 + rr];
        if (!(logits[(size_t)t * ff + rrow] < thr)) {
            float sg = cg[0][rr][t];
            su = cu[0][rr][t];
#pragma unroll
            for (int w = 1; w < kWavesPerBlock; ++w) { su += cu[w][rr][t]; sg += cg[w][rr][t]; }
            h = has_gate ? __fmul_rn(fmaxf(sg, 0.0f), su) : fmaxf(su, 0.0f);
        }
    }
    if (raw) { if (rrow >= 0) raw[(size_t)t * ff + rrow] = su; }
    else hc[(size_t)t * hstride + u0 + rr] = __float2half_rn(h);
}

// The same product with the union rows dealt evenly to the compute units.  What bounds these kernels is the unit that has to pull
// the most bytes (a unit sustains about 1/256 of the chip's rate, weights and activations alike): with one workgroup per 16 union
// rows, 5720 rows are 358 workgroups, 102 units hold two of them and set the pace, and every workgroup pulls the step's whole
// activation matrix for its 16 rows.  Here the grid is one workgroup per unit and workgroup b owns union entries [b R, (b + 1) R)
// with R = n / grid rounded up to even (2 <= R <= 32: two MFMA row tiles that share the activation fragments; beyond 32 * grid
// union rows a workgroup walks several such chunks).  Eight waves split the 128-column super-steps of the rows (w, w + 8, ...);
// a wave reads 4 rows x 256 B per instruction, has two super-steps in flight and passes the tiles through its own LDS buffer as
// batch_upgate_lds_f16_kernel does.  Every load is unconditional, so that the in-order counter gives exact waits: a lane whose row
// lies behind the chunk's end reads what another lane of the same instruction reads (one request), or the chunk's first 16 bytes.
constexpr int kUbWaves = 8, kUbBlock = kUbWaves * PI_WAVE, kUbRows = 32, kUbStep = 128, kUbStride = kUbStep * 2 + 16;
template <bool GATE>
__global__ __launch_bounds__(kUbBlock, 1) void batch_upgate_bal_f16_kernel(const __half * __restrict__ Wup, const __half * __restrict__ Wgate, int cols,
                                                                           const __half * __restrict__ xn, int T, const float * __restrict__ logits, int ff, float thr,
                                                                           int32_t * __restrict__ list, int32_t * __restrict__ n_union,
                                                                           __half * __restrict__ hc, int hstride, int xol, const unsigned char * __restrict__ row_any) {
    // xol != 0: xn in the operand layout (pi_ol_index).
    // row_any != nullptr (ff <= 32 flags x 512 threads, ff % 16 == 0): the union list is made HERE from the per-neuron flags the
    // predictor's mat-mul left (a byte each, 0 or 1) instead of by a launch of its own: every workgroup counts all the flags (a thread
    // takes 32, a scan over the workgroup gives its rank), picks the rows of its own chunk out of them and writes them to `list` for the
    // down projection; workgroup 0 writes the count.  The flags are requested where the list entries would have been, so the
    // launch is no deeper; at 13824 neurons it grows by 3 us (256 workgroups reading the same 13.8 KB) and the list kernel's 4.8 us go.
    __shared__ __align__(16) unsigned char tile[kUbWaves][16 * kUbStride];
    __shared__ float cu[kUbWaves][kUbRows][17], cg[GATE ? kUbWaves : 1][kUbRows][17];
    __shared__ int s_wtot[kUbWaves], s_rows[kUbRows];
    int n, fl_excl = 0, fl_cnt = 0;
    uint32_t fl[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};                 // this thread's 32 flags: neurons 32 t .. 32 t + 31
    if (row_any) {
        const int f0 = (int)threadIdx.x * 32;
#pragma unroll
        for (int q = 0; q < 2; ++q)
            if (f0 + 16 * q < ff) {
                const pi_u32x4 v = *reinterpret_cast<const pi_u32x4 *>(row_any + f0 + 16 * q);
                fl[4 * q] = v.x; fl[4 * q + 1] = v.y; fl[4 * q + 2] = v.z; fl[4 * q + 3] = v.w;
            }
#pragma unroll
        for (int q = 0; q < 8; ++q) fl_cnt += __popc(fl[q] & 0x01010101u);
        int incl = fl_cnt;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { const int v = __shfl_up(incl, o, PI_WAVE); if ((int)(threadIdx.x & 63) >= o) incl += v; }
        if ((threadIdx.x & 63) == 63) s_wtot[threadIdx.x >> 6] = incl;
        __syncthreads();
        n = 0;
#pragma unroll
        for (int w = 0; w < kUbWaves; ++w) { if (w < (int)(threadIdx.x >> 6)) fl_excl += s_wtot[w]; n += s_wtot[w]; }
        fl_excl += incl - fl_cnt;
        if (blockIdx.x == 0 && threadIdx.x == 0) *n_union = n;
    } else {
        n = *n_union;
    }
    const int G = gridDim.x;
    int R = (n + G - 1) / G;
    R = (R + 1) & ~1;
    R = R < 2 ? 2 : R > kUbRows ? kUbRows : R;
    const int n_chunks = (n + R - 1) / R;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int i = lane & 15, g = lane >> 4;                        // MFMA role: row (token) i, k group g
    const int lr = lane >> 4, lc = lane & 15;                      // load role: row within the instruction's four, 16-byte piece of the 256-byte row piece
    const int tok = i < T ? i : T - 1;
    const char * bp = reinterpret_cast<const char *>(xol ? xn + (g * 16 + i) * 8 : xn + (size_t)tok * cols + g * 8);
    const int bs_step = xol ? 4096 : kUbStep * 2, bs_frag = xol ? 1024 : 64;      // bytes from a 128-column step to the next, and between its four 32-column fragments
    unsigned char * mytile = tile[wave];
    const int n_steps = cols / kUbStep;
    const int n_ss = (n_steps - wave + kUbWaves - 1) / kUbWaves;   // super-steps wave, wave + 8, ... of this wave
    for (int c = blockIdx.x; c < n_chunks; c += G) {
        const int u0 = c * R;
        const int Rc = n - u0 < R ? n - u0 : R;                    // rows of this chunk (the list's last chunk may be short, and odd)
        if (row_any) {                                             // this chunk's rows out of the flags: ranks u0 .. u0 + Rc - 1
            if (fl_excl < u0 + Rc && fl_excl + fl_cnt > u0) {
                int k = fl_excl;
#pragma unroll
                for (int q = 0; q < 8; ++q)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if ((fl[q] >> (8 * e)) & 1u) {
                            if (k >= u0 && k < u0 + Rc) { const int row = (int)threadIdx.x * 32 + 4 * q + e; s_rows[k - u0] = row; list[k] = row; }
                            ++k;
                        }
            }
            __syncthreads();
        }
        uint32_t roff[8];                                          // byte offsets of this lane's 8 load instructions (< 2^32: the launcher's test)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int k = 4 * j + lr;
            const int kk = k < Rc ? k : 4 * j < Rc ? 4 * j : 0;
            const int row = row_any ? s_rows[kk] : list[u0 + kk];
            roff[j] = ((uint32_t)row * (uint32_t)cols + (4 * j < Rc ? lc * 8 : 0)) * 2;
        }
        pi_f4 au[2], ag[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) au[t] = ag[t] = pi_f4{0.0f, 0.0f, 0.0f, 0.0f};
        // The weights of two super-steps are in flight; the activations of a super-step are requested when the previous one has been
        // multiplied, BEFORE the weights that replace it (requested after them, the wait for the activations would drain them).
        pi_u32x4 lu[2][8], lg[2][8], bb[4];
        // workgroup b starts its walk over the columns b super-steps further on (and wraps): the units run in step, and all of them
        // asking for the same kilobytes of the activations at the same time queue up on one L2 channel
        const int rot0 = n_ss > 0 ? (int)(blockIdx.x % (unsigned)n_ss) : 0;
        auto rot = [&](int s) { const int v = s + rot0; return v >= n_ss ? v - n_ss : v; };
        auto issue_b = [&](int s) {
            const size_t so = (size_t)(wave + rot(s < n_ss ? s : n_ss - 1) * kUbWaves) * bs_step;
#pragma unroll
            for (int st = 0; st < 4; ++st) bb[st] = pi_ld16(bp + so + st * bs_frag);
        };
        auto issue = [&](int buf, int s) {                         // a super-step behind the wave's last reads the last one again
            const size_t so = (size_t)(wave + rot(s < n_ss ? s : n_ss - 1) * kUbWaves) * (kUbStep * 2);
            const char * wu = reinterpret_cast<const char *>(Wup) + so, * wg = reinterpret_cast<const char *>(Wgate) + so;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                lu[buf][j] = pi_ld_stream(wu + roff[j]);
                if (GATE) lg[buf][j] = pi_ld_stream(wg + roff[j]);
            }
        };
        auto consume = [&](int buf) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {                          // (the second tile also where the chunk has 16 rows or fewer: straight-line code keeps the waits exact)
                {
#pragma unroll
                    for (int j = 0; j < 4; ++j) *reinterpret_cast<pi_u32x4 *>(mytile + (4 * j + lr) * kUbStride + lc * 16) = lu[buf][4 * t + j];
#pragma unroll
                    for (int st = 0; st < 4; ++st) {
                        const pi_u32x4 a = *reinterpret_cast<const pi_u32x4 *>(mytile + i * kUbStride + (4 * st + g) * 16);
                        au[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, a), __builtin_bit_cast(pi_h8, bb[st]), au[t], 0, 0, 0);
                    }
                    if (GATE) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) *reinterpret_cast<pi_u32x4 *>(mytile + (4 * j + lr) * kUbStride + lc * 16) = lg[buf][4 * t + j];
#pragma unroll
                        for (int st = 0; st < 4; ++st) {
                            const pi_u32x4 a = *reinterpret_cast<const pi_u32x4 *>(mytile + i * kUbStride + (4 * st + g) * 16);
                            ag[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(pi_h8, a), __builtin_bit_cast(pi_h8, bb[st]), ag[t], 0, 0, 0);
                        }
                    }
                }
            }
        };
        if (n_ss > 0) {
            issue(0, 0);
            __builtin_amdgcn_sched_barrier(0);
            issue_b(0);
            __builtin_amdgcn_sched_barrier(0);
            issue(1, 1);
            __builtin_amdgcn_sched_barrier(0);
            int s = 0;
            for (; s + 2 < n_ss; s += 2) {        // (the scheduling barriers keep a phase's loads from rising into the MFMAs that free their registers)
                consume(0); __builtin_amdgcn_sched_barrier(0); issue_b(s + 1); __builtin_amdgcn_sched_barrier(0); issue(0, s + 2); __builtin_amdgcn_sched_barrier(0);
                consume(1); __builtin_amdgcn_sched_barrier(0); issue_b(s + 2); __builtin_amdgcn_sched_barrier(0); issue(1, s + 3); __builtin_amdgcn_sched_barrier(0);
            }
            consume(0);
            if (s + 1 < n_ss) { __builtin_amdgcn_sched_barrier(0); issue_b(s + 1); consume(1); }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) { cu[wave][16 * t + 4 * g + r][i] = au[t][r]; if (GATE) cg[wave][16 * t + 4 * g + r][i] = ag[t][r]; }
        __syncthreads();
        const int rr = threadIdx.x >> 4, t = threadIdx.x & 15;     // 512 threads: 32 rows x 16 tokens
        if (rr < Rc) {
            float h = 0.0f;
            if (t < T && !(logits[(size_t)t * ff + (row_any ? s_rows[rr] : list[u0 + rr])] < thr)) {
                float su = cu[0][rr][t], sg = GATE ? cg[0][rr][t] : 0.0f;
#pragma unroll
                for (int w = 1; w < kUbWaves; ++w) { su += cu[w][rr][t]; if (GATE) sg += cg[w][rr][t]; }
                h = GATE ? __fmul_rn(fmaxf(sg, 0.0f), su) : fmaxf(su, 0.0f);
            }
            hc[(size_t)t * hstride + u0 + rr] = __float2half_rn(h);
        }
        // the down projection reads h in steps of 16 union entries: zeros behind the list's end
        if (c == n_chunks - 1 && rr < ((n + 15) & ~15) - n) hc[(size_t)t * hstride + n + rr] = __float2half_rn(0.0f);
        __syncthreads();                                           // cu / cg are reused by the next chunk
    }
}

// sparse down projection for the step: partial[g][t][c] = sum over the union entries of row group g of hc[u][t] * down[row_u][c].
// A workgroup of 8 waves owns 256 columns (4 per lane, one 8-byte load per row) and one of G row groups; wave w of group g
// walks entries u = 8g + w, + 8G, ...: a whole wave works on ONE row at a time, so the row's 16 h values are wave-uniform
// and arrive through the scalar cache.  The 8 waves then add their 16 x 256 tiles into LDS one after the other (fixed order).
constexpr int kBaGroups = 8;
constexpr int kBaBlock = 512;
constexpr int kBaWaves = kBaBlock / PI_WAVE;
constexpr int kBaTile = 256;
__global__ __launch_bounds__(kBaBlock) void batch_axpy_f16_kernel(const __half * __restrict__ Wd, int cols, const __half * __restrict__ hc, int hstride,
                                                                  const int32_t * __restrict__ list, const int32_t * __restrict__ n_union,
                                                                  float * __restrict__ partial) {
    __shared__ float tile[kBtMaxT][kBaTile];
    const int n = *n_union;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int c0 = blockIdx.x * kBaTile + lane * 4;
    const int stride = kBaGroups * kBaWaves;
    float acc[kBtMaxT][4];
#pragma unroll
    for (int t = 0; t < kBtMaxT; ++t)
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[t][k] = 0.0f;
    constexpr int UN = 8;
    for (int u0 = blockIdx.y * kBaWaves + wave; u0 < n; u0 += stride * UN) {
        pi_u32x2 w[UN];
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            const int u = u0 + j * stride;
            w[j] = u < n ? __builtin_nontemporal_load(reinterpret_cast<const pi_u32x2 *>(Wd + (size_t)list[u] * cols + c0)) : pi_u32x2{0u, 0u};
        }
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            const int u = u0 + j * stride;
            if (u < n) {
                const __half2 * hw = reinterpret_cast<const __half2 *>(&w[j]);
                const float2 w01 = __half22float2(hw[0]), w23 = __half22float2(hw[1]);
#pragma unroll
                for (int t = 0; t < kBtMaxT; ++t) {
                    const float h = __half2float(hc[(size_t)t * hstride + u]);
                    acc[t][0] = fmaf(w01.x, h, acc[t][0]); acc[t][1] = fmaf(w01.y, h, acc[t][1]);
                    acc[t][2] = fmaf(w23.x, h, acc[t][2]); acc[t][3] = fmaf(w23.y, h, acc[t][3]);
                }
            }
        }
    }
    for (int w = 0; w < kBaWaves; ++w) {
        if (wave == w) {
#pragma unroll
            for (int t = 0; t < kBtMaxT; ++t) {
                float4 * p = reinterpret_cast<float4 *>(&tile[t][lane * 4]);
                float4 v = w == 0 ? make_float4(0.0f, 0.0f, 0.0f, 0.0f) : *p;
                v.x += acc[t][0]; v.y += acc[t][1]; v.z += acc[t][2]; v.w += acc[t][3];
                *p = v;
            }
        }
        __syncthreads();
    }
    for (int i = threadIdx.x; i < kBtMaxT * kBaTile / 4; i += kBaBlock) {
        const int t = i / (kBaTile / 4), c4 = i % (kBaTile / 4);
        *reinterpret_cast<float4 *>(partial + ((size_t)blockIdx.y * kBtMaxT + t) * cols + blockIdx.x * kBaTile + c4 * 4) =
            *reinterpret_cast<const float4 *>(&tile[t][c4 * 4]);
    }
}

// The down projection on the matrix cores (cols % 256 == 0).  out[t][c] = sum_u h[t][u] * down[row_u][c] has the union rows as its
// reduction dimension, along which the weight matrix is NOT contiguous, while the B operand of v_mfma_f32_16x16x16_f16 wants four
// consecutive k (rows) of ONE column per lane.  The operand's column index is free to name any column, though: lane (i, g) loads
// 16 bytes = columns 8 i .. 8 i + 7 of rows 4 g .. 4 g + 3 (per instruction 4 rows x 256 contiguous bytes), and the e-th of eight
// MFMAs takes column 8 i + e of those four rows, two v_perm_b32 per operand and no trip through LDS; accumulator e then holds
// out[4 g + r][8 i + e], eight consecutive columns per lane for the store.  The A fragment is 4 consecutive entries of h[t][.]
// (one 8-byte load from the token-major h).
// grid = (cols / 512, G row groups), two waves a workgroup; a wave owns 256 columns (two 128-column halves) and walks the 16-row
// steps g, g + G, ...; partial[g][t][c] is summed by batch_reduce_kernel.  At 5120 columns and 5720 union rows a launch takes
// 15.5 us for 58.6 MB of rows and 10.5 MB of partial sums; four waves a workgroup, or 250 workgroups held one to a compute
// unit, take the same time; one wave a workgroup with 128 columns and eight steps in flight takes 18 us, and so do eight waves a
// workgroup (one workgroup per unit, four waves per column half adding their tiles through LDS).
typedef _Float16 pi_h4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(kBlock) void batch_axpy_mfma_f16_kernel(const __half * __restrict__ Wd, int cols, const __half * __restrict__ hc, int hstride,
                                                                     const int32_t * __restrict__ list, const int32_t * __restrict__ n_union,
                                                                     float * __restrict__ partial) {
    const int n = *n_union;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int i = lane & 15, g = lane >> 4;
    const int c0 = (blockIdx.x * (blockDim.x >> 6) + wave) * 256;
    if (c0 >= cols) return;                               // no workgroup barrier below: waves are independent
    pi_f4 acc[16];
#pragma unroll
    for (int ct = 0; ct < 16; ++ct) acc[ct] = pi_f4{0.0f, 0.0f, 0.0f, 0.0f};
    const int n_steps = (n + 15) / 16;
    // Four 16-row steps of loads in flight per wave: a wave is alone on its SIMD most of the time, so what it has requested is all
    // that hides the trip to memory.  Two things keep the requests in flight: the row numbers come through the scalar unit (sixteen
    // uniform loads and a select on g; a vector load of them would sit between the weight loads in the in-order counter and every
    // wait for a row number would drain the weights before it), and every round issues all of its loads unconditionally (steps
    // behind the group's last re-read that step, a cache hit), so the wait before a step's first MFMA is an exact count.
    constexpr int NB = 4;
    const int G = gridDim.y;
    const int my_steps = (n_steps - (int)blockIdx.y + G - 1) / G;                           // steps blockIdx.y, + G, ... of this group
    pi_u32x4 ld[NB][8];
    pi_u32x2 af[NB];
    // the 16 row numbers of the NEXT step to be requested (steps are requested in order): they are asked for right behind a step's
    // weight loads and have arrived when the next step's addresses are made, instead of holding every request up for a trip of
    // their own
    int rn[16];
    auto fetch_rows = [&](int s) {
        const int u0 = ((int)blockIdx.y + (s < my_steps ? s : my_steps - 1) * G) * 16;
#pragma unroll
        for (int k = 0; k < 16; ++k) rn[k] = list[u0 + k < n ? u0 + k : n - 1];
    };
    auto issue = [&](int buf, int s) {
        const int u0 = ((int)blockIdx.y + (s < my_steps ? s : my_steps - 1) * G) * 16;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            // (readfirstlane keeps the row numbers on the scalar unit, ahead of the select)
            const int r0 = __builtin_amdgcn_readfirstlane(rn[r]);
            const int r1 = __builtin_amdgcn_readfirstlane(rn[4 + r]);
            const int r2 = __builtin_amdgcn_readfirstlane(rn[8 + r]);
            const int r3 = __builtin_amdgcn_readfirstlane(rn[12 + r]);
            const __half * wp = Wd + (size_t)(g == 0 ? r0 : g == 1 ? r1 : g == 2 ? r2 : r3) * cols + c0 + 8 * i;
            ld[buf][2 * r]     = pi_ld_stream(wp);
            ld[buf][2 * r + 1] = pi_ld_stream(wp + 128);
        }
        af[buf] = *reinterpret_cast<const pi_u32x2 *>(hc + (size_t)i * hstride + u0 + 4 * g);      // zeros beyond n (written by the gate/up kernel)
        fetch_rows(s + 1);
    };
    auto consume = [&](int buf) {
        const pi_h4 a = __builtin_bit_cast(pi_h4, af[buf]);
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                const uint32_t w0 = ld[buf][half][e2], w1 = ld[buf][2 + half][e2], w2 = ld[buf][4 + half][e2], w3 = ld[buf][6 + half][e2];
                const pi_u32x2 lo = {__builtin_amdgcn_perm(w1, w0, 0x05040100u), __builtin_amdgcn_perm(w3, w2, 0x05040100u)};
                const pi_u32x2 hi = {__builtin_amdgcn_perm(w1, w0, 0x07060302u), __builtin_amdgcn_perm(w3, w2, 0x07060302u)};
                acc[half * 8 + 2 * e2]     = __builtin_amdgcn_mfma_f32_16x16x16f16(a, __builtin_bit_cast(pi_h4, lo), acc[half * 8 + 2 * e2], 0, 0, 0);
                acc[half * 8 + 2 * e2 + 1] = __builtin_amdgcn_mfma_f32_16x16x16f16(a, __builtin_bit_cast(pi_h4, hi), acc[half * 8 + 2 * e2 + 1], 0, 0, 0);
            }
    };
    if (my_steps > 0) {
        fetch_rows(0);
#pragma unroll
        for (int buf = 0; buf < NB; ++buf) issue(buf, buf);
        int s = 0;
        for (; s + NB < my_steps; s += NB) {
#pragma unroll
            for (int buf = 0; buf < NB; ++buf) { consume(buf); issue(buf, s + buf + NB); }
        }
#pragma unroll
        for (int buf = 0; buf < NB; ++buf)
            if (s + buf < my_steps) consume(buf);
    }
    // accumulator e of a half, lane (i, g): tokens 4 g .. 4 g + 3 of column 8 i + e of the half
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float * dst = partial + ((size_t)blockIdx.y * kBtMaxT + 4 * g + r) * cols + c0 + half * 128 + 8 * i;
            *reinterpret_cast<float4 *>(dst)     = make_float4(acc[half * 8][r], acc[half * 8 + 1][r], acc[half * 8 + 2][r], acc[half * 8 + 3][r]);
            *reinterpret_cast<float4 *>(dst + 4) = make_float4(acc[half * 8 + 4][r], acc[half * 8 + 5][r], acc[half * 8 + 6][r], acc[half * 8 + 7][r]);
        }
}

__global__ __launch_bounds__(kBlock) void batch_reduce_kernel(const float * __restrict__ partial, int n_groups, int T, int cols, int epi,
                                                              const float * __restrict__ add1, const float * __restrict__ add2, float * __restrict__ out) {
    const int idx = (blockIdx.x * blockDim.x + threadIdx.x) * 4;          // cols % 4 == 0: four columns of one token
    if (idx >= T * cols) return;
    const int t = idx / cols, c = idx - t * cols;
    const size_t gstride = (size_t)kBtMaxT * cols;
    const float * p = partial + (size_t)t * cols + c;
    // the residual operands are requested with the first partial sums, and 16 partial sums travel together: two trips to memory
    // for 32 groups (the sums are added in group order whatever the batching)
    float4 a1 = make_float4(0.0f, 0.0f, 0.0f, 0.0f), a2 = a1;
    if (epi >= PI_EPI_ADD) a1 = *reinterpret_cast<const float4 *>(add1 + idx);
    if (epi == PI_EPI_ADD2) a2 = *reinterpret_cast<const float4 *>(add2 + idx);
    float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    int g0 = 0;
    for (; g0 + 16 <= n_groups; g0 += 16) {
        float4 v[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = *reinterpret_cast<const float4 *>(p + (size_t)(g0 + j) * gstride);
#pragma unroll
        for (int j = 0; j < 16; ++j) { sum.x += v[j].x; sum.y += v[j].y; sum.z += v[j].z; sum.w += v[j].w; }
    }
    for (; g0 < n_groups; ++g0) {
        const float4 v = *reinterpret_cast<const float4 *>(p + (size_t)g0 * gstride);
        sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
    if (epi >= PI_EPI_ADD) { sum.x = __fadd_rn(sum.x, a1.x); sum.y = __fadd_rn(sum.y, a1.y); sum.z = __fadd_rn(sum.z, a1.z); sum.w = __fadd_rn(sum.w, a1.w); }
    if (epi == PI_EPI_ADD2) { sum.x = __fadd_rn(sum.x, a2.x); sum.y = __fadd_rn(sum.y, a2.y); sum.z = __fadd_rn(sum.z, a2.z); sum.w = __fadd_rn(sum.w, a2.w); }
    *reinterpret_cast<float4 *>(out + idx) = sum;
}

__global__ void embed_f16_batch_kernel(const __half * __restrict__ table, int cols, const int32_t * __restrict__ tokens, float * __restrict__ x) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c < cols) x[(size_t)blockIdx.y * cols + c] = __half2float(table[(size_t)tokens[blockIdx.y] * cols + c]);
}

// greedy choice per sequence (first maximum wins, llama.cpp:8617-8631), then the sequence's state moves on: its next token,
// its position + 1; workgroup 0 also advances the step counter after recording the step's tokens.
__global__ __launch_bounds__(1024) void argmax_batch_kernel(const float * __restrict__ logits, int n, int T, int32_t * __restrict__ tokens,
                                                            int32_t * __restrict__ positions, int32_t * __restrict__ step,
                                                            int32_t * __restrict__ out_tokens, int max_steps) {
    __shared__ float bv[16];
    __shared__ int   bi[16];
    const int t = blockIdx.x;
    const float * lg = logits + (size_t)t * n;
    float best = -INFINITY; int idx = 0x7fffffff;
    if (n % 4 == 0 && ((uintptr_t)lg & 15) == 0) {
        // eight 16-byte loads per thread requested together (a row of 32 000 logits is one such round: one trip to memory instead
        // of one per element); a thread's indices ascend, so the strict comparison keeps its first maximum
        const float4 * lg4 = reinterpret_cast<const float4 *>(lg);
        const int n4 = n / 4;
        for (int i0 = threadIdx.x; i0 < n4; i0 += 8 * (int)blockDim.x) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i4 = i0 + u * (int)blockDim.x;
                v[u] = lg4[i4 < n4 ? i4 : n4 - 1];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i4 = i0 + u * (int)blockDim.x;
                if (i4 < n4) {
                    if (v[u].x > best) { best = v[u].x; idx = 4 * i4; }
                    if (v[u].y > best) { best = v[u].y; idx = 4 * i4 + 1; }
                    if (v[u].z > best) { best = v[u].z; idx = 4 * i4 + 2; }
                    if (v[u].w > best) { best = v[u].w; idx = 4 * i4 + 3; }
                }
            }
        }
    } else {
        for (int i = threadIdx.x; i < n; i += blockDim.x) { const float v = lg[i]; if (v > best) { best = v; idx = i; } }
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, PI_WAVE); const int oi = __shfl_xor(idx, o, PI_WAVE);
        if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { bv[wave] = best; bi[wave] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w) if (bv[w] > best || (bv[w] == best && bi[w] < idx)) { best = bv[w]; idx = bi[w]; }
        if (idx >= n) idx = 0;             // no logit compared greater than -inf (all NaN or -inf): a valid row for the next embedding lookup
        tokens[t] = idx;
        if (positions) positions[t] += 1;
        const int s = step ? *step : 0;
        if (out_tokens && s < max_steps) out_tokens[(size_t)s * T + t] = idx;
    }
}

__global__ void step_advance_kernel(int32_t * step) { if (threadIdx.x == 0) *step += 1; }

}  // namespace

namespace pi {
void launch_union_active(const unsigned char * row_any, int ff, uint32_t * words, int32_t * union_rows, int32_t * n_union, hipStream_t st) {
    hipLaunchKernelGGL(union_active_kernel, dim3(1), dim3(1024), 0, st, row_any, ff, words, union_rows, n_union);
}
void launch_batch_reduce(const float * partial, int n_groups, int T, int cols, int epilogue, const float * add1, const float * add2, float * out, hipStream_t st) {
    hipLaunchKernelGGL(batch_reduce_kernel, dim3((T * cols / 4 + kBlock - 1) / kBlock), dim3(kBlock), 0, st, partial, n_groups, T, cols, epilogue, add1, add2, out);
}
}  // namespace pi

extern "C" {

int pi_k_norm_round_f16(const float * x, int T, int cols, const pi_norm * norm, void * out_f16, void * out_plain_f16, pi_stream_t stream) {
    if (!x || !out_f16 || T <= 0 || cols <= 0) return pi::fail(PI_E_ARG, "pi_k_norm_round_f16: bad arguments");
    hipLaunchKernelGGL(norm_round_f16_kernel, dim3(T), dim3(1024), 0, (hipStream_t)stream, x, cols, to_norm(norm), (__half *)out_f16, (__half *)out_plain_f16, 0, 0);
    return pi::check_launch("pi_k_norm_round_f16");
}

int pi_k_norm_round_f16_ol(const float * x, int T, int cols, const pi_norm * norm, void * out_ol, void * out_plain_ol, pi_stream_t stream) {
    if (!x || !out_ol || T <= 0 || T > kBtMaxT || cols <= 0 || cols % 8) return pi::fail(PI_E_ARG, "pi_k_norm_round_f16_ol: 1 <= T <= 16 and cols % 8 == 0 required");
    hipLaunchKernelGGL(norm_round_f16_kernel, dim3(T), dim3(1024), 0, (hipStream_t)stream, x, cols, to_norm(norm), (__half *)out_ol, (__half *)out_plain_ol, 0, 1);
    return pi::check_launch("pi_k_norm_round_f16_ol");
}

int pi_k_norm_q8_round_f16(const float * x, int T, int cols, const pi_norm * norm, void * out_f16, void * out_plain_f16, pi_stream_t stream) {
    if (!x || !out_f16 || T <= 0 || cols <= 0 || cols % 32 || cols > 8 * 1024) return pi::fail(PI_E_ARG, "pi_k_norm_q8_round_f16: cols must be a multiple of 32, at most 8192");
    hipLaunchKernelGGL(norm_round_f16_kernel, dim3(T), dim3(1024), 0, (hipStream_t)stream, x, cols, to_norm(norm), (__half *)out_f16, (__half *)out_plain_f16, 1, 0);
    return pi::check_launch("pi_k_norm_q8_round_f16");
}

// lay bit 0: xn_f16 in the operand layout of the step's activations (pi_ol_index), bit 1: y_f16 written in it
static int gemm_launch(const char * who, const void * W, int rows, int cols, const void * xn_f16, int T, int epilogue, const float * add1, const float * add2,
                       float * y, void * y_f16, float thr, unsigned char * row_any, pi_stream_t stream, int lay = 0) {
    if (!W || !xn_f16 || !y || rows <= 0) return pi::fail(PI_E_ARG, who);
    if (T < 1 || T > kBtMaxT || cols <= 0 || cols % 128) return pi::fail(PI_E_ARG, "batched mat-mul: 1 <= T <= 16 and cols % 128 == 0 required");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "batched mat-mul: bad epilogue arguments");
    // row tiles per wave: enough workgroups to fill the chip first, then as few reads of the activations as possible
    const int rt = rows >= 16384 ? 4 : rows >= 5120 ? 2 : 1;      // (two tiles already at 5120 rows: the activations, re-read per row tile, are what limits one tile per wave)
#define PI_GEMM_T16(RT) hipLaunchKernelGGL((gemm_t16_f16_kernel<RT>), dim3((rows + 16 * RT - 1) / (16 * RT)), dim3(kBlock), 0, (hipStream_t)stream, \
                       (const __half *)W, (const __half *)xn_f16, T, rows, cols, epilogue, add1, add2, y, (__half *)y_f16, thr, row_any, lay)
#define PI_GEMM_LDS(RT, NW) hipLaunchKernelGGL((gemm_t16_lds_f16_kernel<RT, NW>), dim3((rows + 16 * RT - 1) / (16 * RT)), dim3(64 * NW), 0, (hipStream_t)stream, \
                       (const __half *)W, (const __half *)xn_f16, T, rows, cols, epilogue, add1, add2, y, (__half *)y_f16, thr, row_any, lay)
    if (cols % 256 == 0) {
        // waves per workgroup: when every workgroup has a compute unit to itself (at most one per unit), eight waves keep twice
        // the loads in flight per unit; with more workgroups than units the chip is full with four
        const int rtl = rt >= 2 ? 2 : 1;
        const bool wide = (rows + 16 * rtl - 1) / (16 * rtl) <= pi::compute_units();
        if (rtl == 2) { if (wide) PI_GEMM_LDS(2, 8); else PI_GEMM_LDS(2, 4); }
        else { if (wide) PI_GEMM_LDS(1, 8); else PI_GEMM_LDS(1, 4); }
    }
    else if (rt == 4) PI_GEMM_T16(4); else if (rt == 2) PI_GEMM_T16(2); else PI_GEMM_T16(1);
#undef PI_GEMM_LDS
#undef PI_GEMM_T16
    return pi::check_launch(who);
}

int pi_k_gemm_f16(const void * W, int rows, int cols, const void * xn_f16, int T, int epilogue, const float * add1, const float * add2,
                  float * y, void * y_f16, pi_stream_t stream) {
    return gemm_launch("pi_k_gemm_f16", W, rows, cols, xn_f16, T, epilogue, add1, add2, y, y_f16, 0.0f, nullptr, stream);
}

int pi_k_gemm_f16_ol(const void * W, int rows, int cols, const void * xn_ol, int T, int epilogue, const float * add1, const float * add2,
                     float * y, void * y_ol, pi_stream_t stream) {
    if (y_ol && rows % 8) return pi::fail(PI_E_ARG, "pi_k_gemm_f16_ol: rows % 8 == 0 required for the fp16 copy in the operand layout");
    return gemm_launch("pi_k_gemm_f16_ol", W, rows, cols, xn_ol, T, epilogue, add1, add2, y, y_ol, 0.0f, nullptr, stream, 3);
}

// Output tiles the kernel is built for (weight rows x tokens per workgroup); the first two run eight waves, one workgroup per unit.
constexpr int kGtNShapes = 7;
static const int kGtShapes[kGtNShapes][2] = {{256, 128}, {192, 128}, {128, 128}, {96, 128}, {128, 64}, {64, 128}, {64, 64}};
// Relative time per output of one workgroup (LDS and L2 bytes per MFMA grow as the tile shrinks); measured on 7B and 13B shapes.
static const float kGtCost[kGtNShapes] = {0.95f, 0.95f, 1.00f, 1.05f, 1.25f, 1.25f, 1.45f};

// The device spreads workgroups over its compute units, so a launch lasts as long as the unit with the most workgroups:
// ceil(workgroups / units) tiles one after the other (or side by side at the same total rate).
static int gt_choose(int rows, int T, int n_cu) {
    int best = 0; double best_t = 1e30;
    for (int s = 0; s < kGtNShapes; ++s) {
        const int bm = kGtShapes[s][0], bn = kGtShapes[s][1];
        const long long wgs = (long long)((rows + bm - 1) / bm) * ((T + bn - 1) / bn);
        const double t = (double)((wgs + n_cu - 1) / n_cu) * bm * bn * kGtCost[s];
        if (t < best_t) { best_t = t; best = s; }
    }
    return best;
}

int pi_k_gemm_tile_f16(const void * W, int rows, int cols, const void * xn_f16, int T, int epilogue, const float * add1, const float * add2,
                       float * y, void * y_f16, int tile, pi_stream_t stream) {
    if (!W || !xn_f16 || !y || rows <= 0 || T <= 0) return pi::fail(PI_E_ARG, "pi_k_gemm_tile_f16: null pointer or empty shape");
    if (cols <= 0 || cols % kGtBK) return pi::fail(PI_E_ARG, "pi_k_gemm_tile_f16: cols % 64 == 0 required");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_gemm_tile_f16: bad epilogue arguments");
    if ((((uintptr_t)W | (uintptr_t)xn_f16 | (uintptr_t)y | (uintptr_t)add1 | (uintptr_t)add2) & 15) != 0 || ((uintptr_t)y_f16 & 7) != 0)
        return pi::fail(PI_E_ARG, "pi_k_gemm_tile_f16: operands must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    int shape = -1;
    if (tile == 0) shape = gt_choose(rows, T, pi::compute_units());
    else for (int s = 0; s < kGtNShapes; ++s) if (tile == kGtShapes[s][0] * 1000 + kGtShapes[s][1]) shape = s;
    if (shape < 0) return pi::fail(PI_E_ARG, "pi_k_gemm_tile_f16: tile must be 0 or one of 256128, 192128, 128128, 96128, 128064, 64128, 64064");
#define PI_GEMM_TILE(BM, BN, WGM, WGN) do {                                                                                               \
        const int nx = (rows + BM - 1) / BM, ny = (T + BN - 1) / BN;                                                                      \
        const size_t sh = (size_t)2 * (BM + BN) * kGtRow;                                                                                 \
        static bool raised = false;                                                                                                       \
        if (!raised && sh > 64 * 1024) { PI_HIP_TRY(hipFuncSetAttribute((const void *)gemm_tile_f16_kernel<BM, BN, WGM, WGN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh)); raised = true; } \
        hipLaunchKernelGGL((gemm_tile_f16_kernel<BM, BN, WGM, WGN>), dim3(8 * ((nx + 7) / 8) * ny), dim3(64 * WGM * WGN), sh, st, (const __half *)W, (const __half *)xn_f16, T, rows, cols,   \
                           nx, ny, epilogue, add1, add2, y, (__half *)y_f16);                                                             \
    } while (0)
    switch (shape) {
        case 0: PI_GEMM_TILE(256, 128, 4, 2); break;
        case 1: PI_GEMM_TILE(192, 128, 4, 2); break;
        case 2: PI_GEMM_TILE(128, 128, 2, 2); break;
        case 3: PI_GEMM_TILE(96, 128, 2, 2); break;
        case 4: PI_GEMM_TILE(128, 64, 2, 2); break;
        case 5: PI_GEMM_TILE(64, 128, 2, 2); break;
        default: PI_GEMM_TILE(64, 64, 2, 2); break;
    }
#undef PI_GEMM_TILE
    return pi::check_launch("pi_k_gemm_tile_f16");
}
int pi_k_ffn_h_f16(const float * up, const float * gate, const float * logits, float threshold, int T, int ff, void * h_f16, pi_stream_t stream) {
    if (!up || !logits || !h_f16 || T <= 0 || ff <= 0) return pi::fail(PI_E_ARG, "pi_k_ffn_h_f16: bad arguments");
    hipLaunchKernelGGL(ffn_h_f16_kernel, dim3(1024), dim3(256), 0, (hipStream_t)stream, up, gate, logits, threshold, (size_t)T * ff, (__half *)h_f16, 0);
    return pi::check_launch("pi_k_ffn_h_f16");
}
int pi_k_ffn_h_q8_f16(const float * up, const float * gate, const float * logits, float threshold, int T, int ff, void * h_f16, pi_stream_t stream) {
    if (!up || !logits || !h_f16 || T <= 0 || ff <= 0 || ff % 64) return pi::fail(PI_E_ARG, "pi_k_ffn_h_q8_f16: n_ff must be a multiple of 64");
    hipLaunchKernelGGL(ffn_h_f16_kernel, dim3(1024), dim3(256), 0, (hipStream_t)stream, up, gate, logits, threshold, (size_t)T * ff, (__half *)h_f16, 1);
    return pi::check_launch("pi_k_ffn_h_q8_f16");
}

// W[rows][cols] in Q4_0 blocks -> fp16 (value (q - 8) * d, dequantize_row_q4_0, ggml-quants.c:1074-1092), one thread per block.  With hot
// words the rows of resident neurons come from the compact matrix W and the others from W_rest (both in ascending neuron order).
__global__ void dequant_q4_f16_kernel(const pi_block_q4_0 * __restrict__ W, const pi_block_q4_0 * __restrict__ W_rest,
                                      const uint32_t * __restrict__ hot_words, const int32_t * __restrict__ hot_prefix,
                                      int rows, int nb, __half * __restrict__ out) {
    const size_t n = (size_t)rows * nb;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
        const int row = (int)(idx / nb), blk = (int)(idx % nb);
        const pi_block_q4_0 * src;
        if (hot_words) {
            const uint32_t hot = hot_words[row >> 5];
            const int bit = row & 31, base = hot_prefix[row >> 5], below = __popc(hot & ((1u << bit) - 1u));
            src = ((hot >> bit) & 1u) ? W + (size_t)(base + below) * nb : W_rest + (size_t)((row & ~31) - base + bit - below) * nb;
        } else {
            src = W + (size_t)row * nb;
        }
        src += blk;
        uint16_t dbits; __builtin_memcpy(&dbits, &src->d, 2);
        const float d = pi_f16_from_bits(dbits);
        uint32_t qs[4]; __builtin_memcpy(qs, src->qs, 16);
        __align__(16) __half o[32];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int b = (qs[j >> 2] >> ((j & 3) * 8)) & 0xFF;
            o[j] = __float2half_rn(__fmul_rn((float)((b & 0x0F) - 8), d));
            o[j + 16] = __float2half_rn(__fmul_rn((float)((b >> 4) - 8), d));
        }
        pi_u32x4 * dst = reinterpret_cast<pi_u32x4 *>(out + (size_t)row * nb * 32 + blk * 32);
#pragma unroll
        for (int k = 0; k < 4; ++k) dst[k] = reinterpret_cast<const pi_u32x4 *>(o)[k];
    }
}
int pi_k_dequant_q4_f16(const void * W_q4, const void * W_rest_q4, const uint32_t * hot_words, const int32_t * hot_prefix, int rows, int cols,
                        void * out_f16, pi_stream_t stream) {
    if (!W_q4 || !out_f16 || rows <= 0 || cols <= 0 || cols % 32) return pi::fail(PI_E_ARG, "pi_k_dequant_q4_f16: bad arguments");
    if ((hot_words == nullptr) != (hot_prefix == nullptr) || (hot_words && !W_rest_q4) || (hot_words && rows % 32))
        return pi::fail(PI_E_ARG, "pi_k_dequant_q4_f16: hot_words, hot_prefix and the second matrix go together (rows % 32 == 0)");
    const size_t n = (size_t)rows * (cols / 32);
    size_t blocks = (n + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(dequant_q4_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const pi_block_q4_0 *)W_q4, (const pi_block_q4_0 *)W_rest_q4,
                       hot_words, hot_prefix, rows, cols / 32, (__half *)out_f16);
    return pi::check_launch("pi_k_dequant_q4_f16");
}
// the full fp16 matrix of a hybrid layer from the compact matrix of the resident neurons and the matrix of the others (both in
// ascending neuron order); one workgroup per row, 16 bytes per lane and pass
__global__ void assemble_rows_f16_kernel(const __half * __restrict__ W, const __half * __restrict__ W_rest, const uint32_t * __restrict__ hot_words,
                                         const int32_t * __restrict__ hot_prefix, int cols, __half * __restrict__ out) {
    const int row = blockIdx.x;
    const uint32_t hot = hot_words[row >> 5];
    const int bit = row & 31, base = hot_prefix[row >> 5], below = __popc(hot & ((1u << bit) - 1u));
    const __half * src = ((hot >> bit) & 1u) ? W + (size_t)(base + below) * cols : W_rest + (size_t)((row & ~31) - base + bit - below) * cols;
    const pi_u32x4 * s4 = reinterpret_cast<const pi_u32x4 *>(src);
    pi_u32x4 * d4 = reinterpret_cast<pi_u32x4 *>(out + (size_t)row * cols);
    for (int i = threadIdx.x; i < cols / 8; i += blockDim.x) d4[i] = s4[i];
}
int pi_k_assemble_rows_f16(const void * W_f16, const void * W_rest_f16, const uint32_t * hot_words, const int32_t * hot_prefix, int rows, int cols,
                           void * out_f16, pi_stream_t stream) {
    if (!W_f16 || !W_rest_f16 || !hot_words || !hot_prefix || !out_f16 || rows <= 0 || rows % 32 || cols <= 0 || cols % 8)
        return pi::fail(PI_E_ARG, "pi_k_assemble_rows_f16: bad arguments (rows % 32 == 0, cols % 8 == 0)");
    hipLaunchKernelGGL(assemble_rows_f16_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream, (const __half *)W_f16, (const __half *)W_rest_f16,
                       hot_words, hot_prefix, cols, (__half *)out_f16);
    return pi::check_launch("pi_k_assemble_rows_f16");
}
int pi_k_transpose_f16(const void * in, int rows, int cols, void * out, pi_stream_t stream) {
    if (!in || !out || rows <= 0 || cols <= 0) return pi::fail(PI_E_ARG, "pi_k_transpose_f16: bad arguments");
    hipLaunchKernelGGL(transpose_f16_kernel, dim3((cols + 31) / 32, (rows + 31) / 32), dim3(32, 8), 0, (hipStream_t)stream, (const __half *)in, rows, cols, (__half *)out);
    return pi::check_launch("pi_k_transpose_f16");
}

int pi_k_batch_predictor_fc2(const void * fc2_f16, int ff, int r, const void * hidden_f16, int T, float threshold, float * logits,
                             pi_workspace * ws, pi_stream_t stream) {
    if (!ws || ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_batch_predictor_fc2: ff exceeds the workspace");
    return gemm_launch("pi_k_batch_predictor_fc2", fc2_f16, ff, r, hidden_f16, T, PI_EPI_NONE, nullptr, nullptr, logits, nullptr, threshold, ws->row_any, stream);
}

int pi_k_batch_predictor_fc2_ol(const void * fc2_f16, int ff, int r, const void * hidden_ol, int T, float threshold, float * logits,
                                pi_workspace * ws, pi_stream_t stream) {
    if (!ws || ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_batch_predictor_fc2_ol: ff exceeds the workspace");
    return gemm_launch("pi_k_batch_predictor_fc2_ol", fc2_f16, ff, r, hidden_ol, T, PI_EPI_NONE, nullptr, nullptr, logits, nullptr, threshold, ws->row_any, stream, 1);
}

static int batch_sparse_ffn(const float * logits, int T, int ff, float threshold, const void * up_f16, const void * gate_f16, const void * down_t_f16,
                            int cols, const void * xn_f16, int epilogue, const float * add1, const float * add2, float * out,
                            int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream, int xol) {
    if (!logits || !up_f16 || !down_t_f16 || !xn_f16 || !out || !union_rows || !n_union || !ws) return pi::fail(PI_E_ARG, "pi_k_batch_sparse_ffn: null pointer");
    if (T < 1 || T > kBtMaxT || ff <= 0 || ff > ws->max_ff || cols <= 0 || cols > ws->max_d || cols % kBaTile || cols % 128)
        return pi::fail(PI_E_ARG, "pi_k_batch_sparse_ffn: 1 <= T <= 16, ff <= workspace, cols % 256 == 0 and cols <= workspace required");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || epilogue == PI_EPI_RELU || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_batch_sparse_ffn: bad epilogue arguments");
    hipStream_t st = (hipStream_t)stream;
    const int n_cu = pi::compute_units();
    const bool balanced = cols % 256 == 0 && n_cu > 0 && (size_t)ff * cols * 2 < ((size_t)1 << 32);
    // the one-workgroup-per-unit gate / up kernel makes the union list itself where its threads can hold all the flags
    const unsigned char * flags = (balanced && ff <= 32 * kUbBlock && ff % 16 == 0) ? ws->row_any : nullptr;
    if (!flags) hipLaunchKernelGGL(union_active_kernel, dim3(1), dim3(1024), 0, st, ws->row_any, ff, ws->words, union_rows, n_union);
    const int hstride = ws->max_ff + 16;
    if (cols % 256 == 0) {
        if (balanced) {
            if (gate_f16) hipLaunchKernelGGL(batch_upgate_bal_f16_kernel<true>, dim3(n_cu), dim3(kUbBlock), 0, st, (const __half *)up_f16, (const __half *)gate_f16, cols,
                                             (const __half *)xn_f16, T, logits, ff, threshold, union_rows, n_union, ws->hc_batch, hstride, xol, flags);
            else hipLaunchKernelGGL(batch_upgate_bal_f16_kernel<false>, dim3(n_cu), dim3(kUbBlock), 0, st, (const __half *)up_f16, (const __half *)nullptr, cols,
                                    (const __half *)xn_f16, T, logits, ff, threshold, union_rows, n_union, ws->hc_batch, hstride, xol, flags);
        } else if (xol) return pi::fail(PI_E_ARG, "pi_k_batch_sparse_ffn_ol: the operand layout needs the one-workgroup-per-unit kernel (ff * cols * 2 < 4 GiB)");
        else
            hipLaunchKernelGGL(batch_upgate_lds_f16_kernel, dim3((ff + 15) / 16), dim3(kBlock), 0, st, (const __half *)up_f16, (const __half *)gate_f16, cols,
                               (const __half *)xn_f16, T, logits, ff, threshold, union_rows, n_union, ws->hc_batch, hstride, (float *)nullptr);
        hipLaunchKernelGGL(batch_axpy_mfma_f16_kernel, dim3((cols + 511) / 512, kBmGroups), dim3(128), 0, st, (const __half *)down_t_f16, cols,
                           ws->hc_batch, hstride, union_rows, n_union, ws->ffn_partial);
        hipLaunchKernelGGL(batch_reduce_kernel, dim3((T * cols / 4 + kBlock - 1) / kBlock), dim3(kBlock), 0, st, ws->ffn_partial, kBmGroups, T, cols, epilogue, add1, add2, out);
    } else {
        if (xol) return pi::fail(PI_E_ARG, "pi_k_batch_sparse_ffn_ol: cols % 256 == 0 required");
        hipLaunchKernelGGL(batch_upgate_f16_kernel, dim3((ff + 15) / 16), dim3(kBlock), 0, st, (const __half *)up_f16, (const __half *)gate_f16, cols,
                           (const __half *)xn_f16, T, logits, ff, threshold, union_rows, n_union, ws->hc_batch, hstride);
        hipLaunchKernelGGL(batch_axpy_f16_kernel, dim3(cols / kBaTile, kBaGroups), dim3(kBaBlock), 0, st, (const __half *)down_t_f16, cols,
                           ws->hc_batch, hstride, union_rows, n_union, ws->ffn_partial);
        hipLaunchKernelGGL(batch_reduce_kernel, dim3((T * cols / 4 + kBlock - 1) / kBlock), dim3(kBlock), 0, st, ws->ffn_partial, kBaGroups, T, cols, epilogue, add1, add2, out);
    }
    return pi::check_launch("pi_k_batch_sparse_ffn");
}

int pi_k_batch_sparse_ffn(const float * logits, int T, int ff, float threshold, const void * up_f16, const void * gate_f16, const void * down_t_f16,
                          int cols, const void * xn_f16, int epilogue, const float * add1, const float * add2, float * out,
                          int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream) {
    return batch_sparse_ffn(logits, T, ff, threshold, up_f16, gate_f16, down_t_f16, cols, xn_f16, epilogue, add1, add2, out, union_rows, n_union, ws, stream, 0);
}

int pi_k_batch_sparse_ffn_ol(const float * logits, int T, int ff, float threshold, const void * up_f16, const void * gate_f16, const void * down_t_f16,
                             int cols, const void * xn_ol, int epilogue, const float * add1, const float * add2, float * out,
                             int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream) {
    return batch_sparse_ffn(logits, T, ff, threshold, up_f16, gate_f16, down_t_f16, cols, xn_ol, epilogue, add1, add2, out, union_rows, n_union, ws, stream, 1);
}

// the union of the step's active rows alone (list and count from the flags pi_k_batch_predictor_fc2 left in the workspace): the statistic
// a caller keeps when it runs the step's FFN dense
int pi_k_batch_union_count(int ff, int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream) {
    if (!union_rows || !n_union || !ws || ff <= 0 || ff > ws->max_ff) return pi::fail(PI_E_ARG, "pi_k_batch_union_count: bad arguments");
    hipLaunchKernelGGL(union_active_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, ws->row_any, ff, ws->words, union_rows, n_union);
    return pi::check_launch("pi_k_batch_union_count");
}

// The two sparse operators of a step of T <= 16 tokens AS OPERATORS (the reference's mul_mat_batch_sparse / axpy at batch size > 1,
// ggml-cuda.cu:6994-7034, 8787-8814): the caller supplies the predictor output idx [T][ff]; each weight row is read once for the step.
int pi_k_batch_sparse_mul_mat(const void * W_f16, int ff, int cols, const void * xn_f16, int T, const float * idx, float threshold,
                              float * y, int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream) {
    if (!W_f16 || !xn_f16 || !idx || !y || !union_rows || !n_union || !ws) return pi::fail(PI_E_ARG, "pi_k_batch_sparse_mul_mat: null pointer");
    if (T < 1 || T > kBtMaxT || ff <= 0 || ff > ws->max_ff || cols <= 0 || cols % 256) return pi::fail(PI_E_ARG, "pi_k_batch_sparse_mul_mat: 1 <= T <= 16, ff <= workspace and cols % 256 == 0 required");
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(batch_flag_any_kernel, dim3((ff + 255) / 256), dim3(256), 0, st, idx, T, ff, threshold, ws->row_any);
    hipLaunchKernelGGL(union_active_kernel, dim3(1), dim3(1024), 0, st, ws->row_any, ff, ws->words, union_rows, n_union);
    hipLaunchKernelGGL(zero_f32_kernel, dim3(256), dim3(256), 0, st, y, (size_t)T * ff);
    hipLaunchKernelGGL(batch_upgate_lds_f16_kernel, dim3((ff + 15) / 16), dim3(kBlock), 0, st, (const __half *)W_f16, (const __half *)nullptr, cols,
                       (const __half *)xn_f16, T, idx, ff, threshold, union_rows, n_union, ws->hc_batch, ws->max_ff + 16, y);
    return pi::check_launch("pi_k_batch_sparse_mul_mat");
}
int pi_k_batch_sparse_axpy(const void * down_t_f16, int cols, int ff, const float * h, const float * idx, int T, float threshold,
                           float * out, int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream) {
    if (!down_t_f16 || !h || !idx || !out || !union_rows || !n_union || !ws) return pi::fail(PI_E_ARG, "pi_k_batch_sparse_axpy: null pointer");
    if (T < 1 || T > kBtMaxT || ff <= 0 || ff > ws->max_ff || cols <= 0 || cols > ws->max_d || cols % 256)
        return pi::fail(PI_E_ARG, "pi_k_batch_sparse_axpy: 1 <= T <= 16, ff and cols within the workspace and cols % 256 == 0 required");
    hipStream_t st = (hipStream_t)stream;
    const int hstride = ws->max_ff + 16;
    hipLaunchKernelGGL(batch_flag_any_kernel, dim3((ff + 255) / 256), dim3(256), 0, st, idx, T, ff, threshold, ws->row_any);
    hipLaunchKernelGGL(union_active_kernel, dim3(1), dim3(1024), 0, st, ws->row_any, ff, ws->words, union_rows, n_union);
    hipLaunchKernelGGL(batch_gather_h_kernel, dim3(32, kBtMaxT), dim3(256), 0, st, h, idx, T, ff, threshold, union_rows, n_union, ws->hc_batch, hstride);
    hipLaunchKernelGGL(batch_axpy_mfma_f16_kernel, dim3((cols + 511) / 512, kBmGroups), dim3(128), 0, st, (const __half *)down_t_f16, cols,
                       ws->hc_batch, hstride, union_rows, n_union, ws->ffn_partial);
    hipLaunchKernelGGL(batch_reduce_kernel, dim3((T * cols / 4 + kBlock - 1) / kBlock), dim3(kBlock), 0, st, ws->ffn_partial, kBmGroups, T, cols, PI_EPI_NONE,
                       (const float *)nullptr, (const float *)nullptr, out);
    return pi::check_launch("pi_k_batch_sparse_axpy");
}

int pi_k_step_advance(int32_t * step, pi_stream_t stream) {
    if (!step) return pi::fail(PI_E_ARG, "pi_k_step_advance: null pointer");
    hipLaunchKernelGGL(step_advance_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, step);
    return pi::check_launch("pi_k_step_advance");
}

int pi_k_embed_batch(const void * table_f16, int cols, const int32_t * tokens, int T, float * x, pi_stream_t stream) {
    if (!table_f16 || !tokens || !x || cols <= 0 || T <= 0 || T > kChunkMaxT) return pi::fail(PI_E_ARG, "pi_k_embed_batch: bad arguments");
    hipLaunchKernelGGL(embed_f16_batch_kernel, dim3((cols + 255) / 256, T), dim3(256), 0, (hipStream_t)stream, (const __half *)table_f16, cols, tokens, x);
    return pi::check_launch("pi_k_embed_batch");
}


int pi_k_argmax_batch(const float * logits, int n, int T, int32_t * tokens, int32_t * positions, int32_t * step, int32_t * out_tokens, int max_steps,
                      pi_stream_t stream) {
    if (!logits || !tokens || n <= 0 || T <= 0 || T > kBtMaxT) return pi::fail(PI_E_ARG, "pi_k_argmax_batch: bad arguments");
    hipLaunchKernelGGL(argmax_batch_kernel, dim3(T), dim3(1024), 0, (hipStream_t)stream, logits, n, T, tokens, positions, step, out_tokens, max_steps);
    return pi::check_launch("pi_k_argmax_batch");
}

}  // extern "C"

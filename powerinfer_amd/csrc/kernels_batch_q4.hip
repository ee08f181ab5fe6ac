// Steps of up to 16 tokens on Q4_0 weights with the CPU path's arithmetic: a weight block of 32 quants meets the Q8_0 block of
// the activations in one integer MFMA (v_mfma_i32_16x16x32_i8: K = 32 is exactly one block), the exact int32 sum is scaled by
// d_w * d_x in fp32 and added block after block, as ggml_vec_dot_q4_0_q8_0 does (ggml-quants.c:2512-2650; batch use in the
// reference: mul_mat_q4_0_q8_1 tiles and dequantize_mul_mat_batch_sparse, ggml-cuda.cu:3524-4308, 4757-4830).
//
// Weights are read from a split form made once per model (pi_k_q4_split): the quant bytes in one array and the fp16 scales in
// another (the 18-byte blocks of the file format leave their quants on 2-byte boundaries).  The quants of four consecutive
// blocks are interleaved by dword: [row][block / 4][dword g of the block][block % 4], so that the lane that feeds k-slot group g of
// the integer MFMA reads its dword of four blocks as one 16-byte load, and a wave's 16 rows x 64 bytes per load are whole half
// cache lines whose other half the next load takes.
// Activations come as Q8_0 blocks in three arrays (pi_k_norm_q8_blocks): int8 quants in the MFMA's operand layout, scale d [nblk][16] and
// -8 * sum(q) [nblk][16] - the nibbles go into the MFMA unsigned and the MFMA's accumulator input carries -8 * sum(x), so that
// sum((q - 8) * x) = sum(q * x) - 8 * sum(x) comes out of the instruction, exact in int32.
#include "kernels_common.hpp"

namespace {

typedef int pi_i4 __attribute__((ext_vector_type(4)));

__global__ void q4_split_kernel(const pi_block_q4_0 * __restrict__ w, size_t n_blocks, uint32_t * __restrict__ qs, uint16_t * __restrict__ ds) {
    const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= n_blocks) return;
    const unsigned char * p = reinterpret_cast<const unsigned char *>(w + b);
    uint16_t h[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) h[i] = reinterpret_cast<const uint16_t *>(p)[i];          // 18 bytes on a 2-byte boundary
    ds[b] = h[0];
#pragma unroll
    for (int i = 0; i < 4; ++i) qs[((b >> 2) * 4 + i) * 4 + (b & 3)] = (uint32_t)h[1 + 2 * i] | ((uint32_t)h[2 + 2 * i] << 16);      // blocks per row % 4 == 0
}

// One row per workgroup: norm (as norm_round_f16_kernel), then Q8_0 blocks of 32 (quantize_row_q8_0, ggml-quants.c:702-760):
// d = fp16(amax / 127), q = rint(v * (127 / amax)).  Outputs: q in the MFMA's operand layout (below), d and -8 * sum(q) as [blk][16]
// (token innermost).
__global__ __launch_bounds__(1024) void norm_q8_blocks_kernel(const float * __restrict__ x, int cols, NormArgs na, int8_t * __restrict__ q_out,
                                                              float * __restrict__ d_out, int * __restrict__ s8_out, __half * __restrict__ plain16, int plain_ol) {
    // plain_ol != 0: plain16 in the operand layout of the 16-token fp16 mat-muls (pi_ol_index) instead of [token][cols]
    __shared__ double red[16];
    const int t = blockIdx.x;
    const float * xt = x + (size_t)t * cols;
    float mean = 0.0f, scale = 1.0f;
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
        if (k * 1024 >= cols) break;                              // uniform: the row ends before this slot
        const int i = threadIdx.x + k * 1024;
        float v = xv[k];
        if (plain16 && i < cols) plain16[plain_ol ? pi_ol_index(t, i) : (size_t)t * cols + i] = __float2half_rn(v);
        if (na.kind != 0) {
            v = __fmul_rn(na.kind == 2 ? __fsub_rn(v, mean) : v, scale);
            if (na.w) v = __fmul_rn(v, wv[k]);
            if (na.b) v = __fadd_rn(v, bv[k]);
        }
        if (i >= cols) v = 0.0f;
        // the 32 lanes of a half-wave hold one block
        float amax = fabsf(v);
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, PI_WAVE));
        const float d = pi_round_f16(pi_div(amax, 127.0f)), id = (amax != 0.0f) ? pi_div(127.0f, amax) : 0.0f;
        const int q = (int)rintf(__fmul_rn(v, id));
        int s = q;
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o, PI_WAVE);
        if (i < cols) {
            // operand layout of the integer MFMA: [block][k-slot group g][token][8 bytes]; the group's bytes are elements 4g .. 4g + 3 and
            // 16 + 4g .. 16 + 4g + 3 of the block, so that a lane's 8-byte operand is one load and a wave's 64 lanes read 512 contiguous bytes
            const int e = i & 31;
            q_out[(((size_t)(i >> 5) * 4 + ((e & 15) >> 2)) * 16 + t) * 8 + (e >> 4) * 4 + (e & 3)] = (int8_t)q;
            if ((i & 31) == 0) { d_out[(size_t)(i >> 5) * 16 + t] = d; s8_out[(size_t)(i >> 5) * 16 + t] = -8 * s; }
        }
    }
}

// y[t][row] = epi(sum over blocks of d_w * d_x * isum) for T <= 16 tokens.  A workgroup of four waves owns RT * 16 rows (SPARSE:
// RT = 1 and the rows are 16 entries of the step's union list, for the up and the gate matrix at once); the waves split the
// blocks in groups of eight (wave w takes groups w, w + 4, ...) and their partial sums meet in LDS in wave order.
// MFMA operands: A = activations (lane (i, g): token i, k-slots {4g..4g+3, 16+4g..16+4g+3} of the block), B = weights (lane (i, g):
// row i, dword g of the block's quants: low nibbles are elements 4g..4g+3, high nibbles 16+4g..16+4g+3); D[token 4g + r][row i].
constexpr int kQ4Group = 8;        // blocks per load group
template <int RT, bool SPARSE, bool GATE>
__global__ __launch_bounds__(kBlock) void gemm_q4_t16_kernel(const uint32_t * __restrict__ qs, const uint16_t * __restrict__ ds,
                                                             const uint32_t * __restrict__ qs2, const uint16_t * __restrict__ ds2,
                                                             int rows, int nblk, const int8_t * __restrict__ qx, const float * __restrict__ dx,
                                                             const int * __restrict__ sx8, int T, int epi, const float * __restrict__ add1,
                                                             const float * __restrict__ add2, float * __restrict__ y,
                                                             const int32_t * __restrict__ union_rows, const int32_t * __restrict__ n_union,
                                                             const float * __restrict__ logits, float threshold) {
    constexpr int NM = SPARSE ? (GATE ? 2 : 1) : RT;               // weight tiles a wave multiplies per activation fragment
    __shared__ float red[kWavesPerBlock][NM * 4][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i = lane & 15, g = lane >> 4;
    const int cols = nblk * 32;
    int nu = rows;
    // SPARSE: the list entry of this lane is requested together with the list's length (the list has one entry per row of the
    // matrix, so the address is good whatever the length; an entry behind the end is stale and is replaced by the last one)
    int listed = 0;
    if (SPARSE) {
        listed = union_rows[(int)blockIdx.x * 16 + i];
        nu = *n_union;
        if ((int)blockIdx.x * 16 >= nu) return;
        if ((int)blockIdx.x * 16 + i >= nu) listed = union_rows[nu - 1];
    }
    size_t wrow[NM];
    int my_row[NM];
#pragma unroll
    for (int m = 0; m < NM; ++m) {
        int r = SPARSE ? (int)blockIdx.x * 16 + i : ((int)blockIdx.x * RT + m) * 16 + i;
        if (SPARSE) r = listed;
        else r = r < rows ? r : rows - 1;
        my_row[m] = r;
        wrow[m] = (size_t)r * nblk;
    }
    float acc[NM][4];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[m][r] = 0.0f;
    // LDS: the activations' scales and block sums for every block, [blk][16 tokens]
    extern __shared__ __align__(16) unsigned char q4_smem[];
    float * sdx = reinterpret_cast<float *>(q4_smem);
    int * ssx = reinterpret_cast<int *>(q4_smem + (size_t)nblk * 64);
    const unsigned long * qx64 = reinterpret_cast<const unsigned long *>(qx) + g * 16 + i;      // + block * 64
    const int ngroups = nblk / kQ4Group;
    struct Loads { pi_u32x4 w0[NM], w1[NM], wd[NM]; unsigned long a[kQ4Group]; };
    auto fetch = [&](Loads & L, int grp) {
        const int kb0 = grp * kQ4Group;
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            const uint32_t * q = (SPARSE && m == 1) ? qs2 : qs;
            const uint16_t * d = (SPARSE && m == 1) ? ds2 : ds;
            // dword g of blocks kb0 .. kb0 + 3 and of kb0 + 4 .. kb0 + 7: two 16-byte loads (plain loads: the other lanes' and the next
            // load's bytes of the same cache lines are served from the cache)
            L.w0[m] = pi_ld16(q + ((wrow[m] + kb0) + g) * 4);
            L.w1[m] = pi_ld16(q + ((wrow[m] + kb0 + 4) + g) * 4);
            L.wd[m] = pi_ld16(d + wrow[m] + kb0);                  // eight fp16 scales: nblk % 8 == 0 keeps this 16-byte aligned
        }
#pragma unroll
        for (int u = 0; u < kQ4Group; ++u) L.a[u] = qx64[(size_t)(kb0 + u) * 64];
    };
    auto multiply = [&](const Loads & L, int grp) {
        const int kb0 = grp * kQ4Group;
#pragma unroll
        for (int u = 0; u < kQ4Group; ++u) {
            const float4 dxs = *reinterpret_cast<const float4 *>(sdx + (kb0 + u) * 16 + 4 * g);
            const pi_i4 sxs = *reinterpret_cast<const pi_i4 *>(ssx + (kb0 + u) * 16 + 4 * g);
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                const uint32_t w = u < 4 ? L.w0[m][u & 3] : L.w1[m][u & 3];
                const unsigned long lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
                // the accumulator input carries -8 * sum(x) of the activation block: the result is sum((q - 8) * x), exact in int32
                const pi_i4 sum = __builtin_amdgcn_mfma_i32_16x16x32_i8((long)L.a[u], (long)((hi << 32) | lo), sxs, 0, 0, 0);
                const uint32_t dpair = L.wd[m][u >> 1];
                const float dw = pi_f16_from_bits((uint16_t)((u & 1) ? (dpair >> 16) : (dpair & 0xFFFFu)));
                acc[m][0] = fmaf(__fmul_rn(dw, dxs.x), (float)sum[0], acc[m][0]);
                acc[m][1] = fmaf(__fmul_rn(dw, dxs.y), (float)sum[1], acc[m][1]);
                acc[m][2] = fmaf(__fmul_rn(dw, dxs.z), (float)sum[2], acc[m][2]);
                acc[m][3] = fmaf(__fmul_rn(dw, dxs.w), (float)sum[3], acc[m][3]);
            }
        }
    };
    // A wave's groups (wave, wave + 4, ...) pass through two register buffers: a buffer is requested again as soon as it has been
    // multiplied, so one group is always on its way while the other is multiplied.  Every load of the loop is unconditional (a
    // request behind the wave's last group reads that group again and is not used), which lets the waits be exact counts instead
    // of waits for everything in flight; the first two groups are already under way while the workgroup stages the scales.
    const int my_n = (ngroups - wave + kWavesPerBlock - 1) / kWavesPerBlock;          // groups of this wave (0 for a wave behind a short row's end)
    auto grp_of = [&](int k) { return wave + (k < my_n ? k : my_n - 1) * kWavesPerBlock; };
    Loads L0, L1;
    if (my_n > 0) { fetch(L0, grp_of(0)); fetch(L1, grp_of(1)); }
    for (int k = threadIdx.x; k < nblk * 4; k += kBlock) {
        reinterpret_cast<pi_u32x4 *>(sdx)[k] = pi_ld16(dx + (size_t)k * 4);
        reinterpret_cast<pi_u32x4 *>(ssx)[k] = pi_ld16(sx8 + (size_t)k * 4);
    }
    __syncthreads();
    if (my_n > 0) {
        int k = 0;
        for (; k + 2 < my_n; k += 2) {
            multiply(L0, grp_of(k));
            fetch(L0, grp_of(k + 2));
            multiply(L1, grp_of(k + 1));
            fetch(L1, grp_of(k + 3));
        }
        multiply(L0, grp_of(k));
        if (k + 1 < my_n) multiply(L1, grp_of(k + 1));
    }
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][m * 4 + r][lane] = acc[m][r];
    __syncthreads();
    if (wave != 0) return;
    float v[NM][4];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float s = red[0][m * 4 + r][lane];
            for (int w = 1; w < kWavesPerBlock; ++w) s = __fadd_rn(s, red[w][m * 4 + r][lane]);
            v[m][r] = s;
        }
    if (SPARSE) {
        // v[0] = up . x, v[1] = gate . x (or no gate matrix: relu(up)); h where the predictor says so, 0 elsewhere
        if ((int)blockIdx.x * 16 + i >= nu) return;
        const int n = my_row[0];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int t = 4 * g + r;
            if (t >= T) continue;
            const bool on = !(logits[(size_t)t * rows + n] < threshold);
            const float h = GATE ? __fmul_rn(fmaxf(v[NM - 1][r], 0.0f), v[0][r]) : fmaxf(v[0][r], 0.0f);
            y[(size_t)t * rows + n] = on ? h : 0.0f;
        }
        return;
    }
#pragma unroll
    for (int m = 0; m < NM; ++m) {
        const int row = ((int)blockIdx.x * RT + m) * 16 + i;
        if (row >= rows) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int t = 4 * g + r;
            if (t >= T) continue;
            const size_t o = (size_t)t * rows + row;
            float s = v[m][r];
            if (epi == PI_EPI_RELU) s = fmaxf(s, 0.0f);
            else if (epi == PI_EPI_ADD) s = __fadd_rn(s, add1[o]);
            else if (epi == PI_EPI_ADD2) s = __fadd_rn(__fadd_rn(s, add1[o]), add2[o]);
            y[o] = s;
        }
    }
}

// h of a step as the values its Q8_0 blocks keep (blocks of 32 consecutive neurons; a neuron outside the union is 0 for every
// token): hq[t][n] = q * d, the factor the CPU path's axpy multiplies a down-projection row with (ggml_axpy_q4_0_q8_0,
// ggml.c:14436-14470).  One half-wave per (token, block).
__global__ __launch_bounds__(256) void h_q8_values_kernel(const float * __restrict__ h, const unsigned char * __restrict__ row_any, int T, int ff,
                                                          float * __restrict__ hq) {
    const int blk = (int)blockIdx.x * 8 + (threadIdx.x >> 5), t = blockIdx.y, n = blk * 32 + (threadIdx.x & 31);
    const bool in = n < ff;
    // both operands requested at once (a neuron outside the union holds a stale h, which the flag deselects): one trip to memory
    const float hv = in ? h[(size_t)t * ff + n] : 0.0f;
    const unsigned char any = in ? row_any[n] : (unsigned char)0;
    float v = any ? hv : 0.0f;
    float amax = fabsf(v);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, PI_WAVE));
    const float d = pi_round_f16(pi_div(amax, 127.0f)), id = (amax != 0.0f) ? pi_div(127.0f, amax) : 0.0f;
    if (in) hq[(size_t)n * kBtMaxT + t] = __fmul_rn((float)(int)rintf(__fmul_rn(v, id)), d);          // [neuron][16 tokens]
}

// Down projection of a step over the union rows on fp32 matrix cores: out[t][c] = sum over union neurons n of hq[t][n] * d_w * (q_w - 8).
// A workgroup owns 128 columns (four Q4_0 blocks of every row) and one of KG shares of the union list; its four waves take
// neuron quads in turn.  v_mfma_f32_16x16x4_f32: A[token i][k = g] = hq[i][n_g], B[k = g][j] = weight of neuron n_g; lane (i, g) reads
// dword (i >> 2) of block (i & 3) of row n_g, whose eight nibbles are eight weights: MFMA e of the quad covers, in lane i's column,
// element 4 * (i >> 2) + e (e < 4) or 16 + 4 * (i >> 2) + e - 4 of block (i & 3).  D[token 4g + r][column of lane i].
constexpr int kQ4AxpyGroups = 16;
constexpr int kQ4AxpyUnroll = 4;       // neuron quads whose loads are in flight together
__global__ __launch_bounds__(kBlock) void batch_axpy_q4_kernel(const uint32_t * __restrict__ qs, const uint16_t * __restrict__ ds, int nblk,
                                                               const float * __restrict__ hq, const int32_t * __restrict__ union_rows,
                                                               const int32_t * __restrict__ n_union, float * __restrict__ partial, int cols) {
    __shared__ float red[kWavesPerBlock][32][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i = lane & 15, g = lane >> 4;
    const int nu = *n_union;
    const int cb = (int)blockIdx.x * 4 + (i & 3), wdw = i >> 2;    // this lane's block of the row and its dword of that block: the 16 lanes of a
                                                                   // quarter wave read the 64 contiguous bytes of a four-block group
    pi_f4 acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = pi_f4{0.0f, 0.0f, 0.0f, 0.0f};
    const int nquads = (nu + 3) / 4;
    const int stride = kQ4AxpyGroups * kWavesPerBlock;
    // quad of this wave's u-th slot in iteration it: q0 + (it * kQ4AxpyUnroll + u) * stride.  The loads of three iterations are in flight
    // while a fourth is multiplied.  What keeps them in flight: a quad's four row numbers come through the scalar unit (one
    // 16-byte load; vector loads of them would sit in the in-order counter of the weight loads, and waiting for a row number would
    // drain the weights requested before it), and every load is unconditional - a slot behind the list's end reads the wave's last quad again (every
    // wave reading ONE row there would queue up on that row's memory channel) and counts with h = 0 - so that the wait before an iteration's first MFMA is an exact count.  (union_rows holds ff entries and ff % 4 == 0.)
    const int q0 = (int)blockIdx.y * kWavesPerBlock + __builtin_amdgcn_readfirstlane(wave);
    const int q_last = q0 < nquads ? q0 + (nquads - 1 - q0) / stride * stride : 0;       // this wave's last quad
    struct Quad { uint32_t w[kQ4AxpyUnroll]; uint16_t dw[kQ4AxpyUnroll]; float a[kQ4AxpyUnroll]; bool live[kQ4AxpyUnroll]; };
    int4 rn[kQ4AxpyUnroll];                                        // the row numbers of the next fetch's quads (uniform: scalar registers)
    auto fetch_rows = [&](int it) {
#pragma unroll
        for (int u = 0; u < kQ4AxpyUnroll; ++u) {
            const int q = q0 + (it * kQ4AxpyUnroll + u) * stride;
            rn[u] = *reinterpret_cast<const int4 *>(union_rows + 4 * (q < nquads ? q : q_last));
        }
    };
    auto fetch = [&](Quad & Q, int it) {                            // uses the row numbers requested one fetch earlier, requests the next ones
#pragma unroll
        for (int u = 0; u < kQ4AxpyUnroll; ++u) {
            const int q = q0 + (it * kQ4AxpyUnroll + u) * stride;
            const int r0 = __builtin_amdgcn_readfirstlane(rn[u].x), r1 = __builtin_amdgcn_readfirstlane(rn[u].y);
            const int r2 = __builtin_amdgcn_readfirstlane(rn[u].z), r3 = __builtin_amdgcn_readfirstlane(rn[u].w);
            Q.live[u] = q < nquads && 4 * q + g < nu;
            const int qq = q < nquads ? q : q_last;                 // entry 4 qq of the list is a row of the union
            const size_t row = (size_t)(4 * qq + g < nu ? (g == 0 ? r0 : g == 1 ? r1 : g == 2 ? r2 : r3) : r0);
            Q.w[u]  = qs[(row * nblk + (size_t)blockIdx.x * 4) * 4 + i];
            Q.dw[u] = ds[row * nblk + cb];
            Q.a[u]  = hq[row * kBtMaxT + i];                       // token i (entries of tokens beyond T are stale and feed discarded rows)
        }
        fetch_rows(it + 1);
    };
    auto consume = [&](const Quad & Q) {
#pragma unroll
        for (int u = 0; u < kQ4AxpyUnroll; ++u) {
            const float a = Q.live[u] ? Q.a[u] : 0.0f, dw = pi_f16_from_bits(Q.dw[u]), m8 = -8.0f * dw;
            // d_w * (q - 8) as fma(q, d_w, -8 d_w): the same single rounding of the same exact product (8 d_w is exact), and a byte of
            // the masked dword converts to float in one instruction: two VALU operations per MFMA instead of four
            const uint32_t lo = Q.w[u] & 0x0F0F0F0Fu, hi = (Q.w[u] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float nib = (float)(((e < 4 ? lo : hi) >> (8 * (e & 3))) & 0xFFu);
                acc[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, fmaf(nib, dw, m8), acc[e], 0, 0, 0);
            }
        }
    };
    const int n_it = q0 < nquads ? (nquads - q0 + kQ4AxpyUnroll * stride - 1) / (kQ4AxpyUnroll * stride) : 0;
    if (n_it > 0) {
        // three iterations of loads in flight behind the one being multiplied
        Quad S0, S1, S2, S3;
        fetch_rows(0);
        fetch(S0, 0); fetch(S1, 1); fetch(S2, 2);
        int it = 0;
        for (; it + 4 <= n_it; it += 4) {
            fetch(S3, it + 3); consume(S0);
            fetch(S0, it + 4); consume(S1);
            fetch(S1, it + 5); consume(S2);
            fetch(S2, it + 6); consume(S3);
        }
        if (it < n_it) consume(S0);                                 // the last one to three iterations: their loads are on the way
        if (it + 1 < n_it) consume(S1);
        if (it + 2 < n_it) consume(S2);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][e * 4 + r][lane] = acc[e][r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int c = cb * 32 + (e < 4 ? 4 * wdw + e : 16 + 4 * wdw + (e - 4));
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float s = red[0][e * 4 + r][lane];
            for (int w = 1; w < kWavesPerBlock; ++w) s = __fadd_rn(s, red[w][e * 4 + r][lane]);
            partial[((size_t)blockIdx.y * kBtMaxT + 4 * g + r) * cols + c] = s;
        }
    }
}

}  // namespace

extern "C" {

int pi_k_q4_split(const void * W_q4, int rows, int cols, void * quants, void * scales, pi_stream_t stream) {
    if (!W_q4 || !quants || !scales || rows <= 0 || cols <= 0 || cols % 256) return pi::fail(PI_E_ARG, "pi_k_q4_split: null pointer or cols % 256 != 0");
    const size_t nb = (size_t)rows * (cols / 32);
    hipLaunchKernelGGL(q4_split_kernel, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (const pi_block_q4_0 *)W_q4, nb,
                       (uint32_t *)quants, (uint16_t *)scales);
    return pi::check_launch("pi_k_q4_split");
}

int pi_k_norm_q8_blocks(const float * x, int T, int cols, const pi_norm * norm, void * q, float * d, int32_t * s8, void * plain_f16, pi_stream_t stream) {
    if (!x || !norm || !q || !d || !s8 || T < 1 || T > kBtMaxT || cols <= 0 || cols % 32 || cols > 8192)
        return pi::fail(PI_E_ARG, "pi_k_norm_q8_blocks: 1 <= T <= 16, cols % 32 == 0 and cols <= 8192 required");
    hipLaunchKernelGGL(norm_q8_blocks_kernel, dim3(T), dim3(1024), 0, (hipStream_t)stream, x, cols, to_norm(norm), (int8_t *)q, d, s8, (__half *)plain_f16, 0);
    return pi::check_launch("pi_k_norm_q8_blocks");
}

int pi_k_norm_q8_blocks_ol(const float * x, int T, int cols, const pi_norm * norm, void * q, float * d, int32_t * s8, void * plain_ol, pi_stream_t stream) {
    if (!x || !norm || !q || !d || !s8 || T < 1 || T > kBtMaxT || cols <= 0 || cols % 32 || cols > 8192)
        return pi::fail(PI_E_ARG, "pi_k_norm_q8_blocks_ol: 1 <= T <= 16, cols % 32 == 0 and cols <= 8192 required");
    hipLaunchKernelGGL(norm_q8_blocks_kernel, dim3(T), dim3(1024), 0, (hipStream_t)stream, x, cols, to_norm(norm), (int8_t *)q, d, s8, (__half *)plain_ol, 1);
    return pi::check_launch("pi_k_norm_q8_blocks_ol");
}

int pi_k_gemm_q4_t16(const void * quants, const void * scales, int rows, int cols, const void * xq, const float * xd, const int32_t * xs8, int T,
                     int epilogue, const float * add1, const float * add2, float * y, pi_stream_t stream) {
    if (!quants || !scales || !xq || !xd || !xs8 || !y || rows <= 0) return pi::fail(PI_E_ARG, "pi_k_gemm_q4_t16: null pointer or empty shape");
    if (T < 1 || T > kBtMaxT || cols <= 0 || cols % 256) return pi::fail(PI_E_ARG, "pi_k_gemm_q4_t16: 1 <= T <= 16 and cols % 256 == 0 required");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_gemm_q4_t16: bad epilogue arguments");
    hipStream_t st = (hipStream_t)stream;
    const int nblk = cols / 32;
    if (rows >= 16384)
        hipLaunchKernelGGL((gemm_q4_t16_kernel<2, false, false>), dim3((rows + 31) / 32), dim3(kBlock), (size_t)nblk * 128, st, (const uint32_t *)quants, (const uint16_t *)scales,
                           (const uint32_t *)nullptr, (const uint16_t *)nullptr, rows, nblk, (const int8_t *)xq, xd, xs8, T, epilogue, add1, add2, y,
                           (const int32_t *)nullptr, (const int32_t *)nullptr, (const float *)nullptr, 0.0f);
    else
        hipLaunchKernelGGL((gemm_q4_t16_kernel<1, false, false>), dim3((rows + 15) / 16), dim3(kBlock), (size_t)nblk * 128, st, (const uint32_t *)quants, (const uint16_t *)scales,
                           (const uint32_t *)nullptr, (const uint16_t *)nullptr, rows, nblk, (const int8_t *)xq, xd, xs8, T, epilogue, add1, add2, y,
                           (const int32_t *)nullptr, (const int32_t *)nullptr, (const float *)nullptr, 0.0f);
    return pi::check_launch("pi_k_gemm_q4_t16");
}

int pi_k_batch_sparse_ffn_q4(const float * logits, int T, int ff, float threshold, const void * up_quants, const void * up_scales,
                             const void * gate_quants, const void * gate_scales, const void * down_quants, const void * down_scales, int cols,
                             const void * xq, const float * xd, const int32_t * xs8, int epilogue, const float * add1, const float * add2, float * out,
                             float * h, float * hq, int32_t * union_rows, int32_t * n_union, pi_workspace * ws, pi_stream_t stream) {
    if (!logits || !up_quants || !up_scales || !down_quants || !down_scales || !xq || !xd || !xs8 || !out || !h || !hq || !union_rows || !n_union || !ws)
        return pi::fail(PI_E_ARG, "pi_k_batch_sparse_ffn_q4: null pointer");
    if ((gate_quants == nullptr) != (gate_scales == nullptr)) return pi::fail(PI_E_ARG, "pi_k_batch_sparse_ffn_q4: gate quants and scales go together");
    if (T < 1 || T > kBtMaxT || ff <= 0 || ff > ws->max_ff || ff % 32 || cols <= 0 || cols > ws->max_d || cols % 256)
        return pi::fail(PI_E_ARG, "pi_k_batch_sparse_ffn_q4: 1 <= T <= 16, ff % 32 == 0, ff <= workspace, cols % 256 == 0 and cols <= workspace required");
    if (epilogue < 0 || epilogue > PI_EPI_ADD2 || epilogue == PI_EPI_RELU || (epilogue >= PI_EPI_ADD && !add1) || (epilogue == PI_EPI_ADD2 && !add2))
        return pi::fail(PI_E_ARG, "pi_k_batch_sparse_ffn_q4: bad epilogue arguments");
    hipStream_t st = (hipStream_t)stream;
    pi::launch_union_active(ws->row_any, ff, ws->words, union_rows, n_union, st);
#define PI_Q4_UPGATE(GATE) hipLaunchKernelGGL((gemm_q4_t16_kernel<1, true, GATE>), dim3((ff + 15) / 16), dim3(kBlock), (size_t)cols * 4, st, (const uint32_t *)up_quants,      \
                       (const uint16_t *)up_scales, (const uint32_t *)gate_quants, (const uint16_t *)gate_scales, ff, cols / 32, (const int8_t *)xq, xd, xs8, T,     \
                       PI_EPI_NONE, (const float *)nullptr, (const float *)nullptr, h, union_rows, n_union, logits, threshold)
    if (gate_quants) PI_Q4_UPGATE(true); else PI_Q4_UPGATE(false);
#undef PI_Q4_UPGATE
    hipLaunchKernelGGL(h_q8_values_kernel, dim3((ff / 32 + 7) / 8, T), dim3(256), 0, st, h, ws->row_any, T, ff, hq);
    hipLaunchKernelGGL(batch_axpy_q4_kernel, dim3(cols / 128, kQ4AxpyGroups), dim3(kBlock), 0, st, (const uint32_t *)down_quants, (const uint16_t *)down_scales,
                       cols / 32, hq, union_rows, n_union, ws->ffn_partial, cols);
    pi::launch_batch_reduce(ws->ffn_partial, kQ4AxpyGroups, T, cols, epilogue, add1, add2, out, st);
    return pi::check_launch("pi_k_batch_sparse_ffn_q4");
}

}  // extern "C"

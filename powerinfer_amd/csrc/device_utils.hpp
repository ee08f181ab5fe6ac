// Device-side helpers shared by the CDNA4 (gfx950, wave64) kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#define PI_WAVE 64

// ggml Q4_0 block: fp16 scale + 16 bytes of nibbles; element j in the low nibble of qs[j],
// element j+16 in the high nibble, value (q - 8) * d  (ggml-quants.h:10-15)
struct __attribute__((packed)) pi_block_q4_0 { uint16_t d; uint8_t qs[16]; };
static_assert(sizeof(pi_block_q4_0) == 18, "q4_0 block is 18 bytes");

// 1.0f / sqrtf(v) exactly as the CPU evaluates it: a correctly rounded fp32 square root, then a correctly rounded fp32
// division.  Both are taken through fp64 (53 >= 2 * 24 + 2 bits, so the second rounding is innocuous).  The fp32 forms the
// compiler picks for the device may be one unit in the last place off, and a norm scale that is off by one moves the fp16
// rounding of a few activations of every vector it multiplies (1e-5 of a mat-vec result at 8192 columns).
__host__ __device__ __forceinline__ float pi_inv_sqrt(float v) {
    const float r = (float)sqrt((double)v);
    return (float)(1.0 / (double)r);
}

// a / b rounded once to fp32, as IEEE division on the CPU is (the quotient is formed in fp64 and rounded: innocuous for fp32 operands)
__host__ __device__ __forceinline__ float pi_div(float a, float b) { return (float)((double)a / (double)b); }

// Wave-wide reductions through DPP (data-parallel primitives: lane permutations inside the VALU, no LDS
// crossbar round trip): pairs, quads, half rows and rows by quad_perm / row_half_mirror / row_mirror, then the
// last lane of row 0 (2) is added into row 1 (3) and lane 31 into rows 2-3, so lane 63 holds the total, which
// v_readlane hands to every lane.  The association order is fixed, so results are reproducible.
#define PI_DPP_XOR1        0xB1    /* quad_perm [1,0,3,2] */
#define PI_DPP_XOR2        0x4E    /* quad_perm [2,3,0,1] */
#define PI_DPP_HALF_MIRROR 0x141
#define PI_DPP_MIRROR      0x140
#define PI_DPP_BCAST15     0x142
#define PI_DPP_BCAST31     0x143

template <int CTRL, int ROW_MASK> __device__ __forceinline__ int pi_dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xF, false);
}
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float pi_dpp_f32(float v) {
    return __int_as_float(pi_dpp_i32<CTRL, ROW_MASK>(__float_as_int(v)));
}
template <int CTRL, int ROW_MASK> __device__ __forceinline__ double pi_dpp_f64(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = pi_dpp_i32<CTRL, ROW_MASK>((int)(b & 0xffffffffll)), hi = pi_dpp_i32<CTRL, ROW_MASK>((int)(b >> 32));
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
__device__ __forceinline__ float pi_wave_sum(float v) {
    v += pi_dpp_f32<PI_DPP_XOR1, 0xF>(v);
    v += pi_dpp_f32<PI_DPP_XOR2, 0xF>(v);
    v += pi_dpp_f32<PI_DPP_HALF_MIRROR, 0xF>(v);
    v += pi_dpp_f32<PI_DPP_MIRROR, 0xF>(v);
    v += pi_dpp_f32<PI_DPP_BCAST15, 0xA>(v);
    v += pi_dpp_f32<PI_DPP_BCAST31, 0xC>(v);
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ double pi_wave_sum_f64(double v) {
    v += pi_dpp_f64<PI_DPP_XOR1, 0xF>(v);
    v += pi_dpp_f64<PI_DPP_XOR2, 0xF>(v);
    v += pi_dpp_f64<PI_DPP_HALF_MIRROR, 0xF>(v);
    v += pi_dpp_f64<PI_DPP_MIRROR, 0xF>(v);
    v += pi_dpp_f64<PI_DPP_BCAST15, 0xA>(v);
    v += pi_dpp_f64<PI_DPP_BCAST31, 0xC>(v);
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_readlane((int)(b & 0xffffffffll), 63), hi = __builtin_amdgcn_readlane((int)(b >> 32), 63);
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
__device__ __forceinline__ float pi_wave_max(float v) {
#pragma unroll
    for (int o = PI_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, PI_WAVE));
    return v;
}
__device__ __forceinline__ int pi_wave_sum_i32(int v) {
    v += pi_dpp_i32<PI_DPP_XOR1, 0xF>(v);
    v += pi_dpp_i32<PI_DPP_XOR2, 0xF>(v);
    v += pi_dpp_i32<PI_DPP_HALF_MIRROR, 0xF>(v);
    v += pi_dpp_i32<PI_DPP_MIRROR, 0xF>(v);
    v += pi_dpp_i32<PI_DPP_BCAST15, 0xA>(v);
    v += pi_dpp_i32<PI_DPP_BCAST31, 0xC>(v);
    return __builtin_amdgcn_readlane(v, 63);
}

// round-to-nearest-even through binary16, the rounding the CPU path applies to activations
// before an fp16 dot (ggml.c:9703-9716)
__device__ __forceinline__ float pi_round_f16(float v) { return __half2float(__float2half_rn(v)); }
__device__ __forceinline__ uint16_t pi_f16_bits(float v) { return __half_as_ushort(__float2half_rn(v)); }
__device__ __forceinline__ float pi_f16_from_bits(uint16_t h) { return __half2float(__ushort_as_half(h)); }

typedef uint32_t pi_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t pi_u32x2 __attribute__((ext_vector_type(2)));

// 8 fp16 values packed in a 128-bit load -> fp32
__device__ __forceinline__ void pi_unpack8(const pi_u32x4 & v, float * f) {
    const __half2 * h = reinterpret_cast<const __half2 *>(&v);
#pragma unroll
    for (int i = 0; i < 4; ++i) { const float2 t = __half22float2(h[i]); f[2 * i] = t.x; f[2 * i + 1] = t.y; }
}
__device__ __forceinline__ float pi_dot8(const pi_u32x4 & w, const float * x, float acc) {
    float wf[8];
    pi_unpack8(w, wf);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc = fmaf(wf[i], x[i], acc);
    return acc;
}

// the same with the activations still packed as 8 fp16: both widenings fold into the mixed-precision FMA
__device__ __forceinline__ float pi_dot8h(const pi_u32x4 & w, const pi_u32x4 & x, float acc) {
    const __half2 * a = reinterpret_cast<const __half2 *>(&w);
    const __half2 * b = reinterpret_cast<const __half2 *>(&x);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc = fmaf(__low2float(a[i]), __low2float(b[i]), acc);
        acc = fmaf(__high2float(a[i]), __high2float(b[i]), acc);
    }
    return acc;
}

// streaming 128-bit load: weights are read once per token and must not displace the activations in L2
__device__ __forceinline__ pi_u32x4 pi_ld_stream(const void * p) {
    return __builtin_nontemporal_load(reinterpret_cast<const pi_u32x4 *>(p));
}
__device__ __forceinline__ pi_u32x4 pi_ld16(const void * p) { return *reinterpret_cast<const pi_u32x4 *>(p); }

// Operand layout of a step's fp16 activations ([16 token slots][cols], T <= 16): [cols / 8][16][8], i.e. the eight consecutive columns
// a lane of v_mfma_f32_16x16x32_f16 holds, token after token.  The B fragments of a 32-column step are then one contiguous kilobyte
// (lane (token i, group g) reads 16 bytes at ((4 step + g) * 16 + i) * 8 halves) instead of 16 token rows x 64 bytes, which halves the
// cache lines an activation load touches: with [token][cols] the activation loads cost the vector L1 as many line accesses as the
// weight loads of two row tiles, and the L1 is what these kernels wait for.
__device__ __forceinline__ size_t pi_ol_index(int t, int col) { return ((size_t)(col >> 3) * 16 + t) * 8 + (col & 7); }

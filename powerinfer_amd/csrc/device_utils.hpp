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

__device__ __forceinline__ float pi_wave_sum(float v) {
#pragma unroll
    for (int o = PI_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, PI_WAVE);
    return v;
}
__device__ __forceinline__ double pi_wave_sum_f64(double v) {
#pragma unroll
    for (int o = PI_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, PI_WAVE);
    return v;
}
__device__ __forceinline__ float pi_wave_max(float v) {
#pragma unroll
    for (int o = PI_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, PI_WAVE));
    return v;
}
__device__ __forceinline__ int pi_wave_sum_i32(int v) {
#pragma unroll
    for (int o = PI_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, PI_WAVE);
    return v;
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

// streaming 128-bit load: weights are read once per token and must not displace the activations in L2
__device__ __forceinline__ pi_u32x4 pi_ld_stream(const void * p) {
    return __builtin_nontemporal_load(reinterpret_cast<const pi_u32x4 *>(p));
}
__device__ __forceinline__ pi_u32x4 pi_ld16(const void * p) { return *reinterpret_cast<const pi_u32x4 *>(p); }

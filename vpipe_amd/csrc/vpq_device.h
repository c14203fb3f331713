// Device-side helpers shared by the gfx950 kernels: vector types, bf16
// conversions, nibble unpacking and the wave64 reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vpq {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;

constexpr int kGroup = 64;    // quantization group along K
constexpr int kWave = 64;     // CDNA wavefront

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16)
{
  return __uint_as_float(bits16 << 16);
}

// Upper half of a dword holding two bf16 values, widened in one AND.
__device__ __forceinline__ float bf16_hi_to_f32(uint32_t packed)
{
  return __uint_as_float(packed & 0xffff0000u);
}

__device__ __forceinline__ float bf16_lo_to_f32(uint32_t packed)
{
  return __uint_as_float(packed << 16);
}

// fp32 -> bf16 bits, round to nearest even; NaN stays a quiet NaN.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f)
{
  const uint32_t x = __float_as_uint(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) { return (x >> 16) | 0x40u; }
  return (x + 0x7fffu + ((x >> 16) & 1u)) >> 16;
}

// Two fp32 -> one dword of two bf16 (lo = a, hi = b) through the hardware
// converter (v_cvt_pk_bf16_f32, round to nearest even).
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b)
{
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

// IEEE binary16 bits -> fp32 (exact).
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h)
{
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// fp32 -> IEEE binary16 bits, round to nearest even (v_cvt_f16_f32).
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f)
{
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

// Element-type helpers of the kernels that exist for both element types of the reference
// (VPIPE_ELT = bfloat or half): F16 = false bf16, true IEEE binary16.
template <bool F16>
__device__ __forceinline__ float elt_bits_to_f32(uint32_t bits16)
{
  return F16 ? f16_bits_to_f32(bits16) : bf16_bits_to_f32(bits16);
}
template <bool F16>
__device__ __forceinline__ float elt_lo_to_f32(uint32_t packed)
{
  return F16 ? f16_bits_to_f32(packed & 0xffffu) : bf16_lo_to_f32(packed);
}
template <bool F16>
__device__ __forceinline__ float elt_hi_to_f32(uint32_t packed)
{
  return F16 ? f16_bits_to_f32(packed >> 16) : bf16_hi_to_f32(packed);
}
template <bool F16>
__device__ __forceinline__ uint32_t f32_to_elt_bits(float f)
{
  return F16 ? f32_to_f16_bits(f) : f32_to_bf16_bits(f);
}
template <bool F16>
__device__ __forceinline__ uint32_t pack_elt2(float a, float b)
{
  if constexpr (F16) {
    // one v_cvt_pk_f16_f32 (round to nearest even)
    uint32_t r;
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
  } else {
    return pack_bf16x2(a, b);
  }
}

// Gated activation of one (gate, up) pair of fp32 sums, the store expressions of the fused
// gate|up kernels:
//   kGateSwiglu  silu(gate) * up, silu(g) = g / (1 + exp(-g))
//                (gpu-kernels/metal/quant/affine_qmv.metal:882-888, affine_qmm_steel.metal:755-766)
//   kGateGeglu   gelu_tanh(gate) * up = 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) * up
//                (affine_qmv.metal:1423-1429, affine_qmm_steel.metal:1541-1544)
constexpr int kGateNone = 0, kGateSwiglu = 1, kGateGeglu = 2;
// The store of kStoreGeluMul: gelu_tanh(v) * mul on the GEMV's result already rounded to the element type
// (gpu-kernels/metal/quant/affine_qmv.metal:268-279).
__device__ __forceinline__ float gelu_mul_f32(float v, float mul)
{
  const float t = tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v));
  return 0.5f * v * (1.0f + t) * mul;
}
__device__ __forceinline__ float gated_f32(int act, float gate, float up)
{
  if (act == kGateGeglu) {
    const float t = tanhf(0.7978845608028654f * (gate + 0.044715f * gate * gate * gate));
    return 0.5f * gate * (1.0f + t) * up;
  }
  return (gate / (1.0f + __expf(-gate))) * up;
}

// The value lane^1 holds (quad_perm [1,0,3,2]).
__device__ __forceinline__ float from_neighbour_lane(float v)
{
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));
}

// Sum over the 64 lanes of a wavefront; every lane receives the total.
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) { v += __shfl_xor(v, off, kWave); }
  return v;
}

}  // namespace vpq

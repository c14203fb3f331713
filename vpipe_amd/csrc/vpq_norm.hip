// RMSNorm of the rows of x ahead of the fused-QKV GEMV: the prologue of `qmv_qkv_rmsnorm_impl`
// (gpu-kernels/metal/quant/affine_qmv.metal:570-616) as a kernel of its own --
//   inv = rsqrt(sum(x^2) / K + eps) in fp32, out[k] = elt(float(x[k]) * inv * float(norm_w[k]))
// (norm_w carries Gemma's 1 + w already, folded in at load).  The reference keeps the normalized row in threadgroup
// memory of every GEMV workgroup; here it goes through a caller scratch of K elements per row, which the grouped
// GEMV launch then reads like any x (one small launch more, the same values).
// One workgroup of 256 threads per row; the sum of squares is a fixed-order tree (per-thread strided partials, a
// wave reduction, the four wavefronts in order), so the result is bit-reproducible.
#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

__global__ __launch_bounds__(256) void rmsnorm_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ norm_w,
                                                      uint16_t* __restrict__ out, int K, float eps)
{
  __shared__ float part[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint16_t* xr = x + (size_t)blockIdx.x * K;
  uint16_t* orow = out + (size_t)blockIdx.x * K;
  float sq = 0.0f;
  for (int k = threadIdx.x; k < K; k += 256) {
    const float v = bf16_bits_to_f32(xr[k]);
    sq = fmaf(v, v, sq);
  }
  sq = wave_sum(sq);
  if (lane == 0) { part[wave] = sq; }
  __syncthreads();
  const float total = ((part[0] + part[1]) + part[2]) + part[3];
  const float inv = rsqrtf(total / (float)K + eps);
  for (int k = threadIdx.x; k < K; k += 256) {
    orow[k] = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(xr[k]) * inv * bf16_bits_to_f32(norm_w[k]));
  }
}

}  // namespace

hipError_t launch_rmsnorm(hipStream_t st, const uint16_t* x, const uint16_t* norm_w, uint16_t* out, int K, int M, float eps)
{
  return launch_kernel(rmsnorm_kernel, dim3((unsigned)M), dim3(256), 0, st, x, norm_w, out, K, eps);
}

}  // namespace vpq

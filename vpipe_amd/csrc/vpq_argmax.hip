// Greedy tail of a decode step: index of the largest logit of a row, on the device, so that the
// sampled token feeds the next step's embedding gather without a host round trip
// (gpu-kernels/metal/ops/llm_elementwise.metal:2906-2941 argmax_f16; :2977-3028 argmax_partial_f16;
// :3030-3062 argmax_combine_f16).
//
// The result is the one of a left-to-right scan `if (v > best) take`: the LOWEST index among the
// entries that hold the maximum, and a NaN never wins (a row with nothing but NaNs gives 0, the
// scan's initial index).  Two stages: `parts` workgroups each reduce
// a contiguous slab of the row to a (value, index) pair, one workgroup per row combines the pairs.
// Every comparison is "greater, or equal with a lower index", which makes the reduction order
// irrelevant: the result is exact, not a matter of tolerance.
#include <mutex>

#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

constexpr int kNoIndex = 0x7fffffff;

// Scratch of the entry point that allocates nothing: (value, index) pairs of up to kArgmaxStaticRows rows x 256
// slabs, 128 KB per GPU for the life of the process.  In host code this name only stands for the symbol: the
// memory is reached through the address hipGetSymbolAddress returns for the current device.
__device__ __align__(256) float scratch[kArgmaxStaticRows * 256 * 2];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};

__device__ __forceinline__ void take_better(float& best, int& bi, float v, int i)
{
  if (v > best || (v == best && i < bi)) { best = v; bi = i; }
}

// (value, index) over the workgroup's 256 threads; thread 0 returns the winner.
__device__ __forceinline__ void block_argmax(float& best, int& bi)
{
  __shared__ float wv[4];
  __shared__ int wi[4];
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(best, off, kWave);
    const int oi = __shfl_xor(bi, off, kWave);
    take_better(best, bi, ov, oi);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { wv[wave] = best; wi[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int k = 1; k < 4; ++k) { take_better(best, bi, wv[k], wi[k]); }
  }
}

// grid (parts, rows): slab `blockIdx.x` of row `blockIdx.y` -> pair (row * parts + slab) of
// `partials`, two 4-byte slots each: the value as fp32, the index as int32.
__global__ __launch_bounds__(256) void argmax_partial_kernel(const uint16_t* __restrict__ logits,
                                                             float* __restrict__ partials, int V, int parts)
{
  const int row = blockIdx.y;
  const uint16_t* src = logits + (size_t)row * V;
  const int slab = (V + parts - 1) / parts;
  const int lo = blockIdx.x * slab;
  const int hi = lo + slab < V ? lo + slab : V;
  float best = -INFINITY;
  int bi = kNoIndex;
  for (int i = lo + (int)threadIdx.x; i < hi; i += 256) { take_better(best, bi, bf16_bits_to_f32(src[i]), i); }
  block_argmax(best, bi);
  if (threadIdx.x == 0) {
    float* slot = partials + 2 * ((size_t)row * parts + blockIdx.x);
    slot[0] = best;
    slot[1] = __int_as_float(bi);
  }
}

// grid (rows): the pairs of a row -> out_id[row]
__global__ __launch_bounds__(256) void argmax_combine_kernel(const float* __restrict__ partials, int* __restrict__ out_id,
                                                             int parts)
{
  const int row = blockIdx.x;
  float best = -INFINITY;
  int bi = kNoIndex;
  for (int p = threadIdx.x; p < parts; p += 256) {
    const float* slot = partials + 2 * ((size_t)row * parts + p);
    take_better(best, bi, slot[0], __float_as_int(slot[1]));
  }
  block_argmax(best, bi);
  if (threadIdx.x == 0) { out_id[row] = bi == kNoIndex ? 0 : bi; }
}

// One workgroup per row, no workspace (the single-threadgroup form of the reference).
__global__ __launch_bounds__(256) void argmax_row_kernel(const uint16_t* __restrict__ logits, int* __restrict__ out_id, int V)
{
  const int row = blockIdx.x;
  const uint16_t* src = logits + (size_t)row * V;
  float best = -INFINITY;
  int bi = kNoIndex;
  for (int i = threadIdx.x; i < V; i += 256) { take_better(best, bi, bf16_bits_to_f32(src[i]), i); }
  block_argmax(best, bi);
  if (threadIdx.x == 0) { out_id[row] = bi == kNoIndex ? 0 : bi; }
}

}  // namespace

int argmax_parts(int V)
{
  // about 2048 entries per slab, at most 256 slabs (one combine pass of 256 threads)
  const int p = (V + 2047) / 2048;
  return p < 1 ? 1 : (p > 256 ? 256 : p);
}

hipError_t argmax_static_scratch(float** out)
{
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { return e; }
  if (dev < 0 || dev >= kMaxDevices) { return hipErrorInvalidDevice; }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));     // this device's copy of the array
    if (e != hipSuccess) { return e; }
    if (ptr == nullptr) { return hipErrorInvalidSymbol; }
    g_scratch_ptr[dev] = static_cast<float*>(ptr);
  }
  *out = g_scratch_ptr[dev];
  return hipSuccess;
}

hipError_t launch_argmax_row(hipStream_t st, const uint16_t* logits, int* out_id, int V, int rows)
{
  return launch_kernel(argmax_row_kernel, dim3((unsigned)rows), dim3(256), 0, st, logits, out_id, V);
}

hipError_t launch_argmax_partial(hipStream_t st, const uint16_t* logits, float* partials, int V, int rows, int parts)
{
  return launch_kernel(argmax_partial_kernel, dim3((unsigned)parts, (unsigned)rows), dim3(256), 0, st, logits, partials, V,
                       parts);
}

hipError_t launch_argmax_combine(hipStream_t st, const float* partials, int* out_id, int rows, int parts)
{
  return launch_kernel(argmax_combine_kernel, dim3((unsigned)rows), dim3(256), 0, st, partials, out_id, parts);
}

}  // namespace vpq

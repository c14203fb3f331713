// The adapter's first factor: t[M,r] = elt(alpha * elt(x[M,K] . A[r,K]^T)), elt = bf16 or IEEE binary16 (the
// reference's VPIPE_ELT, gpu-kernels/metal/gemm/dense_gemm_mma.metal:28-33), any rank that is a multiple of 16
// up to kLoraMaxRank (the SCALED tile of gpu-kernels/metal/gemm/dense_gemm_mma.metal:227-273, driven by
// lora_gemm_a_, generative-models/minimax-h3/metal-minimax-h3-transformer.cc:1030-1067; the reference runs rank 16
// adapters and measures rank 384, metal-minimax-h3-transformer.h:365-367, .cc:1126-1132).
//
// r is tiny against K, so this is a bandwidth kernel on x: every row of x is read once, A (r x K,
// at most a few MB) stays in cache.  A workgroup owns 32 rows of x; its 8 wavefronts split K in
// interleaved 64-wide chunks and each contracts its chunks on v_mfma_f32_32x32x16_bf16 with fp32
// accumulators (r/32 tiles of 32 x 32), then the eight partial tiles are added through LDS in a
// fixed tree and wavefront 0 rounds and stores.  Within a chunk the four MFMAs take
// k = 32*half + 8*j + i (half = lane/32, j = MFMA, i < 8), so that a lane's operands for the
// whole chunk are 64 contiguous bytes of its row: two lanes cover a row's 128-byte line, for x
// and for A alike.  Ranks above 128 run as blocks of 128 columns of t on grid.y (x is read once per
// block; its 32 rows stay in L2 between the blocks of a workgroup's neighbours); a rank that is not a
// multiple of 32 leaves the upper half of its last tile unused (rows of A clamped, nothing stored).
#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

constexpr int kRows = 32;        // rows of x per workgroup
constexpr int kWaves = 8;        // K is split over them
constexpr int kChunk = 64;       // k-values per step

struct LoraAParams {
  const uint16_t* x;
  const uint16_t* a;
  uint16_t* t;
  int M, K, r;
  float alpha;
};

}  // namespace

template <int NT, bool F16 = false>
__global__ __launch_bounds__(kWaves * 64) void lora_a_kernel(const LoraAParams p)
{
  __shared__ float part[(kWaves / 2) * NT * 16 * 64];   // four wavefronts' tiles at a time

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 31;             // row of x (A operand) / row of the adapter (B operand)
  const int half = lane >> 5;
  const int m0 = blockIdx.x * kRows;
  const int r0 = blockIdx.y * 128;       // first column of t of this block
  const int xrow = (m0 + col < p.M) ? (m0 + col) : (p.M - 1);
  const uint16_t* xp = p.x + (size_t)xrow * p.K + half * 32;

  floatx16 acc[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) {
#pragma unroll
    for (int e = 0; e < 16; ++e) { acc[n][e] = 0.0f; }
  }

  const int chunks = p.K / kChunk;
  for (int c = wave; c < chunks; c += kWaves) {
    const uint16_t* xc = xp + (size_t)c * kChunk;
    bf16x8 xa[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) { xa[j] = *reinterpret_cast<const bf16x8*>(xc + 8 * j); }
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      const int arow = (r0 + n * 32 + col < p.r) ? (r0 + n * 32 + col) : (p.r - 1);
      const uint16_t* ac = p.a + (size_t)arow * p.K + half * 32 + (size_t)c * kChunk;
      bf16x8 ab[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) { ab[j] = *reinterpret_cast<const bf16x8*>(ac + 8 * j); }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (F16) {
          typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
          acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, xa[j]), __builtin_bit_cast(halfx8, ab[j]),
                                                          acc[n], 0, 0, 0);
        } else {
          acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[j], ab[j], acc[n], 0, 0, 0);
        }
      }
    }
  }

  // Tree over the wavefronts: 4..7 -> 0..3, 2..3 -> 0..1, 1 -> 0; the order is fixed.
#pragma unroll
  for (int step = kWaves / 2; step >= 1; step >>= 1) {
    if (wave >= step && wave < 2 * step) {
      float* dst = part + (size_t)(wave - step) * NT * 16 * 64;
#pragma unroll
      for (int n = 0; n < NT; ++n) {
#pragma unroll
        for (int e = 0; e < 16; ++e) { dst[(n * 16 + e) * 64 + lane] = acc[n][e]; }
      }
    }
    __syncthreads();
    if (wave < step) {
      const float* src = part + (size_t)wave * NT * 16 * 64;
#pragma unroll
      for (int n = 0; n < NT; ++n) {
#pragma unroll
        for (int e = 0; e < 16; ++e) { acc[n][e] += src[(n * 16 + e) * 64 + lane]; }
      }
    }
    __syncthreads();
  }

  if (wave == 0) {
    // D register e of lane l: row 8*(e/4) + 4*(l/32) + e%4 of x, column l%32 of the tile.
#pragma unroll
    for (int n = 0; n < NT; ++n) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m0 + 8 * (e >> 2) + 4 * half + (e & 3);
        if (m < p.M && r0 + n * 32 + col < p.r) {
          const float v = elt_bits_to_f32<F16>(f32_to_elt_bits<F16>(acc[n][e]));
          p.t[(size_t)m * p.r + r0 + n * 32 + col] = (uint16_t)f32_to_elt_bits<F16>(p.alpha * v);
        }
      }
    }
  }
}

hipError_t launch_lora_a(hipStream_t st, const uint16_t* x, const uint16_t* a, uint16_t* t, int M, int K, int r,
                         float alpha, bool f16)
{
  if (r < 16 || r % 16 != 0 || r > kLoraMaxRank) { return hipErrorInvalidValue; }
  LoraAParams p{x, a, t, M, K, r, alpha};
  const dim3 grid((unsigned)((M + kRows - 1) / kRows), (unsigned)((r + 127) / 128)), block(kWaves * 64);
  const int nt = r > 128 ? 4 : (r + 31) / 32;   // tiles of 32 columns per block
  if (f16) {
    switch (nt) {
      case 1: return launch_kernel(lora_a_kernel<1, true>, grid, block, 0, st, p);
      case 2: return launch_kernel(lora_a_kernel<2, true>, grid, block, 0, st, p);
      case 3: return launch_kernel(lora_a_kernel<3, true>, grid, block, 0, st, p);
      default: return launch_kernel(lora_a_kernel<4, true>, grid, block, 0, st, p);
    }
  }
  switch (nt) {
    case 1: return launch_kernel(lora_a_kernel<1>, grid, block, 0, st, p);
    case 2: return launch_kernel(lora_a_kernel<2>, grid, block, 0, st, p);
    case 3: return launch_kernel(lora_a_kernel<3>, grid, block, 0, st, p);
    default: return launch_kernel(lora_a_kernel<4>, grid, block, 0, st, p);
  }
}

}  // namespace vpq

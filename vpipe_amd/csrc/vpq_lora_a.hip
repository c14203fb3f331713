// The adapter's first factor: t[M,r] = elt(alpha * elt(x[M,K] . A[r,K]^T)), elt = bf16 or IEEE binary16 (the
// reference's VPIPE_ELT, gpu-kernels/metal/gemm/dense_gemm_mma.metal:28-33), any rank that is a multiple of 8
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

// Ranks up to 32 (one tile of 32 columns; what the video-DiT adapters and the reference's rank-16 adapters run): the
// same decomposition with x AND A brought in by 128-bit direct-to-LDS loads -- one instruction covers 8 rows x 128
// contiguous bytes (whole cache lines) instead of 16-byte pieces of 32 rows, which is what held the kernel above to a
// third of the HBM rate (16320 x 5120 at rank 32: 58 -> 34 us; x is read once either way).  Every wavefront owns a
// ring of two 8 KB slots (32 rows of x and 32 rows of A, 64 values of K each, the 16-byte pieces of a row XOR-swizzled
// by the row so that the operand reads do not collide on banks) and walks its chunks with two in flight; the waits
// are counted by hand and the LDS reads are asm so that the compiler adds none of its own.  Within a chunk MFMA j
// takes k = 16 j + 8 (lane / 32) + i.
namespace {

constexpr int kDmaSlot = 8192, kDmaSlots = 2;

__device__ __forceinline__ void lora_dma16(uint32_t lds_dst, const void* src)
{
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_dst);
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "{m0}"(m0v) : "memory");
}

__device__ __forceinline__ bf16x8 lora_lds_read(uint32_t addr)
{
  bf16x8 v;
  asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
  return v;
}

}  // namespace

template <bool F16>
__global__ __launch_bounds__(kWaves * 64) void lora_a_dma_kernel(const LoraAParams p)
{
  __shared__ __attribute__((aligned(16))) uint8_t ring[kWaves * kDmaSlots * kDmaSlot];      // 128 KB; the tree reuses it

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 31, half = lane >> 5;
  const int m0 = blockIdx.x * kRows;
  const uint32_t ring_a = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)ring +
                          (uint32_t)(wave * kDmaSlots * kDmaSlot);
  // request: instruction i covers rows 8 i .. 8 i + 7; lane l takes row 8 i + l / 8 and the piece (l % 8) ^ (row & 7)
  const uint16_t* xsrc[4];
  const uint16_t* asrc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int R = 8 * i + (lane >> 3), piece = (lane & 7) ^ (R & 7);
    const int xr = (m0 + R < p.M) ? (m0 + R) : (p.M - 1);
    const int ar = R < p.r ? R : (p.r - 1);
    xsrc[i] = p.x + (size_t)xr * p.K + piece * 8;
    asrc[i] = p.a + (size_t)ar * p.K + piece * 8;
  }
  // operand read of MFMA j: row `col`, piece 2 j + half
  uint32_t frag_off[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) { frag_off[j] = (uint32_t)(col * 128 + (((2 * j + half) ^ (col & 7)) * 16)); }

  const int chunks = p.K / kChunk;
  const int mine = (chunks - wave + kWaves - 1) / kWaves;      // chunks wave, wave + 8, ...; may be 0
  auto request = [&](int i, int slot) {
    const int ii = i < mine ? i : mine - 1;                      // past the end: the last chunk again (uniform counts)
    const size_t k0 = (size_t)(wave + ii * kWaves) * kChunk;
    const uint32_t dst = ring_a + (uint32_t)(slot * kDmaSlot);
#pragma unroll
    for (int q = 0; q < 4; ++q) { lora_dma16(dst + q * 1024, xsrc[q] + k0); }
#pragma unroll
    for (int q = 0; q < 4; ++q) { lora_dma16(dst + 4096 + q * 1024, asrc[q] + k0); }
  };

  floatx16 acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) { acc[e] = 0.0f; }
  if (mine > 0) {
    request(0, 0);
    request(1, 1);
    for (int i = 0; i < mine; ++i) {
      const int slot = i & 1;
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");          // everything but the other slot's eight loads
      const uint32_t base = ring_a + (uint32_t)(slot * kDmaSlot);
      bf16x8 xa[4], ab[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) { xa[j] = lora_lds_read(base + frag_off[j]); }
#pragma unroll
      for (int j = 0; j < 4; ++j) { ab[j] = lora_lds_read(base + 4096 + frag_off[j]); }
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(xa[0]), "+v"(xa[1]), "+v"(xa[2]), "+v"(xa[3]), "+v"(ab[0]), "+v"(ab[1]), "+v"(ab[2]), "+v"(ab[3])
                   :
                   : "memory");
      request(i + 2, slot);                                      // the slot is free: its content is in registers
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (F16) {
          typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
          acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, xa[j]), __builtin_bit_cast(halfx8, ab[j]), acc,
                                                       0, 0, 0);
        } else {
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[j], ab[j], acc, 0, 0, 0);
        }
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");            // the requests past the end still write the slots
  }
  __syncthreads();                                              // every wavefront's ring is quiet: the tree may use it

  float* part = reinterpret_cast<float*>(ring);
#pragma unroll
  for (int step = kWaves / 2; step >= 1; step >>= 1) {
    if (wave >= step && wave < 2 * step) {
      float* dst = part + (size_t)(wave - step) * 16 * 64;
#pragma unroll
      for (int e = 0; e < 16; ++e) { dst[e * 64 + lane] = acc[e]; }
    }
    __syncthreads();
    if (wave < step) {
      const float* src = part + (size_t)wave * 16 * 64;
#pragma unroll
      for (int e = 0; e < 16; ++e) { acc[e] += src[e * 64 + lane]; }
    }
    __syncthreads();
  }
  if (wave == 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int m = m0 + 8 * (e >> 2) + 4 * half + (e & 3);
      if (m < p.M && col < p.r) {
        const float v = elt_bits_to_f32<F16>(f32_to_elt_bits<F16>(acc[e]));
        p.t[(size_t)m * p.r + col] = (uint16_t)f32_to_elt_bits<F16>(p.alpha * v);
      }
    }
  }
}

hipError_t launch_lora_a(hipStream_t st, const uint16_t* x, const uint16_t* a, uint16_t* t, int M, int K, int r,
                         float alpha, bool f16)
{
  if (r < 8 || r % 8 != 0 || r > kLoraMaxRank) { return hipErrorInvalidValue; }
  LoraAParams p{x, a, t, M, K, r, alpha};
  const dim3 grid((unsigned)((M + kRows - 1) / kRows), (unsigned)((r + 127) / 128)), block(kWaves * 64);
  if (r <= 32) {
    const dim3 g1((unsigned)((M + kRows - 1) / kRows));
    return f16 ? launch_kernel(lora_a_dma_kernel<true>, g1, block, 0, st, p)
               : launch_kernel(lora_a_dma_kernel<false>, g1, block, 0, st, p);
  }
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

// QMM main kernel: y[M,N] = x[M,K] . bf16(W)^T (+ t[M,r] . B[N,r]^T) on
// v_mfma_f32_32x32x16_bf16 with fp32 accumulation.
//
// One workgroup (4 wavefronts, 2x2) owns a 256(M) x 128(N) tile of y; each
// wavefront accumulates 128 x 64 of it in 128 registers.  Per 64-wide K step (one
// quantization group, so one scale/bias per weight row per step):
//   x tile [256,64] bf16   global -> LDS by 128-bit direct-to-LDS loads (no
//                          registers, no VALU), 8 rows x 128 contiguous bytes per
//                          load instruction;
//   W tile [128,64]        32 codes per thread: global -> registers ->
//                          fp32 fma(s,q,b) -> bf16 RNE -> LDS.  The value is
//                          bf16_rne(fp32(s*q+b)), the tile arithmetic of
//                          gpu-kernels/metal/quant/affine_qmm_steel.metal:78-96
//                          (Compute=float) and affine_qmm_mma.metal:96-104.
// LDS rows are 128 bytes (64 bf16) with the eight 16-byte chunks of a row stored
// at position chunk ^ ((row >> 1) & 7): the 128-bit operand reads of the MFMAs
// (lane = row) then spread over all 64 banks.  Two LDS stages: while the MFMAs
// consume stage s, the loads of stage s+1 are in flight and its W tile is
// dequantized into the other stage; one barrier per step.
// With a LoRA the same accumulators take r more values of K from t[M,r] and
// B[N,r] (dense, both through direct-to-LDS loads) before the single store
// (gpu-kernels/metal/gemm/dense_gemm_mma.metal:297-348).
#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

constexpr int TM = 256, TN = 128, TK = 64;
constexpr int kThreads = 256;
constexpr int kRowB = TK * 2;                       // 128 bytes per LDS row
constexpr int kStageBytes = (TM + TN) * kRowB;      // 48 KB
constexpr int kLds = 2 * kStageBytes;               // 96 KB

struct TileParams {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  const uint16_t* x;
  uint16_t* y;
  const uint16_t* lora_t;   // [M,r] or nullptr
  const uint16_t* lora_b;   // [N,r]
  int K, N, M, r;
  int tiles_m, tiles_n;
};

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

// Byte I of a dword as fp32 (selects v_cvt_f32_ubyteI).
template <int I>
__device__ __forceinline__ float ubyte_f32(uint32_t v) { return (float)((v >> (8 * I)) & 0xffu); }

// 8 nibbles of one word -> 8 bf16 of fma(s, q, b), as one 16-byte LDS chunk.
__device__ __forceinline__ uint4 dequant_word(uint32_t word, float s, float b)
{
  const uint32_t lo = word & 0x0f0f0f0fu;          // q0 q2 q4 q6
  const uint32_t hi = (word >> 4) & 0x0f0f0f0fu;   // q1 q3 q5 q7
  const float v0 = fmaf(s, ubyte_f32<0>(lo), b);
  const float v1 = fmaf(s, ubyte_f32<0>(hi), b);
  const float v2 = fmaf(s, ubyte_f32<1>(lo), b);
  const float v3 = fmaf(s, ubyte_f32<1>(hi), b);
  const float v4 = fmaf(s, ubyte_f32<2>(lo), b);
  const float v5 = fmaf(s, ubyte_f32<2>(hi), b);
  const float v6 = fmaf(s, ubyte_f32<3>(lo), b);
  const float v7 = fmaf(s, ubyte_f32<3>(hi), b);
  uint4 o;
  o.x = pack_bf16x2(v0, v1);
  o.y = pack_bf16x2(v2, v3);
  o.z = pack_bf16x2(v4, v5);
  o.w = pack_bf16x2(v6, v7);
  return o;
}

}  // namespace

template <bool LORA>
__global__ __launch_bounds__(kThreads) void qmm_tile_kernel(const TileParams p)
{
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // Consecutive workgroups walk M first: they share one weight tile.
  const int tile = blockIdx.x;
  const int tm = tile % p.tiles_m;
  const int tn = tile / p.tiles_m;
  const int m0 = tm * TM, n0 = tn * TN;
  const int KT = p.K / TK;

  // ---- x tile: 32 direct-to-LDS loads per step, 8 per wavefront.  Load i of wave w covers
  //      tile rows (8w + i)*8 .. +8; lane l takes row l/8, LDS position l%8.
  const uint8_t* xblk = reinterpret_cast<const uint8_t*>(p.x) + (size_t)m0 * p.K * 2;
  uint32_t a_off[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = (wave * 8 + i) * 8 + (lane >> 3);
    const int chunk = swz(row, lane & 7);
    const int rg = (m0 + row < p.M) ? row : (p.M - 1 - m0);
    a_off[i] = (uint32_t)rg * (uint32_t)p.K * 2u + (uint32_t)chunk * 16u;
  }
  // ---- W tile: thread t dequantizes 32 codes of row t/2 (k half t%2) per step.
  const int qrow = tid >> 1, qhalf = tid & 1;
  const int qrg = (n0 + qrow < p.N) ? (n0 + qrow) : (p.N - 1);
  const uint8_t* wrow = reinterpret_cast<const uint8_t*>(p.w) + (size_t)qrg * (p.K >> 1) + qhalf * 16;
  const uint16_t* srow = p.scales + (size_t)qrg * (p.K >> 6);
  const uint16_t* brow = p.biases + (size_t)qrg * (p.K >> 6);
  int b_dst[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) { b_dst[i] = TM * kRowB + qrow * kRowB + swz(qrow, qhalf * 4 + i) * 16; }

  auto issue_x = [&](int step, int stage) {
    const uint8_t* src = xblk + (size_t)step * (TK * 2);
    uint8_t* dst = lds + stage * kStageBytes + wave * (64 * kRowB);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + a_off[i]),
                                       (__attribute__((address_space(3))) void*)(dst + i * (8 * kRowB)), 16, 0, 0);
    }
  };

  floatx16 acc[2][4];   // [jt: 32 weight rows][it: 32 x rows]
#pragma unroll
  for (int jt = 0; jt < 2; ++jt) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
#pragma unroll
      for (int e = 0; e < 16; ++e) { acc[jt][it][e] = 0.0f; }
    }
  }

  const int frow = lane & 31;      // row of a 32-row operand fragment
  const int fkh = lane >> 5;       // which 8 of the 16 k
  // Operand read addresses (stage-relative) for k-step 0; k-step ks adds chunk 2*ks.
  int w_rd[2], x_rd[4];
#pragma unroll
  for (int jt = 0; jt < 2; ++jt) { w_rd[jt] = TM * kRowB + (wn * 64 + jt * 32 + frow) * kRowB; }
#pragma unroll
  for (int it = 0; it < 4; ++it) { x_rd[it] = (wm * 128 + it * 32 + frow) * kRowB; }
  const int w_sw = ((wn * 64 + frow) >> 1) & 7;   // jt*32 does not change (row >> 1) & 7
  const int x_sw = ((wm * 128 + frow) >> 1) & 7;

  auto mma_stage = [&](int stage, int ksteps) {
    const uint8_t* base = lds + stage * kStageBytes;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks < ksteps) {
        const int cw = ((2 * ks + fkh) ^ w_sw) * 16;
        const int cx = ((2 * ks + fkh) ^ x_sw) * 16;
        bf16x8 wf[2], xf[4];
#pragma unroll
        for (int jt = 0; jt < 2; ++jt) { wf[jt] = *reinterpret_cast<const bf16x8*>(base + w_rd[jt] + cw); }
#pragma unroll
        for (int it = 0; it < 4; ++it) { xf[it] = *reinterpret_cast<const bf16x8*>(base + x_rd[it] + cx); }
#pragma unroll
        for (int jt = 0; jt < 2; ++jt) {
#pragma unroll
          for (int it = 0; it < 4; ++it) {
            acc[jt][it] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[jt], xf[it], acc[jt][it], 0, 0, 0);
          }
        }
      }
    }
  };

  // ---- prologue: stage 0 ----
  uint4 codes = *reinterpret_cast<const uint4*>(wrow);
  float sc = bf16_bits_to_f32(srow[0]), bi = bf16_bits_to_f32(brow[0]);
  issue_x(0, 0);
  {
    const uint32_t cw4[4] = {codes.x, codes.y, codes.z, codes.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { *reinterpret_cast<uint4*>(lds + b_dst[i]) = dequant_word(cw4[i], sc, bi); }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  for (int s = 0; s < KT; ++s) {
    const int stage = s & 1;
    const bool more = s + 1 < KT;
    if (more) {
      // codes and scales first, then the x tile: the dequant below then waits for its own
      // loads only, with the eight direct-to-LDS loads still in flight.
      codes = *reinterpret_cast<const uint4*>(wrow + (size_t)(s + 1) * (TK / 2));
      sc = bf16_bits_to_f32(srow[s + 1]);
      bi = bf16_bits_to_f32(brow[s + 1]);
      issue_x(s + 1, stage ^ 1);
    }
    mma_stage(stage, 4);
    if (more) {
      const uint32_t cw4[4] = {codes.x, codes.y, codes.z, codes.w};
      uint8_t* nb = lds + (stage ^ 1) * kStageBytes;
#pragma unroll
      for (int i = 0; i < 4; ++i) { *reinterpret_cast<uint4*>(nb + b_dst[i]) = dequant_word(cw4[i], sc, bi); }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }

  if (LORA) {
    // r more values of K: t[M,r] against B[N,r], 64 per step, both tiles by direct-to-LDS loads.
    const int steps = (p.r + TK - 1) / TK;
    for (int st = 0; st < steps; ++st) {
      const int kleft = p.r - st * TK;                 // >= 32, a multiple of 32
      const int chunks = kleft >= TK ? 8 : (kleft >> 3);
      uint8_t* sbase = lds;                            // stage 0 is free after the last barrier
      // t tile: 256 rows, as the x tile.
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int row = (wave * 8 + i) * 8 + (lane >> 3);
        const int chunk = swz(row, lane & 7);
        const int rg = (m0 + row < p.M) ? (m0 + row) : (p.M - 1);
        if (chunk < chunks) {
          __builtin_amdgcn_global_load_lds(
              (const __attribute__((address_space(1))) void*)(p.lora_t + (size_t)rg * p.r + st * TK + chunk * 8),
              (__attribute__((address_space(3))) void*)(sbase + wave * (64 * kRowB) + i * (8 * kRowB)), 16, 0, 0);
        }
      }
      // B tile: 128 rows, 4 loads per wavefront.
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = (wave * 4 + i) * 8 + (lane >> 3);
        const int chunk = swz(row, lane & 7);
        const int rg = (n0 + row < p.N) ? (n0 + row) : (p.N - 1);
        if (chunk < chunks) {
          __builtin_amdgcn_global_load_lds(
              (const __attribute__((address_space(1))) void*)(p.lora_b + (size_t)rg * p.r + st * TK + chunk * 8),
              (__attribute__((address_space(3))) void*)(sbase + TM * kRowB + wave * (32 * kRowB) + i * (8 * kRowB)), 16, 0, 0);
        }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      mma_stage(0, chunks >> 1);
      __syncthreads();
    }
  }

  // ---- store: lane holds, for x row m = lane%32 of each it, 4 consecutive n per register quad ----
  const bool vec_ok = (p.N & 3) == 0;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int m = m0 + wm * 128 + it * 32 + frow;
    if (m >= p.M) { continue; }
    uint16_t* yrow = p.y + (size_t)m * p.N;
#pragma unroll
    for (int jt = 0; jt < 2; ++jt) {
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int n = n0 + wn * 64 + jt * 32 + rq * 8 + fkh * 4;
        if (n >= p.N) { continue; }
        const float v0 = acc[jt][it][rq * 4 + 0], v1 = acc[jt][it][rq * 4 + 1];
        const float v2 = acc[jt][it][rq * 4 + 2], v3 = acc[jt][it][rq * 4 + 3];
        if (vec_ok && n + 3 < p.N) {
          uint2 o;
          o.x = pack_bf16x2(v0, v1);
          o.y = pack_bf16x2(v2, v3);
          *reinterpret_cast<uint2*>(yrow + n) = o;
        } else {
          const float v[4] = {v0, v1, v2, v3};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (n + e < p.N) { yrow[n + e] = (uint16_t)f32_to_bf16_bits(v[e]); }
          }
        }
      }
    }
  }
}

hipError_t launch_qmm_tile(hipStream_t st, const GemmArgs& a)
{
  TileParams p;
  p.w = a.w; p.scales = a.scales; p.biases = a.biases; p.x = a.x; p.y = a.y;
  p.lora_t = a.lora_t; p.lora_b = a.lora_b;
  p.K = a.K; p.N = a.N; p.M = a.M; p.r = a.r;
  p.tiles_m = (a.M + TM - 1) / TM;
  p.tiles_n = (a.N + TN - 1) / TN;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n)), block(kThreads);
  static bool attr_done[2] = {false, false};
  auto launch = [&](auto kern, int slot) -> hipError_t {
    if (!attr_done[slot]) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
      if (e != hipSuccess) { return e; }
      attr_done[slot] = true;
    }
    return launch_kernel(kern, grid, block, (size_t)kLds, st, p);
  };
  return a.lora_t != nullptr ? launch(qmm_tile_kernel<true>, 0) : launch(qmm_tile_kernel<false>, 1);
}

}  // namespace vpq

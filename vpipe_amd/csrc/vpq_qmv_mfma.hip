// QMV (1 <= M <= 16) as a bandwidth kernel on bf16 MFMA.
//
// Work decomposition.  The [N,K] pack is cut into items of 16 weight rows x 512
// k-values (8 quantization groups, 4 KB of codes).  A workgroup owns one 16-row
// tile of N and a K range; its wavefronts take the items of that range
// round-robin and their partial sums are added through LDS at the end (split-K
// inside the workgroup).
//
// Per item and wavefront:
//   codes   16 rows x 256 bytes, fetched with 128-bit direct-to-LDS loads in
//           which 16 consecutive lanes cover 256 contiguous bytes of one row
//           (full cache lines), into a wave-private LDS buffer.  The 16-byte
//           chunks of a row are stored XOR-swizzled so that the later 64-bit
//           reads (lane = weight row) do not collide on LDS banks.
//   scales, biases   one 128-bit load per lane (8 groups of the lane's row).
//   x       M <= 4: the wavefront loads its 512-value slice of each row with
//           one coalesced 128-bit load per lane, reorders it once and parks it
//           in wave-private LDS, from where every lane reads its MFMA A
//           operands.  M > 4: each lane loads its A operands from global/L2.
//   math    the integer codes are turned into bf16 (128 + q) by one
//           v_and_or_b32 per nibble pair and contracted with x on
//           v_mfma_f32_16x16x32_bf16, two MFMAs per group.  The accumulator is
//           seeded with -128*sum(x) so the MFMA result is exactly the group's
//           sum(x*q); then y += scale*sum(x*q) + bias*sum(x) in fp32 -- the
//           factored form of gpu-kernels/metal/quant/affine_qmv.metal:151-174,
//           with sum(x) in fp32 (the reference forms it in bf16 quad sums,
//           affine_qmv.metal:60-67, an error source not reproduced here).
// The weight is never rounded to bf16: q, 128+q and x are exact in bf16, the
// products are exact in fp32.
//
// No inline-assembly VALU instruction may sit near the MFMAs: the compiler's
// hazard recogniser cannot see what such a statement writes, and a register an
// MFMA in flight still reads can be overwritten.  Everything here is plain C
// and builtins.
#include <atomic>

#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

constexpr int kTileN = 16;
constexpr int kKS = 512;                 // k-values per item
constexpr int kG = kKS / kGroup;         // groups per item (8)
constexpr int kRowBytes = kKS / 2;       // code bytes per row per item (256)
constexpr int kItemBytes = kTileN * kRowBytes;
constexpr int kXRowBytes = kKS * 2 + 16; // LDS stride of one staged x row (bf16) + pad
constexpr int kXsumBytes = 4 * kG * 4;   // -128*sum(x) per staged row and group (fp32)
constexpr int kMaxWaves = 16;

struct QmvParams {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  const uint16_t* x;
  void* y;
  const uint16_t* residual;
  int K, N, M;
  int slices;            // K / 512
  int wave_lds_bytes;    // codes buffer + staged x rows of one wavefront
  // Grouped launch (nseg > 1): workgroup blockIdx.x belongs to the segment whose tile range
  // holds it; each segment is its own [N_i, K] pack and output.
  int gate_act;          // rows are interleaved gate|up; y is [M, N/2] = act(gate) * up (1 SwiGLU, 2 GEGLU)
  int nseg;
  QmvSeg seg[4];
  int seg_tile_end[4];
};

// Eight nibbles of one packed word -> eight bf16 values 128+q, element order
// [k0,k4,k1,k5,k2,k6,k3,k7] (nibbles i and i+4 sit 16 bits apart, which is what
// one (w >> 4i) & 0x000f000f extracts into the two halves of a dword).  `mask`
// and `magic` arrive as opaque register values so that each pair costs a single
// v_and_or_b32 (VOP3 on gfx9 encodes no literal operand).
__device__ __forceinline__ bf16x8 codes_to_bf16(uint32_t word, uint32_t mask, uint32_t magic)
{
  u32x4 v;
  v[0] = (word & mask) | magic;
  v[1] = ((word >> 4) & mask) | magic;
  v[2] = ((word >> 8) & mask) | magic;
  v[3] = ((word >> 12) & mask) | magic;
  return __builtin_bit_cast(bf16x8, v);
}

// Eight consecutive bf16 of x -> the element order codes_to_bf16 produces.
__device__ __forceinline__ uint4 permute_x(uint4 d)
{
  uint4 v;
  v.x = __builtin_amdgcn_perm(d.z, d.x, 0x05040100u);  // x0,x4
  v.y = __builtin_amdgcn_perm(d.z, d.x, 0x07060302u);  // x1,x5
  v.z = __builtin_amdgcn_perm(d.w, d.y, 0x05040100u);  // x2,x6
  v.w = __builtin_amdgcn_perm(d.w, d.y, 0x07060302u);  // x3,x7
  return v;
}

// Sum over each aligned run of 8 lanes (one quantization group of the staged x slice);
// every lane of the run receives it.  Three DPP steps: lane^1, lane^2, then the mirror
// image inside the run, which exchanges its two quads.
__device__ __forceinline__ float sum_over_8_lanes(float v)
{
  int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false);   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false);       // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false);      // row_half_mirror
  v += __builtin_bit_cast(float, t);
  return v;
}

}  // namespace

// MR: accumulator registers per lane = ceil(M/4).  Row m of x sits in MFMA row
// 4*(m%4) + m/4, so that output row m is register m/4 of lane group m%4 and
// M <= 4 needs a single accumulator register.
// XLDS: x is staged through wave-private LDS (M <= 4).
template <int MR, bool XLDS, bool F32OUT>
__global__ __launch_bounds__(1024) void qmv_mfma_kernel(const QmvParams p)
{
  constexpr int CH = kRowBytes / 16;          // 16-byte chunks per row (16)
  constexpr int ROWS_PER_LOAD = kWave / CH;   // rows one load instruction covers (4)
  constexpr int NLOAD = kTileN / ROWS_PER_LOAD;

  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int NW = blockDim.x >> 6;
  uint8_t* wbuf = lds + wave * p.wave_lds_bytes;
  uint8_t* xbuf = wbuf + kItemBytes;
  float* xsum = reinterpret_cast<float*>(xbuf + p.M * kXRowBytes);   // [M][8 groups], XLDS only
  const int xsum_row = (lane >> 4) < p.M ? (lane >> 4) : p.M - 1;
  float* red = reinterpret_cast<float*>(lds + NW * p.wave_lds_bytes);

  // The pack this workgroup works on: the single one, or its segment of a grouped launch.
  const uint32_t* w_ = p.w;
  const uint16_t* scales_ = p.scales;
  const uint16_t* biases_ = p.biases;
  void* y_ = p.y;
  int N_ = p.N;
  int tile = blockIdx.x;
  if (p.nseg > 1) {
    int s = 0;
    while (s + 1 < p.nseg && tile >= p.seg_tile_end[s]) { ++s; }
    if (s > 0) { tile -= p.seg_tile_end[s - 1]; }
    w_ = p.seg[s].w; scales_ = p.seg[s].scales; biases_ = p.seg[s].biases; y_ = p.seg[s].y; N_ = p.seg[s].N;
  }
  const int n0 = tile * kTileN;
  const int fr = lane & 15;                 // MFMA row (A) / column (B, D) of this lane
  const int g = lane >> 4;                  // k sub-block of this lane
  const int m_real = 4 * (fr & 3) + (fr >> 2);
  // MFMA rows beyond M produce outputs nobody stores; they read the last live row.
  const int x_row = m_real < p.M ? m_real : p.M - 1;
  const int Kg = p.K >> 6;
  const uint32_t row_bytes_total = (uint32_t)p.K >> 1;

  // Wave-uniform bases (tile origin) + 32-bit per-lane offsets.
  const uint8_t* wtile = reinterpret_cast<const uint8_t*>(w_) + (size_t)n0 * row_bytes_total;
  uint32_t code_off[NLOAD];
#pragma unroll
  for (int i = 0; i < NLOAD; ++i) {
    const int row = i * ROWS_PER_LOAD + lane / CH;
    const int chunk = (lane % CH) ^ (row & (CH - 1));
    const int rrow = (n0 + row < N_) ? row : (N_ - 1 - n0);
    code_off[i] = (uint32_t)rrow * row_bytes_total + (uint32_t)chunk * 16;
  }
  const int srow = (n0 + fr < N_) ? fr : (N_ - 1 - n0);
  const uint16_t* stile = scales_ + (size_t)n0 * Kg;
  const uint16_t* btile = biases_ + (size_t)n0 * Kg;
  const uint32_t sb_off = (uint32_t)srow * (uint32_t)Kg;
  // LDS byte address of this lane's two words of group 0: row fr, chunk g/2 (swizzled), half g%2.
  const int lds_code0 = fr * kRowBytes + (g & 1) * 8;
  const int lds_chunk0 = (g >> 1) ^ fr;
  const int lds_x0 = x_row * kXRowBytes + g * 32;

  uint32_t magic = 0x43004300u;             // bf16 128.0 in both halves
  uint32_t mask = 0x000f000fu;
  asm volatile("" : "+v"(magic));           // no instruction: only hides the constants
  asm volatile("" : "+s"(mask));            // from constant folding (see codes_to_bf16)
  u32x4 m128;
  m128[0] = m128[1] = m128[2] = m128[3] = 0xc300c300u;  // bf16 -128.0
  const bf16x8 neg128 = __builtin_bit_cast(bf16x8, m128);

  float acc[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) { acc[r] = 0.0f; }

  for (int sl = wave; sl < p.slices; sl += NW) {
    // 1. codes: global -> LDS, no registers in between.
    const uint8_t* wbase = wtile + (size_t)sl * kRowBytes;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(wbase + code_off[i]),
          (__attribute__((address_space(3))) void*)(wbuf + i * (kWave * 16)), 16, 0, 0);
    }
    // 2. scales and biases of this lane's row: 8 groups each.
    const uint4 sv = *reinterpret_cast<const uint4*>(stile + (size_t)sl * kG + sb_off);
    const uint4 bv = *reinterpret_cast<const uint4*>(btile + (size_t)sl * kG + sb_off);
    // 3. x.
    bf16x8 afrag[XLDS ? 1 : 2 * kG];
    if (XLDS) {
      // Lane l takes k = 8l..8l+7 of each row: one coalesced 1 KB load per row.
      const uint16_t* xs = p.x + (size_t)sl * kKS + lane * 8;
      // The 8 lanes that hold one group also form -128 * sum(x) of that group on the way.
      for (int m = 0; m < p.M; ++m) {
        const uint4 d = *reinterpret_cast<const uint4*>(xs + (size_t)m * p.K);
        *reinterpret_cast<uint4*>(xbuf + m * kXRowBytes + lane * 16) = permute_x(d);
        float s8 = (bf16_lo_to_f32(d.x) + bf16_hi_to_f32(d.x)) + (bf16_lo_to_f32(d.y) + bf16_hi_to_f32(d.y)) +
                   (bf16_lo_to_f32(d.z) + bf16_hi_to_f32(d.z)) + (bf16_lo_to_f32(d.w) + bf16_hi_to_f32(d.w));
        s8 = sum_over_8_lanes(s8);
        if ((lane & 7) == 0) { xsum[m * kG + (lane >> 3)] = -128.0f * s8; }
      }
    } else {
      const uint16_t* xp = p.x + (size_t)x_row * p.K + (size_t)sl * kKS + g * 16;
#pragma unroll
      for (int grp = 0; grp < kG; ++grp) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          afrag[2 * grp + t] = __builtin_bit_cast(
              bf16x8, permute_x(*reinterpret_cast<const uint4*>(xp + grp * kGroup + t * 8)));
        }
      }
    }
    // 4. codes have landed in this wave's buffer.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    const uint32_t sd[4] = {sv.x, sv.y, sv.z, sv.w};
    const uint32_t bd[4] = {bv.x, bv.y, bv.z, bv.w};
    float xn[kG];                               // XLDS: -128 * sum(x) per group, row lane/16
    if (XLDS) {
      const floatx4 lo = *reinterpret_cast<const floatx4*>(xsum + xsum_row * kG);
      const floatx4 hi = *reinterpret_cast<const floatx4*>(xsum + xsum_row * kG + 4);
#pragma unroll
      for (int i = 0; i < 4; ++i) { xn[i] = lo[i]; xn[4 + i] = hi[i]; }
    }
#pragma unroll
    for (int grp = 0; grp < kG; ++grp) {
      bf16x8 a0, a1;
      if (XLDS) {
        a0 = *reinterpret_cast<const bf16x8*>(xbuf + lds_x0 + grp * 128);
        a1 = *reinterpret_cast<const bf16x8*>(xbuf + lds_x0 + grp * 128 + 16);
      } else {
        a0 = afrag[2 * grp];
        a1 = afrag[2 * grp + 1];
      }
      // -128 * sum(x) of the group, in the accumulator layout (same for every column): from the
      // staging pass when x went through LDS (only register 0 is a live row then), else by MFMA.
      floatx4 xneg = {0.f, 0.f, 0.f, 0.f};
      if (XLDS) {
        xneg[0] = xn[grp];
      } else {
        xneg = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, neg128, xneg, 0, 0, 0);
        xneg = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, neg128, xneg, 0, 0, 0);
      }
      const int chunk = (2 * grp) ^ lds_chunk0;      // == (2*grp + g/2) ^ fr
      const uint2 cw = *reinterpret_cast<const uint2*>(wbuf + lds_code0 + chunk * 16);
      floatx4 s4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, codes_to_bf16(cw.x, mask, magic), xneg, 0, 0, 0);
      s4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, codes_to_bf16(cw.y, mask, magic), s4, 0, 0, 0);
      const float s = (grp & 1) ? bf16_hi_to_f32(sd[grp >> 1]) : bf16_lo_to_f32(sd[grp >> 1]);
      const float b = (grp & 1) ? bf16_hi_to_f32(bd[grp >> 1]) : bf16_lo_to_f32(bd[grp >> 1]);
      const float b2 = b * -0.0078125f;              // bias * sum(x) = (bias / -128) * xneg
#pragma unroll
      for (int r = 0; r < MR; ++r) {
        acc[r] = fmaf(s, s4[r], acc[r]);
        acc[r] = fmaf(b2, xneg[r], acc[r]);
      }
    }
  }

  // Sum the wavefronts' partials.  acc[r] of lane l is y[m = 4r + l/16][n0 + l%16].
#pragma unroll
  for (int r = 0; r < MR; ++r) { red[(wave * MR + r) * kWave + lane] = acc[r]; }
  __syncthreads();

  const int t = threadIdx.x;
  float total = 0.0f;
  int m = 0, n = 0;
  const bool owner = t < MR * kWave;
  if (owner) {
    const int r = t >> 6, l = t & 63;
    for (int wv = 0; wv < NW; ++wv) { total += red[(wv * MR + r) * kWave + l]; }
    m = 4 * r + (l >> 4);
    n = n0 + (l & 15);
  }
  const bool valid = owner && m < p.M && n < N_;

  if (p.gate_act) {
    // Lanes 2j and 2j+1 hold the gate and the up sum of feature (n0 + 2j) / 2; N is even, so both
    // are valid or neither.
    const float up = from_neighbour_lane(total);
    if (valid && (t & 1) == 0) {
      const float v = gated_f32(p.gate_act, total, up);
      const size_t o = (size_t)m * (N_ >> 1) + (n >> 1);
      if (F32OUT) {
        reinterpret_cast<float*>(y_)[o] = v;
      } else {
        reinterpret_cast<uint16_t*>(y_)[o] = (uint16_t)f32_to_bf16_bits(v);
      }
    }
    return;
  }
  if (valid) {
    const size_t o = (size_t)m * N_ + n;
    if (F32OUT) {
      reinterpret_cast<float*>(y_)[o] = total;
    } else {
      uint32_t v = f32_to_bf16_bits(total);
      if (p.residual != nullptr) {
        v = f32_to_bf16_bits(bf16_bits_to_f32(v) + bf16_bits_to_f32(p.residual[o]));
      }
      reinterpret_cast<uint16_t*>(y_)[o] = (uint16_t)v;
    }
  }
}

namespace {

// Largest dynamic LDS a launch asks for: 16 wave buffers (codes + 4 staged x
// rows) + 16 x 4 reduction rows.  The kernel also holds a few bytes of static
// LDS, so this stays below the 160 KB of a CU.
constexpr int kMaxLdsBytes = kMaxWaves * (kItemBytes + 4 * kXRowBytes + kXsumBytes) + kMaxWaves * 4 * kWave * 4;

}  // namespace

bool qmv_mfma_supports(int K, int N, int M)
{
  return K % kKS == 0 && N >= 1 && M >= 1 && M <= 16;
}

hipError_t launch_qmv_mfma(hipStream_t st, const QmvArgs& a)
{
  QmvParams p;
  p.w = a.w; p.scales = a.scales; p.biases = a.biases; p.x = a.x; p.y = a.y;
  p.residual = a.residual;
  p.K = a.K; p.N = a.N; p.M = a.M;
  p.gate_act = a.gate_act;
  p.nseg = 1;
  p.slices = a.K / kKS;

  // Wavefronts per workgroup: every wavefront gets the same number of items
  // where the slice count allows it.
  const int per_wave = (p.slices + kMaxWaves - 1) / kMaxWaves;
  int nw = (p.slices + per_wave - 1) / per_wave;
  int mr = (a.M + 3) / 4;
  if (mr == 3) { mr = 4; }
  // The final reduction is done by mr*64 threads.
  if (nw < mr) { nw = mr; }

  const bool xlds = a.M <= 4;
  p.wave_lds_bytes = kItemBytes + (xlds ? a.M * kXRowBytes + kXsumBytes : 0);
  const size_t lds_bytes = (size_t)nw * p.wave_lds_bytes + (size_t)nw * mr * kWave * sizeof(float);
  const dim3 grid((unsigned)((a.N + kTileN - 1) / kTileN)), block((unsigned)(nw * kWave));

  // the attribute is set once per kernel, whichever thread comes first (atomic flags: two threads may both set
  // it, which is harmless; neither launches before its own call has returned)
  static std::atomic<bool> attr_done[8];
  auto launch = [&](auto kern, int slot) -> hipError_t {
    if (!attr_done[slot].load(std::memory_order_acquire)) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsBytes);
      if (e != hipSuccess) { return e; }
      attr_done[slot].store(true, std::memory_order_release);
    }
    return launch_kernel(kern, grid, block, lds_bytes, st, p);
  };
  if (a.y_f32) {
    if (mr == 1) { return launch(qmv_mfma_kernel<1, true, true>, 0); }
    if (mr == 2) { return launch(qmv_mfma_kernel<2, false, true>, 1); }
    return launch(qmv_mfma_kernel<4, false, true>, 2);
  }
  if (mr == 1) { return launch(qmv_mfma_kernel<1, true, false>, 3); }
  if (mr == 2) { return launch(qmv_mfma_kernel<2, false, false>, 4); }
  return launch(qmv_mfma_kernel<4, false, false>, 5);
}

hipError_t launch_qmv_mfma_group(hipStream_t st, const QmvArgs& a, const QmvGroup& g)
{
  QmvParams p;
  p.w = nullptr; p.scales = nullptr; p.biases = nullptr; p.x = a.x; p.y = nullptr;
  p.residual = nullptr;
  p.K = a.K; p.N = 0; p.M = a.M;
  p.gate_act = 0;
  p.slices = a.K / kKS;
  p.nseg = g.count;
  int tiles = 0;
  for (int i = 0; i < 4; ++i) {
    if (i < g.count) {
      p.seg[i] = g.seg[i];
      tiles += (g.seg[i].N + kTileN - 1) / kTileN;
    } else {
      p.seg[i] = g.seg[g.count - 1];
    }
    p.seg_tile_end[i] = tiles;
  }
  if (g.count == 1) {          // the kernel's single-pack path reads p.w etc.
    p.w = g.seg[0].w; p.scales = g.seg[0].scales; p.biases = g.seg[0].biases; p.y = g.seg[0].y; p.N = g.seg[0].N;
  }
  const int per_wave = (p.slices + kMaxWaves - 1) / kMaxWaves;
  int nw = (p.slices + per_wave - 1) / per_wave;
  int mr = (a.M + 3) / 4;
  if (mr == 3) { mr = 4; }
  if (nw < mr) { nw = mr; }
  const bool xlds = a.M <= 4;
  p.wave_lds_bytes = kItemBytes + (xlds ? a.M * kXRowBytes + kXsumBytes : 0);
  const size_t lds_bytes = (size_t)nw * p.wave_lds_bytes + (size_t)nw * mr * kWave * sizeof(float);
  const dim3 grid((unsigned)tiles, 1u), block((unsigned)(nw * kWave));
  static std::atomic<bool> attr_done[3];
  auto launch = [&](auto kern, int slot) -> hipError_t {
    if (!attr_done[slot].load(std::memory_order_acquire)) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsBytes);
      if (e != hipSuccess) { return e; }
      attr_done[slot].store(true, std::memory_order_release);
    }
    return launch_kernel(kern, grid, block, lds_bytes, st, p);
  };
  if (mr == 1) { return launch(qmv_mfma_kernel<1, true, false>, 0); }
  if (mr == 2) { return launch(qmv_mfma_kernel<2, false, false>, 1); }
  return launch(qmv_mfma_kernel<4, false, false>, 2);
}

}  // namespace vpq

// QMV at M = 1 as a pure streaming kernel: every load of a wavefront is in flight before its
// first multiply.
//
// Work decomposition.  A wavefront owns RB consecutive weight rows and a K range of SPW slices of
// 2048 values (a lane takes 16 bytes = 32 values of a row per slice, so one load instruction
// covers 1 KB of one row).  WK wavefronts of a workgroup share a row set and split K between
// them; their row sums meet in LDS at the end.  A launch has one wavefront per (row set, K part):
// all of them are resident at once, so the whole pack is requested in the first microsecond and
// the arithmetic runs in the shadow of the arriving data.
//
// Order of requests (vector-memory results return in order, so what a multiply needs must have
// been requested before the codes it goes with):
//   1. scales and biases of the wavefront's rows and K range: 16-byte direct-to-LDS loads
//      (1 KB per instruction, scales and biases in the same instruction where they fit);
//   2. the lane's 32 values of x per slice (kept in registers for all rows, as packed pairs,
//      with their fp32 sum);
//   3. the codes, RB * SPW loads of 16 bytes per lane.
// The loads are inline assembly so that the only waits are the counted ones written here: the
// compiler would otherwise wait for every outstanding load before the first LDS read.
//
// Arithmetic (the factored form of gpu-kernels/metal/quant/affine_qmv.metal:151-174, weight
// never rounded): codes become packed bf16 pairs (128 + q_i, 128 + q_{i+4}) with one
// v_and_or_b32 per pair and are contracted against the matching pair of x with
// v_dot2c_f32_bf16 (products exact, fp32 sums); with sx the sum of the lane's 32 values of x,
//     y += s * dot + (b - 128 * s) * sx
// per row and slice (a lane's 32 values lie in one quantization group), one wave reduction per
// row at the end.
#include <type_traits>

#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));

constexpr int kSlice = 2048;          // values of K per slice (64 lanes x 32)
constexpr int kMaxWavesPerWg = 8;

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c)
{
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
  if constexpr (I < N) {
    f(std::integral_constant<int, I>());
    static_for<I + 1, N>(f);
  }
}

// 16 bytes per lane from a wave-uniform base plus a byte offset per lane.  The compiler does not
// know that the result arrives later: nothing may read it before wait_vm + touch.
__device__ __forceinline__ u32x4v gload16(const void* base, uint32_t voff)
{
  u32x4v r;
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r) : "v"(voff), "s"(base) : "memory");
  return r;
}

// 16 bytes per lane, global -> LDS at lds_dst + 16 * lane.  M0 is used by nothing else here.
__device__ __forceinline__ void dma16(uint32_t lds_dst, const void* src)
{
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_dst);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m0v), "v"(src) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vm()
{
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// The same, placed after the computation of `dep` (keeps the arithmetic of a slice between the
// waits of that slice and the next instead of after the last wait).
template <int N>
__device__ __forceinline__ void wait_vm_after(float& dep)
{
  asm volatile("s_waitcnt vmcnt(%1)" : "+v"(dep) : "n"(N) : "memory");
}

__device__ __forceinline__ void touch(u32x4v& v) { asm volatile("" : "+v"(v)); }

// Total over the 64 lanes, valid in lane 63.
__device__ __forceinline__ float wave_total_l63(float v)
{
  int t;
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false);    // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false);    // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false);   // row_half_mirror
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false);   // row_mirror
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false);   // row_bcast15 into rows 1, 3
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false);   // row_bcast31 into rows 2, 3
  v += __builtin_bit_cast(float, t);
  return v;
}

struct FlowSeg {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  void* y;
  int N;
  int first_block;
};

struct FlowParams {
  int count;
  FlowSeg seg[4];
  const uint16_t* x;
  const uint16_t* residual;
  int K;
  int wk;          // wavefronts that share a row set (K parts)
  int wr;          // row sets per workgroup
  int gate_act;
};

}  // namespace

template <int SPW, int RB, bool F32OUT>
__global__ __launch_bounds__(64 * kMaxWavesPerWg) void qmv_flow_kernel(const FlowParams p)
{
  constexpr int NL = RB * SPW;                 // code loads of a wavefront
  constexpr int PPR = SPW * 4;                 // 16-byte pieces of scales (or biases) per row and K part
  constexpr int P = RB * PPR;
  constexpr int NDMA = (2 * P + 63) / 64;
  __shared__ __attribute__((aligned(16))) uint8_t sb_lds[kMaxWavesPerWg * NDMA * 1024];
  __shared__ float red[kMaxWavesPerWg * RB];

  FlowSeg sg = p.seg[0];
#pragma unroll
  for (int i = 1; i < 4; ++i) {
    if (i < p.count && (int)blockIdx.x >= p.seg[i].first_block) { sg = p.seg[i]; }
  }
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rs = wave / p.wk, part = wave - rs * p.wk;
  const int K = p.K, N = sg.N;
  const int Kg = K >> 6;
  const int row_begin = (((int)blockIdx.x - sg.first_block) * p.wr + rs) * RB;
  const bool active = row_begin < N;           // wave-uniform
  const int slice0 = part * SPW;

  uint32_t magic = 0x43004300u;                // bf16 128.0 in both halves
  uint32_t mask = 0x000f000fu;
  asm volatile("" : "+v"(magic));              // no instruction: hides the constants from folding, so
  asm volatile("" : "+s"(mask));               // that each pair costs one v_and_or_b32
  const uint32_t ones = 0x3f803f80u;           // bf16 1.0 twice

  float tot[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) { tot[r] = 0.0f; }

  if (active) {
    bool kvalid[SPW];
    uint32_t koff[SPW];                        // byte offset of the lane's 16 bytes in a row of codes
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      const int k0 = (slice0 + s) * kSlice + lane * 32;
      kvalid[s] = k0 < K;
      koff[s] = kvalid[s] ? (uint32_t)(k0 >> 1) : 0u;
    }

    // 1. scales and biases -> this wavefront's LDS window: piece i < P is 16 bytes of scales of row
    // i / PPR, P <= i < 2P the same of the biases; pieces past K re-read the first piece of the part
    // (finite values; their lanes multiply them by zero).
    uint8_t* sbl = sb_lds + wave * (NDMA * 1024);
    const uint32_t sbl_a = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)sbl;
    const int g0 = slice0 * 32;                // first group of the part (< Kg for an active part)
#pragma unroll
    for (int j = 0; j < NDMA; ++j) {
      int i = lane + 64 * j;
      const bool isb = i >= P;
      if (isb) { i -= P; }
      if (i >= P) { i = 0; }
      const int row = i / PPR, pc = i % PPR;
      const int n = (row_begin + row < N) ? (row_begin + row) : (N - 1);
      const int g = (g0 + pc * 8 < Kg) ? (g0 + pc * 8) : g0;
      const uint16_t* src = (isb ? sg.biases : sg.scales) + (size_t)n * Kg + g;
      dma16(sbl_a + j * 1024, src);
    }
    // 2. x
    u32x4v xr[SPW][4];
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      const uint32_t xo = kvalid[s] ? (uint32_t)((slice0 + s) * (kSlice * 2) + lane * 64) : 0u;
#pragma unroll
      for (int t = 0; t < 4; ++t) { xr[s][t] = gload16(p.x, xo + t * 16); }
    }
    // 3. codes
    u32x4v c[RB][SPW];
    const uint8_t* wbase = reinterpret_cast<const uint8_t*>(sg.w) + (size_t)row_begin * (size_t)(K >> 1);
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int rr = (row_begin + r < N) ? r : (N - 1 - row_begin);
      const uint8_t* wr = wbase + (size_t)rr * (size_t)(K >> 1);
#pragma unroll
      for (int s = 0; s < SPW; ++s) { c[r][s] = gload16(wr, koff[s]); }
    }

    wait_vm<NL>();                             // scales, biases and x have landed
    uint32_t xp[SPW][16];
    float sx[SPW];
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      float sum = 0.0f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        touch(xr[s][t]);
        u32x4v d = xr[s][t];
        if (!kvalid[s]) { d = u32x4v{0u, 0u, 0u, 0u}; }
        xp[s][4 * t + 0] = __builtin_amdgcn_perm(d.z, d.x, 0x05040100u);   // x0,x4
        xp[s][4 * t + 1] = __builtin_amdgcn_perm(d.z, d.x, 0x07060302u);   // x1,x5
        xp[s][4 * t + 2] = __builtin_amdgcn_perm(d.w, d.y, 0x05040100u);   // x2,x6
        xp[s][4 * t + 3] = __builtin_amdgcn_perm(d.w, d.y, 0x07060302u);   // x3,x7
        sum = dot2(d.x, ones, sum);
        sum = dot2(d.y, ones, sum);
        sum = dot2(d.z, ones, sum);
        sum = dot2(d.w, ones, sum);
      }
      sx[s] = sum;
    }
    uint32_t sraw[RB][SPW], braw[RB][SPW];
#pragma unroll
    for (int r = 0; r < RB; ++r) {
#pragma unroll
      for (int s = 0; s < SPW; ++s) {
        const int o = r * (PPR * 16) + s * 64 + (lane >> 1) * 2;
        sraw[r][s] = *reinterpret_cast<const uint16_t*>(sbl + o);
        braw[r][s] = *reinterpret_cast<const uint16_t*>(sbl + P * 16 + o);
      }
    }

    float acc[RB];
    float chain = sx[0];
    static_for<0, RB>([&](auto rc) {
      constexpr int r = decltype(rc)::value;
      acc[r] = 0.0f;
      static_for<0, SPW>([&](auto sc_) {
        constexpr int s = decltype(sc_)::value;
        wait_vm_after<NL - 1 - (r * SPW + s)>(chain);
        touch(c[r][s]);
        const uint32_t cw[4] = {c[r][s].x, c[r][s].y, c[r][s].z, c[r][s].w};
        float d0 = 0.0f, d1 = 0.0f;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          d0 = dot2(xp[s][4 * t + 0], ((cw[t] >> 0) & mask) | magic, d0);
          d1 = dot2(xp[s][4 * t + 1], ((cw[t] >> 4) & mask) | magic, d1);
          d0 = dot2(xp[s][4 * t + 2], ((cw[t] >> 8) & mask) | magic, d0);
          d1 = dot2(xp[s][4 * t + 3], ((cw[t] >> 12) & mask) | magic, d1);
        }
        const float sc = bf16_bits_to_f32(sraw[r][s]);
        const float bi = bf16_bits_to_f32(braw[r][s]);
        acc[r] = fmaf(sc, d0 + d1, acc[r]);
        acc[r] = fmaf(fmaf(-128.0f, sc, bi), sx[s], acc[r]);
        chain = acc[r];
      });
    });
#pragma unroll
    for (int r = 0; r < RB; ++r) { tot[r] = wave_total_l63(acc[r]); }
  }

  // Row sums of the K parts meet in LDS; the wavefront of part 0 adds them in part order.
  if (p.wk > 1) {
    if (lane == 63) {
#pragma unroll
      for (int r = 0; r < RB; ++r) { red[wave * RB + r] = tot[r]; }
    }
    __syncthreads();
    if (part != 0) { return; }
    if (lane == 63) {
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        float v = tot[r];
        for (int q = 1; q < p.wk; ++q) { v += red[(wave + q) * RB + r]; }
        tot[r] = v;
      }
    }
  }
  if (!active || lane != 63) { return; }

  if (p.gate_act) {
    // rows 2g and 2g+1 are the gate and the up row of feature g; RB is even, so a pair is one wavefront's
#pragma unroll
    for (int r = 0; r < RB; r += 2) {
      const int n = row_begin + r;
      if (n + 1 < N) {
        const float v = gated_f32(p.gate_act, tot[r], tot[r + 1]);
        const size_t o = (size_t)(n >> 1);
        if (F32OUT) {
          reinterpret_cast<float*>(sg.y)[o] = v;
        } else {
          reinterpret_cast<uint16_t*>(sg.y)[o] = (uint16_t)f32_to_bf16_bits(v);
        }
      }
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int n = row_begin + r;
    if (n < N) {
      if (F32OUT) {
        reinterpret_cast<float*>(sg.y)[n] = tot[r];
      } else {
        uint32_t v = f32_to_bf16_bits(tot[r]);
        if (p.residual != nullptr) { v = f32_to_bf16_bits(bf16_bits_to_f32(v) + bf16_bits_to_f32(p.residual[n])); }
        reinterpret_cast<uint16_t*>(sg.y)[n] = (uint16_t)v;
      }
    }
  }
}

namespace {

struct FlowPlan {
  int spw, wk, wr, rb;
};

// Slices per wavefront and K parts: the fewest idle slice slots, then the fewest parts.
FlowPlan flow_plan(int K, double pack_bytes)
{
  const int slices = (K + kSlice - 1) / kSlice;
  FlowPlan best{0, 0, 0, 0};
  int best_waste = 1 << 30;
  for (int spw = 4; spw >= 1; --spw) {
    const int wk = (slices + spw - 1) / spw;
    if (wk > kMaxWavesPerWg) { continue; }
    const int waste = wk * spw - slices;
    if (waste < best_waste) {
      best_waste = waste;
      best.spw = spw;
      best.wk = wk;
    }
  }
  if (best.spw == 0) { return best; }
  int wr = 4 / best.wk;
  if (wr < 1) { wr = 1; }
  if (best.wk == 3) { wr = 2; }
  best.wr = wr;
  // Rows per wavefront: 8 to 12 code loads in flight per wavefront on layer-sized packs; fewer on small
  // ones, where more wavefronts spread the pack over the CUs.
  best.rb = (best.spw <= 2 && pack_bytes >= 12e6) ? 4 : 2;
  return best;
}

hipError_t launch_flow(hipStream_t st, FlowParams& p, const QmvArgs& a, double pack_bytes, const FlowPlan* forced)
{
  const FlowPlan pl = forced != nullptr ? *forced : flow_plan(a.K, pack_bytes);
  if (pl.spw == 0 || pl.wk * pl.wr > kMaxWavesPerWg || pl.wk * pl.spw * kSlice < a.K) { return hipErrorInvalidValue; }
  p.x = a.x;
  p.K = a.K;
  p.wk = pl.wk;
  p.wr = pl.wr;
  const int rows_per_block = pl.wr * pl.rb;
  int blocks = 0;
  for (int i = 0; i < p.count; ++i) {
    p.seg[i].first_block = blocks;
    blocks += (p.seg[i].N + rows_per_block - 1) / rows_per_block;
  }
  const dim3 grid((unsigned)blocks), block((unsigned)(64 * pl.wk * pl.wr));
#define VPQ_FLOW(S, R)                                                                              \
  if (pl.spw == S && pl.rb == R) {                                                                  \
    return a.y_f32 ? launch_kernel(qmv_flow_kernel<S, R, true>, grid, block, 0, st, p)              \
                   : launch_kernel(qmv_flow_kernel<S, R, false>, grid, block, 0, st, p);            \
  }
  VPQ_FLOW(1, 2) VPQ_FLOW(2, 2) VPQ_FLOW(3, 2) VPQ_FLOW(4, 2) VPQ_FLOW(6, 2)
  VPQ_FLOW(1, 4) VPQ_FLOW(2, 4) VPQ_FLOW(3, 4) VPQ_FLOW(4, 4)
#undef VPQ_FLOW
  return hipErrorInvalidValue;
}

}  // namespace

bool qmv_flow_supports(int K, int N, int M)
{
  return M == 1 && N >= 1 && K >= kSlice && K % 512 == 0 && (K + kSlice - 1) / kSlice <= 4 * kMaxWavesPerWg;
}

hipError_t launch_qmv_flow(hipStream_t st, const QmvArgs& a)
{
  FlowParams p{};
  p.count = 1;
  p.seg[0] = FlowSeg{a.w, a.scales, a.biases, a.y, a.N, 0};
  p.residual = a.residual;
  p.gate_act = a.gate_act;
  return launch_flow(st, p, a, (double)a.N * (double)a.K * 9.0 / 16.0, nullptr);
}

// Measurement only: the single-pack launch with the plan given (slices per wavefront, K parts, row sets per
// workgroup, rows per wavefront).
hipError_t launch_qmv_flow_planned(hipStream_t st, const QmvArgs& a, int spw, int wk, int wr, int rb)
{
  FlowParams p{};
  p.count = 1;
  p.seg[0] = FlowSeg{a.w, a.scales, a.biases, a.y, a.N, 0};
  p.residual = a.residual;
  p.gate_act = a.gate_act;
  const FlowPlan pl{spw, wk, wr, rb};
  return launch_flow(st, p, a, 0.0, &pl);
}

hipError_t launch_qmv_flow_group(hipStream_t st, const QmvArgs& a, const QmvGroup& g)
{
  FlowParams p{};
  p.count = g.count;
  double bytes = 0.0;
  for (int i = 0; i < g.count; ++i) {
    p.seg[i] = FlowSeg{g.seg[i].w, g.seg[i].scales, g.seg[i].biases, g.seg[i].y, g.seg[i].N, 0};
    bytes += (double)g.seg[i].N * (double)a.K * 9.0 / 16.0;
  }
  p.residual = nullptr;
  p.gate_act = 0;
  return launch_flow(st, p, a, bytes, nullptr);
}

}  // namespace vpq

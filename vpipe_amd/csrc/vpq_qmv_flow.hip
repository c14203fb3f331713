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
//   1. x of the workgroup's K range, by direct-to-LDS loads shared between its wavefronts (a
//      wavefront then keeps its lanes' 32 values per slice in registers for all rows, as packed
//      pairs, with their fp32 sum);
//   2. the codes, RB * SPW loads of 16 bytes per lane, as soon as their addresses are known:
//      the time to the first code request is paid by every wavefront of the launch;
//   3. scales and biases of the wavefront's rows and K range: 16-byte direct-to-LDS loads
//      (1 KB per instruction, scales and biases in the same instruction where they fit).  They
//      are applied to the per-(row, slice) dot products at the end.
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
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));

constexpr int kSlice = 2048;          // values of K per slice (64 lanes x 32)
constexpr int kMaxWavesPerWg = 8;
constexpr int kMaxLdsBytes = 96 * 1024;   // x of the K range + the scale/bias windows; K <= 32768 fits

typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));

// a.lo * b.lo + a.hi * b.hi + c on pairs of bf16 (F16 = false) or IEEE binary16 (true), fp32 accumulation
template <bool F16 = false>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c)
{
  if constexpr (F16) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(halfx2, a), __builtin_bit_cast(halfx2, b), c, false);
  } else {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
  }
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

// 16 bytes per lane, global -> LDS at lds_dst + 16 * lane.  The LDS base travels in M0, bound as an operand: the
// compiler writes it and knows its value (the s_nop is the wait state between that write and the load).
__device__ __forceinline__ void dma16(uint32_t lds_dst, const void* src)
{
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_dst);
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "{m0}"(m0v) : "memory");
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
};

// Kernel arguments.  The single-pack form is 64 bytes, one cache line of the argument buffer: every wavefront of
// the launch waits for its arguments before its first request, and each further line costs a quarter of a
// microsecond on layer-sized packs.
struct FlowHead {
  const uint16_t* x;
  const uint16_t* residual;
  int K;
  // bits 0-23: 3 bits per wavefront of a workgroup, its row set (wavefront = row set * wk + K part);
  // 24-25: wk - 1 (wavefronts that share a row set); 26-28: wr - 1 (row sets per workgroup); 29-30: gate_act
  uint32_t shape;
};
// C packs that share x; pack i owns the workgroups from first_block[i] on (first_block[0] = 0).
template <int C>
struct FlowParams {
  FlowHead h;
  const uint32_t* w[C];
  const uint16_t* scales[C];
  const uint16_t* biases[C];
  void* y[C];
  int N[C];
  int first_block[C];
};
static_assert(sizeof(FlowParams<1>) == 64, "single-pack arguments: one line");
static_assert(sizeof(FlowParams<2>) <= 128, "two packs: two lines");

// Forces a kernel argument into scalar registers here, so that all argument loads go out together at the
// top of the kernel instead of one round trip per first use.
template <typename T>
__device__ __forceinline__ void pin_scalar(const T& v) { asm volatile("" : : "s"(v)); }

}  // namespace


// x reaches a wavefront through LDS: the workgroup's K range of x is copied there once by direct-to-LDS loads
// shared between its wavefronts (one barrier); the codes are requested right after the wavefront's share of x,
// scales and biases last, and they are applied to the per-(row, slice) dot products at the end.
//
// F16: the elements (x, scales, biases, y, residual) are IEEE binary16 instead of bf16 (the reference's
// VPIPE_ELT = half build).  The codes then become binary16 pairs 16 + q (the code shifted to mantissa bits 6..9,
// exact; 1024 + q with the code left in bits 0..3 would cost eight times bf16's cancellation noise).
// PRELOADED: the arguments are already in scalar registers (nothing to batch; the residual is left to be loaded
// when the store needs it).
template <int SPW, int RB, bool F32OUT, int C, bool F16 = false, bool PRELOADED = false>
__device__ __forceinline__ void qmv_flow_body(const FlowParams<C>& p)
{
  constexpr int NL = RB * SPW;                 // code loads of a wavefront
  constexpr int PPR = SPW * 4;                 // 16-byte pieces of scales (or biases) per row and K part
  constexpr int P = RB * PPR;
  constexpr int NDMA = (2 * P + 63) / 64;
  // LDS: x of the workgroup's K range (wk * SPW slices of 4 KB), one window of scales/biases per wavefront, the
  // row sums of the K parts.
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  // ---- arguments: everything in one batch of scalar loads, the segment chosen without branches
  const uint16_t* xg = p.h.x;
  const uint16_t* residual = p.h.residual;
  const int K = p.h.K;
  const uint32_t shape = p.h.shape;
  if constexpr (!PRELOADED) { pin_scalar(xg); pin_scalar(residual); pin_scalar(K); pin_scalar(shape); }
  const int blk = (int)blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t* w_[C]; const uint16_t* s_[C]; const uint16_t* b_[C]; void* y_[C]; int n_[C], fb_[C];
#pragma unroll
  for (int i = 0; i < C; ++i) {
    w_[i] = p.w[i]; s_[i] = p.scales[i]; b_[i] = p.biases[i]; y_[i] = p.y[i]; n_[i] = p.N[i]; fb_[i] = p.first_block[i];
    if constexpr (!PRELOADED) {
      pin_scalar(w_[i]); pin_scalar(s_[i]); pin_scalar(b_[i]); pin_scalar(y_[i]); pin_scalar(n_[i]); pin_scalar(fb_[i]);
    }
  }
  const uint32_t* wq = w_[0]; const uint16_t* sq = s_[0]; const uint16_t* bq = b_[0]; void* yq = y_[0];
  int N = n_[0], first_block = 0;
  if constexpr (PRELOADED && C > 1) {
    // The first pack's arguments are in registers already, the others' are still on their way from the argument
    // buffer: a branch, so that the workgroups of the first pack (which come first) do not wait for them.
    if (blk >= fb_[1]) {
      wq = w_[1]; sq = s_[1]; bq = b_[1]; yq = y_[1]; N = n_[1]; first_block = fb_[1];
#pragma unroll
      for (int i = 2; i < C; ++i) {
        const bool take = blk >= fb_[i];
        wq = take ? w_[i] : wq; sq = take ? s_[i] : sq; bq = take ? b_[i] : bq; yq = take ? y_[i] : yq;
        N = take ? n_[i] : N; first_block = take ? fb_[i] : first_block;
      }
      asm volatile("" : "+s"(wq), "+s"(sq), "+s"(bq), "+s"(N), "+s"(first_block));   // keeps this a branch
    }
  } else {
#pragma unroll
    for (int i = 1; i < C; ++i) {
      const bool take = blk >= fb_[i];
      wq = take ? w_[i] : wq; sq = take ? s_[i] : sq; bq = take ? b_[i] : bq; yq = take ? y_[i] : yq;
      N = take ? n_[i] : N; first_block = take ? fb_[i] : first_block;
    }
  }
  const int wk = (int)((shape >> 24) & 3u) + 1, wr = (int)((shape >> 26) & 7u) + 1, gate_act = (int)((shape >> 29) & 3u);

  const int rs = (int)((shape >> (3 * wave)) & 7u), part = wave - rs * wk;
  const int W = wk * wr;
  const int Kg = K >> 6;
  const int row_begin = ((blk - first_block) * wr + rs) * RB;
  const bool active = row_begin < N;           // wave-uniform
  const int slice0 = part * SPW;
  const int x_bytes = wk * SPW * (kSlice * 2);
  uint8_t* sbl = lds + x_bytes + wave * (NDMA * 1024);
  float* red = reinterpret_cast<float*>(lds + x_bytes + W * (NDMA * 1024));
  const uint32_t lds_a = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)lds;

  uint32_t magic = F16 ? 0x4c004c00u : 0x43004300u;   // 16.0 (binary16) or 128.0 (bf16) in both halves
  uint32_t mask = F16 ? 0x03c003c0u : 0x000f000fu;
  asm volatile("" : "+v"(magic));              // no instruction: hides the constants from folding, so
  asm volatile("" : "+s"(mask));               // that each pair costs one v_and_or_b32
  const uint32_t ones = F16 ? 0x3c003c00u : 0x3f803f80u;   // 1.0 twice
  constexpr float kOffset = F16 ? -16.0f : -128.0f;

  bool kvalid[SPW];
#pragma unroll
  for (int s = 0; s < SPW; ++s) { kvalid[s] = (slice0 + s) * kSlice + lane * 32 < K; }

  // Scales and biases -> this wavefront's LDS window: piece i < P is 16 bytes of scales of row i / PPR,
  // P <= i < 2P the same of the biases; pieces past K re-read the first piece of the part (finite values; their
  // lanes multiply them by zero).
  auto request_scales_biases = [&]() {
    const int g0 = slice0 * 32;                // first group of the part (< Kg: every part holds a slice)
#pragma unroll
    for (int j = 0; j < NDMA; ++j) {
      int i = lane + 64 * j;
      const bool isb = i >= P;
      if (isb) { i -= P; }
      if (i >= P) { i = 0; }
      const int row = i / PPR, pc = i % PPR;
      const int n = (row_begin + row < N) ? (row_begin + row) : (N - 1);
      const int g = (g0 + pc * 8 < Kg) ? (g0 + pc * 8) : g0;
      const uint16_t* src = (isb ? bq : sq) + (size_t)n * Kg + g;
      dma16(lds_a + (uint32_t)(x_bytes + wave * (NDMA * 1024) + j * 1024), src);
    }
  };

  {
    // x of the workgroup's K range -> LDS, the wavefronts taking the 1 KB pieces round-robin.  Piece j is
    // quarter t = j % 4 of slice j / 4: lane i brings the 16 bytes at values 32 i + 8 t of the slice, so that a
    // lane's later reads (its 32 values, quarter by quarter) are one 16-byte word per lane at consecutive
    // addresses.  Pieces past K re-read the start of x; their lanes use zeros instead.
    for (int j = wave; j < 4 * wk * SPW; j += W) {
      const int k = (j >> 2) * kSlice + lane * 32 + (j & 3) * 8;
      dma16(lds_a + (uint32_t)(j * 1024), xg + (k < K ? k : 0));
    }
  }

  // A wavefront without rows (past N in the last workgroup) only brings its share of x and meets the barriers.  It
  // leaves here, on a path of its own, so that no path on which code loads are in flight joins one on which they
  // were never issued: the build checks the registers of those loads along every static path.
  if (!active) {
    wait_vm<0>();
    __syncthreads();
    if (wk > 1) { __syncthreads(); }
    return;
  }

  float tot[RB];

  // codes
  constexpr int AFTER = NDMA;                  // requests that follow the codes
  u32x4v c[RB][SPW];
  {
    const uint8_t* wbase = reinterpret_cast<const uint8_t*>(wq) + (size_t)row_begin * (size_t)(K >> 1);
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int rr = (row_begin + r < N) ? r : (N - 1 - row_begin);
      const uint8_t* wrow = wbase + (size_t)rr * (size_t)(K >> 1);
#pragma unroll
      for (int s = 0; s < SPW; ++s) {
        const uint32_t koff = kvalid[s] ? (uint32_t)((slice0 + s) * (kSlice / 2) + lane * 16) : 0u;
        c[r][s] = gload16(wrow, koff);
      }
    }
    request_scales_biases();
    wait_vm<NL + AFTER>();                       // this wavefront's share of x has landed
  }
  __syncthreads();                               // ... and everybody else's share

  {
    uint32_t xp[SPW][16];                        // pairs (x_i, x_{i+4}) of each run of eight
    float sx[SPW];
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      float sum = 0.0f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        uint4 d = *reinterpret_cast<const uint4*>(lds + (((slice0 + s) * 4 + t) * 64 + lane) * 16);
        if (!kvalid[s]) { d = make_uint4(0u, 0u, 0u, 0u); }
        xp[s][4 * t + 0] = __builtin_amdgcn_perm(d.z, d.x, 0x05040100u);   // x0,x4
        xp[s][4 * t + 1] = __builtin_amdgcn_perm(d.z, d.x, 0x07060302u);   // x1,x5
        xp[s][4 * t + 2] = __builtin_amdgcn_perm(d.w, d.y, 0x05040100u);   // x2,x6
        xp[s][4 * t + 3] = __builtin_amdgcn_perm(d.w, d.y, 0x07060302u);   // x3,x7
        sum = dot2<F16>(d.x, ones, sum);
        sum = dot2<F16>(d.y, ones, sum);
        sum = dot2<F16>(d.z, ones, sum);
        sum = dot2<F16>(d.w, ones, sum);
      }
      sx[s] = sum;
    }
    // The dot products of every (row, slice) as the codes arrive; scales and biases when everything has landed.
    float dots[RB][SPW];
    float chain = sx[0];
    static_for<0, RB>([&](auto rc) {
      constexpr int r = decltype(rc)::value;
      static_for<0, SPW>([&](auto sc_) {
        constexpr int s = decltype(sc_)::value;
        wait_vm_after<AFTER + NL - 1 - (r * SPW + s)>(chain);
        touch(c[r][s]);
        const uint32_t cw[4] = {c[r][s].x, c[r][s].y, c[r][s].z, c[r][s].w};
        float d0 = 0.0f, d1 = 0.0f;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          if constexpr (F16) {
            // the code goes to mantissa bits 6..9 of 16.0: 16 + q, exact (a step of 1/64 there)
            d0 = dot2<true>(xp[s][4 * t + 0], ((cw[t] << 6) & mask) | magic, d0);
            d1 = dot2<true>(xp[s][4 * t + 1], ((cw[t] << 2) & mask) | magic, d1);
            d0 = dot2<true>(xp[s][4 * t + 2], ((cw[t] >> 2) & mask) | magic, d0);
            d1 = dot2<true>(xp[s][4 * t + 3], ((cw[t] >> 6) & mask) | magic, d1);
          } else {
            d0 = dot2(xp[s][4 * t + 0], ((cw[t] >> 0) & mask) | magic, d0);
            d1 = dot2(xp[s][4 * t + 1], ((cw[t] >> 4) & mask) | magic, d1);
            d0 = dot2(xp[s][4 * t + 2], ((cw[t] >> 8) & mask) | magic, d0);
            d1 = dot2(xp[s][4 * t + 3], ((cw[t] >> 12) & mask) | magic, d1);
          }
        }
        dots[r][s] = d0 + d1;                    // sum x * (128 + q), binary16: sum x * (16 + q)
        chain = dots[r][s];
      });
    });
    wait_vm_after<0>(chain);
    float acc[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      acc[r] = 0.0f;
#pragma unroll
      for (int s = 0; s < SPW; ++s) {
        const int o = r * (PPR * 16) + s * 64 + (lane >> 1) * 2;
        const float sc = elt_bits_to_f32<F16>(*reinterpret_cast<const uint16_t*>(sbl + o));
        const float bi = elt_bits_to_f32<F16>(*reinterpret_cast<const uint16_t*>(sbl + P * 16 + o));
        acc[r] = fmaf(sc, dots[r][s], acc[r]);
        acc[r] = fmaf(fmaf(kOffset, sc, bi), sx[s], acc[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < RB; ++r) { tot[r] = wave_total_l63(acc[r]); }
  }

  // Row sums of the K parts meet in LDS; the wavefront of part 0 adds them in part order.
  if (wk > 1) {
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
        for (int q = 1; q < wk; ++q) { v += red[(wave + q) * RB + r]; }
        tot[r] = v;
      }
    }
  }
  if (lane != 63) { return; }

  if (gate_act == kGateSwiglu || gate_act == kGateGeglu) {
    // rows 2g and 2g+1 are the gate and the up row of feature g; RB is even, so a pair is one wavefront's
#pragma unroll
    for (int r = 0; r < RB; r += 2) {
      const int n = row_begin + r;
      if (n + 1 < N) {
        const float v = gated_f32(gate_act, tot[r], tot[r + 1]);
        const size_t o = (size_t)(n >> 1);
        if (F32OUT) {
          reinterpret_cast<float*>(yq)[o] = v;
        } else {
          reinterpret_cast<uint16_t*>(yq)[o] = (uint16_t)f32_to_elt_bits<F16>(v);
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
        reinterpret_cast<float*>(yq)[n] = tot[r];
      } else {
        uint32_t v = f32_to_elt_bits<F16>(tot[r]);
        if (gate_act == kStoreGeluMul) {
          v = f32_to_elt_bits<F16>(gelu_mul_f32(elt_bits_to_f32<F16>(v), elt_bits_to_f32<F16>(residual[n])));
        } else if (residual != nullptr) {
          v = f32_to_elt_bits<F16>(elt_bits_to_f32<F16>(v) + elt_bits_to_f32<F16>(residual[n]));
        }
        reinterpret_cast<uint16_t*>(yq)[n] = (uint16_t)v;
      }
    }
  }
}

// The single-pack form with its sixteen argument words as separate kernel arguments: this file is compiled with
// kernel-argument preloading, which delivers the first sixteen words in scalar registers when a wavefront starts,
// so a wavefront's first requests do not wait for a load of the argument buffer (an aggregate argument is not
// preloaded).
template <int SPW, int RB, bool F32OUT, bool F16 = false>
__global__ __launch_bounds__(64 * kMaxWavesPerWg) void qmv_flow_kernel_1(
    const uint16_t* x, const uint32_t* w, const uint16_t* scales, const uint16_t* biases, void* y, int K, uint32_t shape,
    int N, const uint16_t* residual)
{
  // Fourteen words arrive preloaded: everything a wavefront needs for its requests.  The residual (read at the
  // store) follows them and is loaded from the argument buffer in the usual way.
  FlowParams<1> p;
  p.h.x = x; p.h.residual = residual; p.h.K = K; p.h.shape = shape;
  p.w[0] = w; p.scales[0] = scales; p.biases[0] = biases; p.y[0] = y; p.N[0] = N; p.first_block[0] = 0;
  qmv_flow_body<SPW, RB, F32OUT, 1, F16, true>(p);
}

// The grouped form (2..4 packs sharing x) with preloaded arguments: the fourteen preloaded words hold what every
// workgroup needs (x, K, the shape word, where each pack's workgroups start) and the first pack; the other packs
// and the first pack's y follow as an aggregate, which is read from the argument buffer.
template <int C>
struct FlowRest {
  void* y0;
  const uint32_t* w[C - 1];
  const uint16_t* scales[C - 1];
  const uint16_t* biases[C - 1];
  void* y[C - 1];
  int N[C - 1];
};

template <int SPW, int RB, bool F32OUT, int C, bool F16 = false>
__global__ __launch_bounds__(64 * kMaxWavesPerWg) void qmv_flow_kernel_g(
    const uint16_t* x, int K, uint32_t shape, int N0, int fb1, int fb2, int fb3, const uint32_t* w0,
    const uint16_t* scales0, const uint16_t* biases0, const FlowRest<C> rest)
{
  FlowParams<C> p;
  p.h.x = x; p.h.residual = nullptr; p.h.K = K; p.h.shape = shape;
  p.w[0] = w0; p.scales[0] = scales0; p.biases[0] = biases0; p.y[0] = rest.y0; p.N[0] = N0; p.first_block[0] = 0;
  const int fb[3] = {fb1, fb2, fb3};
#pragma unroll
  for (int i = 1; i < C; ++i) {
    p.w[i] = rest.w[i - 1]; p.scales[i] = rest.scales[i - 1]; p.biases[i] = rest.biases[i - 1]; p.y[i] = rest.y[i - 1];
    p.N[i] = rest.N[i - 1]; p.first_block[i] = fb[i - 1];
  }
  qmv_flow_body<SPW, RB, F32OUT, C, F16, true>(p);
}

namespace {

struct FlowPlan {
  int spw, wk, wr, rb;
};

// Slices per wavefront and K parts, from measurements on MI355X with HBM-cold packs: up to three slices (K <= 6144)
// a wavefront walks the whole K; longer rows are split between 2 to 4 wavefronts of the workgroup (12288->4096:
// 7.5 us as 2 parts x 3 slices x 4 rows against 8.0 as one part of 6 slices; 17408->5120: 14.2 us with one row set
// of 3 parts per workgroup against 15.9 with two, while 12288->4096 prefers two row sets of 2 parts: 8.0 against
// 9.2; eight rows per wavefront measured slower everywhere).  Four wavefronts per workgroup up to two parts; two
// rows per wavefront on small packs (more, shorter wavefronts spread the pack over the CUs sooner), four on large
// ones; x shared through LDS.
FlowPlan flow_plan(int K, double pack_bytes)
{
  const int slices = (K + kSlice - 1) / kSlice;
  FlowPlan pl{0, 0, 0, 0};
  // A forced plan for measurements, "spw,wk,wr,rb" in VPQ_FLOW_PLAN (the counterpart of the reference's forced GEMM
  // route, metal-minimax-h3-transformer.cc:1912-1967); taken only if it covers K, checked again by the caller.
  static const char* forced = getenv("VPQ_FLOW_PLAN");
  if (forced != nullptr) {
    FlowPlan f{0, 0, 0, 0};
    if (sscanf(forced, "%d,%d,%d,%d", &f.spw, &f.wk, &f.wr, &f.rb) == 4 && f.spw * f.wk >= slices) { return f; }
  }
  pl.wk = slices <= 3 ? 1 : (slices + 3) / 4;
  if (pl.wk == 1 && slices > 3) { pl.wk = 2; }
  if (slices > 3 && slices <= 8) { pl.wk = 2; }
  if (pl.wk > 4) { return pl; }
  pl.spw = (slices + pl.wk - 1) / pl.wk;
  pl.wr = pl.wk == 1 ? 4 : (pl.wk == 2 ? 2 : 1);
  pl.rb = pl.wk == 1 ? ((pl.spw <= 2 && pack_bytes >= 40e6) ? 4 : 2) : (pack_bytes >= 20e6 ? 4 : 2);
  return pl;
}

template <int S, int R, bool F32, int C, bool F16 = false>
hipError_t launch_flow_kernel(dim3 grid, dim3 block, size_t lds_bytes, hipStream_t st, const FlowParams<C>& p)
{
  static std::once_flag once;          // one per instantiation
  static hipError_t attr_status = hipSuccess;
  if constexpr (C == 1) {
    const auto kern = qmv_flow_kernel_1<S, R, F32, F16>;
    std::call_once(once, [&] {
      attr_status = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        kMaxLdsBytes);
    });
    if (attr_status != hipSuccess) { return attr_status; }
    return launch_kernel(kern, grid, block, lds_bytes, st, p.h.x, p.w[0], p.scales[0], p.biases[0], p.y[0], p.h.K,
                         p.h.shape, p.N[0], p.h.residual);
  } else {
    // a grouped launch has no residual
    const auto kern = qmv_flow_kernel_g<S, R, F32, C, F16>;
    std::call_once(once, [&] {
      attr_status = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        kMaxLdsBytes);
    });
    if (attr_status != hipSuccess) { return attr_status; }
    if (p.h.residual != nullptr) { return hipErrorInvalidValue; }
    FlowRest<C> rest;
    rest.y0 = p.y[0];
    int fb[3] = {0x7fffffff, 0x7fffffff, 0x7fffffff};
    for (int i = 1; i < C; ++i) {
      rest.w[i - 1] = p.w[i]; rest.scales[i - 1] = p.scales[i]; rest.biases[i - 1] = p.biases[i]; rest.y[i - 1] = p.y[i];
      rest.N[i - 1] = p.N[i];
      fb[i - 1] = p.first_block[i];
    }
    return launch_kernel(kern, grid, block, lds_bytes, st, p.h.x, p.h.K, p.h.shape, p.N[0], fb[0], fb[1], fb[2], p.w[0],
                         p.scales[0], p.biases[0], rest);
  }
}

template <int C>
hipError_t dispatch_flow(const FlowPlan& pl, bool y_f32, const FlowHead& h, const FlowSeg* segs, int rows_per_block,
                         dim3 block, size_t lds_bytes, hipStream_t st, bool f16)
{
  FlowParams<C> p;
  p.h = h;
  int blocks = 0;
  for (int i = 0; i < C; ++i) {
    p.w[i] = segs[i].w; p.scales[i] = segs[i].scales; p.biases[i] = segs[i].biases; p.y[i] = segs[i].y; p.N[i] = segs[i].N;
    p.first_block[i] = blocks;
    blocks += (segs[i].N + rows_per_block - 1) / rows_per_block;
  }
  const dim3 grid((unsigned)blocks);
  // grouped launches store the element type
  if (C > 1 && y_f32) { return hipErrorInvalidValue; }
#define VPQ_FLOW(S, R)                                                                                    \
  if (pl.spw == S && pl.rb == R) {                                                                        \
    if constexpr (C == 1) {                                                                               \
      if (y_f32) {                                                                                        \
        return f16 ? launch_flow_kernel<S, R, true, 1, true>(grid, block, lds_bytes, st, p)               \
                   : launch_flow_kernel<S, R, true, 1, false>(grid, block, lds_bytes, st, p);             \
      }                                                                                                   \
    }                                                                                                     \
    return f16 ? launch_flow_kernel<S, R, false, C, true>(grid, block, lds_bytes, st, p)                  \
               : launch_flow_kernel<S, R, false, C, false>(grid, block, lds_bytes, st, p);                \
  }
  // every (slices per wavefront, rows per wavefront) that flow_plan can return
  VPQ_FLOW(1, 2) VPQ_FLOW(2, 2) VPQ_FLOW(3, 2) VPQ_FLOW(4, 2)
  VPQ_FLOW(1, 4) VPQ_FLOW(2, 4) VPQ_FLOW(3, 4) VPQ_FLOW(4, 4)
#undef VPQ_FLOW
  return hipErrorInvalidValue;
}

// segs[0 .. count): the packs; count == 1 takes the one-line argument form.
hipError_t launch_flow(hipStream_t st, const FlowSeg* segs, int count, const QmvArgs& a, double pack_bytes,
                       bool f16 = false)
{
  const FlowPlan pl = flow_plan(a.K, pack_bytes);
  if (pl.spw == 0 || pl.wk < 1 || pl.wk > 4 || pl.wr < 1 || pl.wk * pl.wr > kMaxWavesPerWg ||
      pl.wk * pl.spw * kSlice < a.K) {
    return hipErrorInvalidValue;
  }
  FlowHead h;
  h.x = a.x;
  h.residual = count == 1 ? a.residual : nullptr;
  h.K = a.K;
  h.shape = ((uint32_t)(pl.wk - 1) << 24) | ((uint32_t)(pl.wr - 1) << 26) | ((uint32_t)(count == 1 ? a.gate_act : 0) << 29);
  for (int wv = 0; wv < pl.wk * pl.wr; ++wv) { h.shape |= (uint32_t)(wv / pl.wk) << (3 * wv); }
  const int rows_per_block = pl.wr * pl.rb;
  const int W = pl.wk * pl.wr;
  const int ndma = (2 * pl.rb * pl.spw * 4 + 63) / 64;
  const size_t lds_bytes = (size_t)pl.wk * pl.spw * (kSlice * 2) + (size_t)W * ndma * 1024 +
                           (size_t)W * pl.rb * sizeof(float);
  if (lds_bytes > (size_t)kMaxLdsBytes) { return hipErrorInvalidValue; }
  const dim3 block((unsigned)(64 * W));
  switch (count) {
    case 1: return dispatch_flow<1>(pl, a.y_f32, h, segs, rows_per_block, block, lds_bytes, st, f16);
    case 2: return dispatch_flow<2>(pl, a.y_f32, h, segs, rows_per_block, block, lds_bytes, st, f16);
    case 3: return dispatch_flow<3>(pl, a.y_f32, h, segs, rows_per_block, block, lds_bytes, st, f16);
    case 4: return dispatch_flow<4>(pl, a.y_f32, h, segs, rows_per_block, block, lds_bytes, st, f16);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

bool qmv_flow_supports(int K, int N, int M)
{
  return M == 1 && N >= 1 && K >= kSlice && K % 512 == 0 && K <= 32768;
}

hipError_t launch_qmv_flow(hipStream_t st, const QmvArgs& a)
{
  const FlowSeg seg{a.w, a.scales, a.biases, a.y, a.N};
  return launch_flow(st, &seg, 1, a, (double)a.N * (double)a.K * 9.0 / 16.0);
}

// The same kernel over IEEE binary16 elements (x, scales, biases, y, residual).
hipError_t launch_qmv_flow_f16(hipStream_t st, const QmvArgs& a)
{
  const FlowSeg seg{a.w, a.scales, a.biases, a.y, a.N};
  return launch_flow(st, &seg, 1, a, (double)a.N * (double)a.K * 9.0 / 16.0, true);
}

hipError_t launch_qmv_flow_group(hipStream_t st, const QmvArgs& a, const QmvGroup& g, bool f16)
{
  FlowSeg segs[4];
  double bytes = 0.0;
  for (int i = 0; i < g.count; ++i) {
    segs[i] = FlowSeg{g.seg[i].w, g.seg[i].scales, g.seg[i].biases, g.seg[i].y, g.seg[i].N};
    bytes += (double)g.seg[i].N * (double)a.K * 9.0 / 16.0;
  }
  QmvArgs b = a;
  b.residual = nullptr;
  b.gate_act = 0;
  return launch_flow(st, segs, g.count, b, bytes, f16);
}

}  // namespace vpq

// QMM main kernel: y[M,N] = x[M,K] . bf16(W)^T (+ t[M,r] . B[N,r]^T) on
// v_mfma_f32_32x32x16_bf16 with fp32 accumulation.
//
// One workgroup owns a 256(M) x 128(N) tile of y and runs 8 wavefronts in two
// roles, one of each on every SIMD, so that the matrix pipe and the vector ALU
// work at the same time without relying on instruction scheduling inside a
// wavefront:
//   * 4 consumer wavefronts (2x2) only read operand fragments from LDS and issue
//     MFMAs; each accumulates 128 x 64 of the tile in 128 registers (0.75 KB of
//     LDS reads per MFMA; on this part sustained MFMA throughput on real data is
//     bounded by power, so bytes moved per MFMA matter as much as issue slots);
//   * 4 producer wavefronts bring the next tiles in.  Per 64-wide K step (one
//     quantization group, so one scale/bias per weight row per step):
//       x tile [256,64] bf16   global -> LDS by 128-bit direct-to-LDS loads (no
//                              registers, no VALU), 8 rows x 128 contiguous bytes
//                              per load instruction;
//       W tile [128,64]        32 codes per thread: global -> registers ->
//                              fp32 fma(s,q,b) -> bf16 RNE -> LDS.  The value is
//                              bf16_rne(fp32(s*q+b)), the tile arithmetic of
//                              gpu-kernels/metal/quant/affine_qmm_steel.metal:78-96
//                              (Compute=float) and affine_qmm_mma.metal:96-104.
// Three LDS stages: while the consumers work on step s the producers fill the
// stage of step s+2, so a global load has two steps to land; one s_barrier per
// step.  Keeping loads in flight across a barrier needs exact waits on the load
// counter, which the compiler cannot provide for values carried around a loop
// (it waits for everything).  So in the steady state the producers request
// their codes and scales with load instructions written out by hand and wait
// for them with explicit counts, and the x tiles and W tiles live in two
// separate LDS arrays, so that a store of dequantized weights is not ordered
// after the x tile still in flight.
// LDS rows are 128 bytes (64 bf16) with the eight 16-byte chunks of a row stored
// at position chunk ^ ((row >> 1) & 7): the 128-bit operand reads of the MFMAs
// (lane = row) then spread over all 64 banks.
// With a LoRA the same accumulators take r more values of K from t[M,r] and
// B[N,r] (dense, both through direct-to-LDS loads) before the single store
// (gpu-kernels/metal/gemm/dense_gemm_mma.metal:297-348).
#include <type_traits>

#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

constexpr int TM = 256, TN = 128, TK = 64;
constexpr int kConsumers = 4;                        // consumer wavefronts: kConsumers/2 along M, 2 along N
constexpr int kProducers = 4;                        // producer wavefronts (8 in the 128 x 256 grouped form)
constexpr int kThreads = (kConsumers + kProducers) * 64;
constexpr int kStages = 3;
constexpr int kRowB = TK * 2;                       // 128 bytes per LDS row

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
  // SwiGLU store (gpu-kernels/metal/quant/affine_qmm_steel.metal:663-768): the pack is an
  // interleaved gate|up matrix and y[m * out_stride + out_off + g] = silu(gate_g) * up_g.
  int gate_act, out_stride, out_off;
  // Split-K (ksplit > 1): workgroup blockIdx.x covers tile blockIdx.x % tiles and the K steps
  // [ks * steps_per_split, ...) with ks = blockIdx.x / tiles; its fp32 accumulators go to
  // plane[ks][M][N] and a fold kernel adds the planes in order and rounds once
  // (generative-models/shared/mma-splitk.h:30-52: f32 planes, so the output is rounded once
  // whatever the split count).
  int ksplit, steps_per_split;
  float* plane;
  // Grouped (expert-sorted) form, rows in blocks of the tile height that each belong to one expert
  // (gpu-kernels/metal/quant/affine_qmm_steel.metal:1022-1040): tile2e[block] is the expert whose
  // slab of the batched pack [E, N, ...] the block multiplies (< 0: nothing to do); with srow, x row
  // of slot i is x[srow[i]] (< 0: a padding slot, whose output is zero); with sdst, the output row of
  // slot i goes to y[sdst[i]] (< 0: not written).
  const int* tile2e = nullptr;
  const int* srow = nullptr;
  const int* sdst = nullptr;
  int n_experts = 0, rows_x = 0, rows_y = 0;
};

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

// Byte I of a dword as fp32 (selects v_cvt_f32_ubyteI).
template <int I>
__device__ __forceinline__ float ubyte_f32(uint32_t v) { return (float)((v >> (8 * I)) & 0xffu); }

// 8 nibbles of one word -> 8 bf16 (F16: IEEE binary16) of fma(s, q, b), as one 16-byte LDS chunk.
template <bool F16 = false>
__device__ __forceinline__ uint4 dequant_word(uint32_t word, float s, float b)
{
  uint32_t lo = word & 0x0f0f0f0fu;                // q0 q2 q4 q6
  uint32_t hi = (word >> 4) & 0x0f0f0f0fu;         // q1 q3 q5 q7
  // No instruction: keeps the masked words as they are, so that each value is one v_cvt_f32_ubyteN
  // of them (otherwise the mask is folded into a bit-field extract per value, one instruction more).
  asm volatile("" : "+v"(lo), "+v"(hi));
  const float v0 = fmaf(s, ubyte_f32<0>(lo), b);
  const float v1 = fmaf(s, ubyte_f32<0>(hi), b);
  const float v2 = fmaf(s, ubyte_f32<1>(lo), b);
  const float v3 = fmaf(s, ubyte_f32<1>(hi), b);
  const float v4 = fmaf(s, ubyte_f32<2>(lo), b);
  const float v5 = fmaf(s, ubyte_f32<2>(hi), b);
  const float v6 = fmaf(s, ubyte_f32<3>(lo), b);
  const float v7 = fmaf(s, ubyte_f32<3>(hi), b);
  uint4 o;
  o.x = pack_elt2<F16>(v0, v1);
  o.y = pack_elt2<F16>(v2, v3);
  o.z = pack_elt2<F16>(v4, v5);
  o.w = pack_elt2<F16>(v6, v7);
  return o;
}

// Workgroup barrier without a memory fence: the callers wait on the counters they need.
// The empty statements keep the compiler from moving LDS accesses across it.
__device__ __forceinline__ void wg_barrier()
{
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// One step's codes (32 values: 16 bytes at 4 bits, 2 x 16 at 8 bits), scale and bias of a producer
// thread, requested by load instructions the compiler does not track: the owner waits for them with
// wait_codes().
template <int BITS>
struct CodeRegsT {
  u32x4 codes;
  uint32_t s_bits, b_bits;
};
template <>
struct CodeRegsT<8> {
  u32x4 codes, codes2;
  uint32_t s_bits, b_bits;
};
using CodeRegs = CodeRegsT<4>;

__device__ __forceinline__ void request_code_words(CodeRegsT<4>& r, const uint8_t* codes)
{
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r.codes) : "v"(codes) : "memory");
}
__device__ __forceinline__ void request_code_words(CodeRegsT<8>& r, const uint8_t* codes)
{
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r.codes) : "v"(codes) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(r.codes2) : "v"(codes) : "memory");
}

template <int BITS>
__device__ __forceinline__ void request_codes(CodeRegsT<BITS>& r, const uint8_t* codes, const uint16_t* s,
                                              const uint16_t* b)
{
  request_code_words(r, codes);
  asm volatile("global_load_ushort %0, %1, off" : "=v"(r.s_bits) : "v"(s) : "memory");
  asm volatile("global_load_ushort %0, %1, off" : "=v"(r.b_bits) : "v"(b) : "memory");
}

// The codes alone (scale and bias come from the LDS ring, see SBR).
template <int BITS>
__device__ __forceinline__ void request_codes_only(CodeRegsT<BITS>& r, const uint8_t* codes)
{
  request_code_words(r, codes);
}

// Scale and bias of one row and step from the ring, as loads the compiler does not track (it would order
// them after every direct-to-LDS load of the wavefront); the caller's LDS queue is empty before them.
template <int BITS>
__device__ __forceinline__ void read_scale_bias(CodeRegsT<BITS>& r, uint32_t s_addr, uint32_t b_addr)
{
  asm volatile("ds_read_u16 %0, %1" : "=v"(r.s_bits) : "v"(s_addr) : "memory");
  asm volatile("ds_read_u16 %0, %1" : "=v"(r.b_bits) : "v"(b_addr) : "memory");
}

__device__ __forceinline__ uint32_t lds_addr_of(const uint8_t* q)
{
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)q;
}

// 16 bytes per lane, global -> LDS at lds_dst + 16 * lane, written out by hand for the same reason.
// The LDS base travels in M0, bound as an operand: the compiler writes it and knows its value, as for the
// builtin form used elsewhere in this kernel (the s_nop is the wait state between that write and the load).
__device__ __forceinline__ void dma16_raw(uint32_t lds_dst, const uint8_t* src)
{
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_dst);
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "{m0}"(m0v) : "memory");
}

// Waits until at most YOUNGER vector-memory requests issued after r's are outstanding; the
// registers pass through the statement so that no use of them can be moved above the wait.
template <int YOUNGER>
__device__ __forceinline__ void wait_codes(CodeRegsT<4>& r)
{
  asm volatile("s_waitcnt vmcnt(%3)" : "+v"(r.codes), "+v"(r.s_bits), "+v"(r.b_bits) : "n"(YOUNGER) : "memory");
}
template <int YOUNGER>
__device__ __forceinline__ void wait_codes(CodeRegsT<8>& r)
{
  asm volatile("s_waitcnt vmcnt(%4)" : "+v"(r.codes), "+v"(r.codes2), "+v"(r.s_bits), "+v"(r.b_bits) : "n"(YOUNGER) : "memory");
}

// The same for the register set of a step (one per producer thread in every form built).
template <int YOUNGER, int BITS>
__device__ __forceinline__ void wait_codes(CodeRegsT<BITS> (&r)[1]) { wait_codes<YOUNGER>(r[0]); }

// 8 bytes of two packed words -> 8 bf16 of fma(s, q, b), as one 16-byte LDS chunk (the 8-bit pack).
__device__ __forceinline__ uint4 dequant_bytes(uint32_t w0, uint32_t w1, float s, float b)
{
  uint4 o;
  o.x = pack_bf16x2(fmaf(s, ubyte_f32<0>(w0), b), fmaf(s, ubyte_f32<1>(w0), b));
  o.y = pack_bf16x2(fmaf(s, ubyte_f32<2>(w0), b), fmaf(s, ubyte_f32<3>(w0), b));
  o.z = pack_bf16x2(fmaf(s, ubyte_f32<0>(w1), b), fmaf(s, ubyte_f32<1>(w1), b));
  o.w = pack_bf16x2(fmaf(s, ubyte_f32<2>(w1), b), fmaf(s, ubyte_f32<3>(w1), b));
  return o;
}

}  // namespace

// TMK x TNK: rows of x and weight rows per workgroup: 256 x 128, or 128 x {128, 256} for the grouped
// form, whose blocks of rows are 128 tall (the wider tile gives a K step as much work as 256 x 128).
// P: producer wavefronts.  Where the step is as long as a producer's chain (wait, dequantize, store,
// wait, barrier) -- the 128-row forms, with half the MFMAs per weight -- 8 producers halve that chain.
// SBR: scales and biases come through an LDS ring in windows of 8 K steps (16 bytes per row and array),
// brought in by the CONSUMER wavefronts, whose load counter nothing else uses: a 2-byte load per row, array
// and step costs a 32-byte sector each, twice the bytes of the codes.  Needs K % 512 == 0, 16-byte
// aligned scales and biases and no split of K.
// F16: x, scales, biases, the adapter's factors and y are IEEE binary16 (the reference's VPIPE_ELT = half build): the
// weight tile is f16_rne(fp32(s*q+b)), the MFMA v_mfma_f32_32x32x16_f16; everything else is the same byte traffic.
template <bool LORA, int TMK = TM, int TNK = TN, bool GROUPED = false, int P = kProducers, bool SBR = false, int BITS = 4,
          int GROUP = 64, bool F16 = false>
__global__ __launch_bounds__((kConsumers + P) * 64) void qmm_tile_kernel(const TileParams p)
{
  static_assert(!F16 || (BITS == 4 && GROUP == 64 && !GROUPED && !SBR), "binary16 elements: the plain 4-bit group-64 tile");
  static_assert((TMK == 256 && TNK == 128 && P == 4) || (TMK == 128 && !LORA && (TNK == 128 || TNK == 256)), "tiles built");
  static_assert(TMK % (8 * P) == 0 && TNK % (32 * P) == 0, "whole loads per producer");
  constexpr int kWStage = TNK * kRowB;             // 16 KB at 128 weight rows
  constexpr int kWH = TNK / (32 * P);              // weight rows (code requests) per producer thread and step
  constexpr int kJT = TNK / 64;                    // 32-row W fragments per consumer wavefront
  constexpr int kCR = ((SBR ? 0 : 2) + BITS / 4) * kWH;   // code (, scale and bias) requests per producer thread and step
  static_assert(BITS == 4 || (BITS == 8 && kWH == 1 && !LORA), "widths built");
  // GROUP: values per scale and bias, 64 or 32 (affine_qmm_steel_w4g32, gpu-kernels/metal/quant/
  // affine_qmm_steel.metal:618-640).  A producer thread's 32 values of a step are one group of 32: it reads
  // the scale of its half.
  static_assert(GROUP == 64 || (GROUP == 32 && !SBR && !GROUPED && !LORA && BITS == 4), "groups built");
  constexpr int kGPS = TK / GROUP;                 // groups per K step
  using CodeRegs = CodeRegsT<BITS>;                // BITS: 4, or 8 (one byte per value: gpu-kernels/metal/quant/affine_qmm_steel.metal:1601-1672)
  constexpr int kSbSlot = 2 * TNK * 16;            // one window of the ring: scales | biases, 16 bytes per row
  static_assert(!SBR || kWH == 1, "one row per producer thread");
  constexpr int kWaveM = TMK / (kConsumers / 2);   // x rows per consumer wavefront
  constexpr int kIT = kWaveM / 32;                 // 32-row x fragments per consumer wavefront
  constexpr int kXStage = TMK * kRowB;             // 32 KB at 256 rows
  constexpr int kXL = TMK / (8 * P);               // x-tile loads per producer wavefront and step
  __shared__ __attribute__((aligned(16))) uint8_t x_lds[kStages * kXStage];   // 96 KB
  __shared__ __attribute__((aligned(16))) uint8_t w_lds[kStages * kWStage];   // 48 KB
  __shared__ __attribute__((aligned(16))) uint8_t sb_ring[SBR ? 2 * kSbSlot : 16];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool producer = wave >= kConsumers;

  // Consecutive workgroups walk M first: they share one weight tile.
  const int tiles = p.tiles_m * p.tiles_n;
  const int ks = p.ksplit > 1 ? (int)blockIdx.x / tiles : 0;
  const int tile = (int)blockIdx.x - ks * tiles;
  const int tm = tile % p.tiles_m;
  const int tn = tile / p.tiles_m;
  const int m0 = tm * TMK, n0 = tn * TNK;
  const uint32_t* pw_base = p.w;
  const uint16_t* ps_base = p.scales;
  const uint16_t* pb_base = p.biases;
  if constexpr (GROUPED) {
    const int e = p.tile2e[tm];
    if (e < 0 || e >= p.n_experts) { return; }        // the whole workgroup, before any barrier
    pw_base += (size_t)e * (size_t)p.N * (size_t)(p.K >> (BITS == 4 ? 3 : 2));
    ps_base += (size_t)e * (size_t)p.N * (size_t)(p.K >> 6);
    pb_base += (size_t)e * (size_t)p.N * (size_t)(p.K >> 6);
  }
  // This workgroup's K steps: all of them, or its share of a split.
  const int k_first = ks * p.steps_per_split;
  const int KT = p.ksplit > 1 ? ((p.K / TK - k_first) < p.steps_per_split ? (p.K / TK - k_first) : p.steps_per_split)
                              : p.K / TK;

  if (producer) {
    // ======================= producers =======================
    const int pw = wave - kConsumers;     // 0..P-1
    const int pt = tid - kConsumers * 64; // 0..64P-1
    // x tile: 32 direct-to-LDS loads per step, 8 per wavefront.  Load i of wave pw covers tile
    // rows (8 pw + i)*8 .. +8; lane l takes row l/8, LDS position l%8.
    const bool gathered = GROUPED && p.srow != nullptr;
    const uint8_t* xblk = reinterpret_cast<const uint8_t*>(p.x) + (gathered ? (size_t)0 : (size_t)m0 * p.K * 2) +
                          (size_t)k_first * (TK * 2);
    uint32_t a_off[kXL];
#pragma unroll
    for (int i = 0; i < kXL; ++i) {
      const int row = (pw * kXL + i) * 8 + (lane >> 3);
      const int chunk = swz(row, lane & 7);
      int rg = (m0 + row < p.M) ? row : (p.M - 1 - m0);
      if (gathered) {
        // A padding slot reads row 0 (any readable row): its output is written as zero.
        const int src = p.srow[m0 + rg];
        rg = (src >= 0 && src < p.rows_x) ? src : 0;
      }
      a_off[i] = (uint32_t)rg * (uint32_t)p.K * 2u + (uint32_t)chunk * 16u;
    }
    // W tile: thread pt dequantizes 32 codes of row pt/2 (k half pt%2) per step, and with kWH = 2 those of
    // row pt/2 + 32 P as well.
    const int qrow = pt >> 1, qhalf = pt & 1;
    const uint8_t* wrow[kWH];
    const uint16_t* srow[kWH];
    const uint16_t* brow[kWH];
#pragma unroll
    for (int h = 0; h < kWH; ++h) {
      const int qrg = (n0 + qrow + 32 * P * h < p.N) ? (n0 + qrow + 32 * P * h) : (p.N - 1);
      wrow[h] = reinterpret_cast<const uint8_t*>(pw_base) + (size_t)qrg * (p.K * BITS / 8) + qhalf * (4 * BITS) +
                (size_t)k_first * (TK * BITS / 8);
      srow[h] = ps_base + (size_t)qrg * (p.K / GROUP) + (size_t)k_first * kGPS + (GROUP == 32 ? qhalf : 0);
      brow[h] = pb_base + (size_t)qrg * (p.K / GROUP) + (size_t)k_first * kGPS + (GROUP == 32 ? qhalf : 0);
    }
    int b_dst[4];                          // row + 32 P has the same swizzle: + 32 P rows of bytes
#pragma unroll
    for (int i = 0; i < 4; ++i) { b_dst[i] = qrow * kRowB + swz(qrow, qhalf * 4 + i) * 16; }

    auto issue_x = [&](int step, int stage) {
      const uint8_t* src = xblk + (size_t)step * (TK * 2);
      uint8_t* dst = x_lds + stage * kXStage + pw * (kXL * 8 * kRowB);
#pragma unroll
      for (int i = 0; i < kXL; ++i) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + a_off[i]),
                                         (__attribute__((address_space(3))) void*)(dst + i * (8 * kRowB)), 16, 0, 0);
      }
    };
    auto dequant_to = [&](int stage, const CodeRegs (&r)[kWH]) {
#pragma unroll
      for (int h = 0; h < kWH; ++h) {
        const float sc = elt_bits_to_f32<F16>(r[h].s_bits), bi = elt_bits_to_f32<F16>(r[h].b_bits);
        uint8_t* nb = w_lds + stage * kWStage + h * (32 * P * kRowB);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if constexpr (BITS == 4) {
            *reinterpret_cast<uint4*>(nb + b_dst[i]) = dequant_word<F16>(r[h].codes[i], sc, bi);
          } else {
            const u32x4& cw = i < 2 ? r[h].codes : r[h].codes2;
            *reinterpret_cast<uint4*>(nb + b_dst[i]) = dequant_bytes(cw[2 * (i & 1)], cw[2 * (i & 1) + 1], sc, bi);
          }
        }
      }
    };
    auto request = [&](CodeRegs (&r)[kWH], int step) {
#pragma unroll
      for (int h = 0; h < kWH; ++h) {
        if constexpr (SBR) {
          request_codes_only(r[h], wrow[h] + (size_t)step * (TK * BITS / 8));
        } else {
          request_codes(r[h], wrow[h] + (size_t)step * (TK * BITS / 8), srow[h] + step * kGPS, brow[h] + step * kGPS);
        }
      }
    };
    // SBR: scale and bias of this thread's row for step t, from the window t / 8 of the ring.
    const uint32_t sb_row = lds_addr_of(sb_ring) + (uint32_t)qrow * 16u;
    auto fetch_sb = [&](CodeRegs (&r)[kWH], int t) {
      if constexpr (SBR) {
        const uint32_t a = sb_row + (uint32_t)((t >> 3) & 1) * kSbSlot + (uint32_t)(t & 7) * 2u;
        read_scale_bias(r[0], a, a + TNK * 16);
      }
    };
    auto settle_sb = [&](CodeRegs (&r)[kWH]) {
      if constexpr (SBR) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0].s_bits), "+v"(r[0].b_bits) : : "memory"); }
    };

    // Prologue: steps 0 and 1 complete in stages 0 and 1; codes of steps 2 and 3 requested.
    CodeRegs ra[kWH], rb[kWH];             // codes of even / odd steps
    request(ra, 0);
    request(rb, KT > 1 ? 1 : 0);
    issue_x(0, 0);
    if (KT > 1) { issue_x(1, 1); }
    wait_codes<0>(ra);
    wait_codes<0>(rb);
    if constexpr (SBR) {
      wg_barrier();                        // the consumers have brought in the first two windows of the ring
      fetch_sb(ra, 0);
      fetch_sb(rb, KT > 1 ? 1 : 0);
      settle_sb(ra);
      settle_sb(rb);
    }
    dequant_to(0, ra);
    if (KT > 1) { dequant_to(1, rb); }
    request(ra, KT > 2 ? 2 : 0);
    request(rb, KT > 3 ? 3 : 0);
    fetch_sb(ra, 2);                       // step 2's scale and bias (window 0)
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" : : "n"(2 * kCR) : "memory");   // all but the code requests of steps 2, 3
    settle_sb(ra);
    wg_barrier();

    // Steady state, step s fills the stage of step t = s+2.  Requests in issue order, with X = kXL
    // (8 at 256 rows of x) and C = kCR (3 at 128 weight rows):
    //   ..., x(t-1) [X], codes(t+1) [C], x(t) [X], codes(t+2) [C]
    // x(t) goes out first so that it has two whole steps to land.  codes(t) were requested two
    // steps ago: X + C + X younger requests may stay in flight while they are awaited (19).
    // Before the barrier x(t-1), the tile of step s+1, must have landed: C + X + C younger requests (14).
    // The first fill follows the prologue, where only codes(3) [C] and x(2) [X] are younger (11).
    // rn: the other register set, which the next fill uses.  SBR: its scale and bias are read from the ring
    // here, behind this step's work, and have landed by the wait at the end (not in the chain of the next fill).
    auto fill = [&](auto younger, int t, int stage, CodeRegs (&r)[kWH], CodeRegs (&rn)[kWH]) {
      issue_x(t, stage);
      wait_codes<decltype(younger)::value>(r);
      dequant_to(stage, r);
      request(r, t + 2 < KT ? t + 2 : t);           // the last two requests are never used
      fetch_sb(rn, t + 1);
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" : : "n"(kXL + 2 * kCR) : "memory");
      settle_sb(rn);
    };
    auto next_stage = [](int stage) { return stage == kStages - 1 ? 0 : stage + 1; };
    auto odd_fill = [&](int t, int stage) {
      if (t < KT) {
        fill(std::integral_constant<int, 2 * kXL + kCR>(), t, stage, rb, ra);
      } else {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      }
    };
    int tstage = 2;                        // stage of step s+2
    int s = 0;
    if (KT > 2) {
      fill(std::integral_constant<int, kXL + kCR>(), 2, tstage, ra, rb);
      wg_barrier();
      tstage = next_stage(tstage);
      odd_fill(3, tstage);
      wg_barrier();
      tstage = next_stage(tstage);
      s = 2;
    }
    for (; s + 2 < KT; s += 2) {
      fill(std::integral_constant<int, 2 * kXL + kCR>(), s + 2, tstage, ra, rb);   // even step: codes in ra
      wg_barrier();
      tstage = next_stage(tstage);
      odd_fill(s + 3, tstage);
      wg_barrier();
      tstage = next_stage(tstage);
    }
    for (; s < KT; ++s) {                  // the last one or two steps fill nothing
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      wg_barrier();
    }

    if (LORA) {
      const int steps = (p.r + TK - 1) / TK;
      for (int st = 0; st < steps; ++st) {
        const int kleft = p.r - st * TK;                 // >= 8, a multiple of 8
        const int chunks = kleft >= TK ? 8 : (kleft >> 3);
        // an odd number of 8-value pieces (a rank of 8 mod 16): the quarter step's other half is zeros in both tiles
        const int zero_chunk = (chunks & 1) ? chunks : -1;
        // t tile: 256 rows, as the x tile; B tile: 128 rows, 4 loads per wavefront.  Stage 0.
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int row = (pw * 8 + i) * 8 + (lane >> 3);
          const int chunk = swz(row, lane & 7);
          const int rg = (m0 + row < p.M) ? (m0 + row) : (p.M - 1);
          if (chunk < chunks) {
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(p.lora_t + (size_t)rg * p.r + st * TK + chunk * 8),
                (__attribute__((address_space(3))) void*)(x_lds + pw * (64 * kRowB) + i * (8 * kRowB)), 16, 0, 0);
          } else if (chunk == zero_chunk) {
            *reinterpret_cast<uint4*>(x_lds + pw * (64 * kRowB) + i * (8 * kRowB) + lane * 16) = make_uint4(0, 0, 0, 0);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = (pw * 4 + i) * 8 + (lane >> 3);
          const int chunk = swz(row, lane & 7);
          const int rg = (n0 + row < p.N) ? (n0 + row) : (p.N - 1);
          if (chunk < chunks) {
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(p.lora_b + (size_t)rg * p.r + st * TK + chunk * 8),
                (__attribute__((address_space(3))) void*)(w_lds + pw * (32 * kRowB) + i * (8 * kRowB)), 16, 0, 0);
          } else if (chunk == zero_chunk) {
            *reinterpret_cast<uint4*>(w_lds + pw * (32 * kRowB) + i * (8 * kRowB) + lane * 16) = make_uint4(0, 0, 0, 0);
          }
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        wg_barrier();                                    // tiles ready
        wg_barrier();                                    // consumers done with them
      }
    }
    return;
  }

  // ======================= consumers =======================
  const int wm = wave >> 1, wn = wave & 1;
  floatx16 acc[kJT][kIT];   // [jt: 32 weight rows][it: 32 x rows]
#pragma unroll
  for (int jt = 0; jt < kJT; ++jt) {
#pragma unroll
    for (int it = 0; it < kIT; ++it) {
#pragma unroll
      for (int e = 0; e < 16; ++e) { acc[jt][it][e] = 0.0f; }
    }
  }
  const int frow = lane & 31;      // row of a 32-row operand fragment
  const int fkh = lane >> 5;       // which 8 of the 16 k
  int w_rd[kJT], x_rd[kIT];        // stage-relative operand rows
#pragma unroll
  for (int jt = 0; jt < kJT; ++jt) { w_rd[jt] = (wn * (TNK / 2) + jt * 32 + frow) * kRowB; }
#pragma unroll
  for (int it = 0; it < kIT; ++it) { x_rd[it] = (wm * kWaveM + it * 32 + frow) * kRowB; }
  const int f_sw = (frow >> 1) & 7;   // the tile offsets are multiples of 16 rows: same swizzle for all
  // Grouped form: a 32-row fragment of x whose slots are all padding (the tail of an expert's last block)
  // is neither read nor multiplied; its accumulators stay zero.
  bool frag_live[kIT];
#pragma unroll
  for (int it = 0; it < kIT; ++it) { frag_live[it] = true; }
  if constexpr (GROUPED) {
    static_assert(!GROUPED || kWaveM == 64, "one index per lane covers the wavefront's rows");
    const int* idx = p.srow != nullptr ? p.srow : p.sdst;
    const int lim = p.srow != nullptr ? p.rows_x : p.rows_y;
    const int v = idx[m0 + wm * kWaveM + lane];
    const unsigned long long mask = __ballot(v >= 0 && v < lim);
#pragma unroll
    for (int it = 0; it < kIT; ++it) { frag_live[it] = ((mask >> (32 * it)) & 0xffffffffull) != 0; }
  }

  auto mma_stage = [&](int stage, int ksteps) {
    const uint8_t* xb = x_lds + stage * kXStage;
    const uint8_t* wb = w_lds + stage * kWStage;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks < ksteps) {
        const int c = ((2 * ks + fkh) ^ f_sw) * 16;
        bf16x8 wf[kJT], xf[kIT];
#pragma unroll
        for (int jt = 0; jt < kJT; ++jt) { wf[jt] = *reinterpret_cast<const bf16x8*>(wb + w_rd[jt] + c); }
#pragma unroll
        for (int it = 0; it < kIT; ++it) {
          if (!GROUPED || frag_live[it]) { xf[it] = *reinterpret_cast<const bf16x8*>(xb + x_rd[it] + c); }
        }
#pragma unroll
        for (int jt = 0; jt < kJT; ++jt) {
#pragma unroll
          for (int it = 0; it < kIT; ++it) {
            if (!GROUPED || frag_live[it]) {
              if constexpr (F16) {
                typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
                acc[jt][it] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, wf[jt]),
                                                                     __builtin_bit_cast(halfx8, xf[it]), acc[jt][it], 0, 0, 0);
              } else {
                acc[jt][it] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[jt], xf[it], acc[jt][it], 0, 0, 0);
              }
            }
          }
        }
      }
    }
  };

  // SBR: window wdw of the scales and biases (K steps 8 wdw .. 8 wdw + 7) into its slot of the ring.  The
  // 2 TNK (array, row) entries of a window are dealt out 64 to a load over the four consumer wavefronts.
  auto issue_window = [&](int wdw) {
    if constexpr (SBR) {
      constexpr int kLoads = 2 * TNK / 64 / kConsumers;        // 1 at 128 rows, 2 at 256
#pragma unroll
      for (int j = 0; j < kLoads; ++j) {
        const int e = (wave * kLoads + j) * 64 + lane;         // entry: array e / TNK, row e % TNK
        const int arr = e / TNK, row = e % TNK;
        const int rg = (n0 + row < p.N) ? (n0 + row) : (p.N - 1);
        const uint16_t* src = (arr ? pb_base : ps_base) + (size_t)rg * (p.K >> 6) + (size_t)wdw * 8;
        dma16_raw(lds_addr_of(sb_ring) + (uint32_t)(wdw & 1) * kSbSlot + (uint32_t)(wave * kLoads + j) * 1024u,
                  reinterpret_cast<const uint8_t*>(src));
      }
    }
  };
  if constexpr (SBR) {
    issue_window(0);
    if (KT > 8) { issue_window(1); }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    wg_barrier();                        // the producers read the ring from here on
  }
  wg_barrier();                          // stages 0 and 1 are ready
  int cstage = 0;
  if constexpr (SBR) {
    // The producers fill two steps ahead: window s/8 + 1 is first read in step s + 5 and the slot it
    // replaces (window s/8 - 1) was last read in step s - 4.  Landed before the barrier of step s + 3.
    for (int s = 0; s < KT; ++s) {
      if ((s & 7) == 0 && s > 0 && s + 8 < KT) { issue_window((s >> 3) + 1); }
      mma_stage(cstage, 4);
      if ((s & 7) == 3) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // every operand read of this stage is done
      wg_barrier();
      cstage = (cstage == kStages - 1) ? 0 : cstage + 1;
    }
  } else {
    for (int s = 0; s < KT; ++s) {
      mma_stage(cstage, 4);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // every operand read of this stage is done
      wg_barrier();
      cstage = (cstage == kStages - 1) ? 0 : cstage + 1;
    }
  }
  if (LORA) {
    const int steps = (p.r + TK - 1) / TK;
    for (int st = 0; st < steps; ++st) {
      const int kleft = p.r - st * TK;
      const int chunks = kleft >= TK ? 8 : (kleft >> 3);
      wg_barrier();
      mma_stage(0, (chunks + 1) >> 1);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      wg_barrier();
    }
  }

  // ---- store: lane holds, for x row m = lane%32 of each it, 4 consecutive n per register quad ----
  if (p.ksplit > 1) {
    const bool vec4 = (p.N & 3) == 0;
#pragma unroll
    for (int it = 0; it < kIT; ++it) {
      const int m = m0 + wm * kWaveM + it * 32 + frow;
      if (m >= p.M) { continue; }
      float* prow = p.plane + ((size_t)ks * p.M + m) * p.N;
#pragma unroll
      for (int jt = 0; jt < kJT; ++jt) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int n = n0 + wn * (TNK / 2) + jt * 32 + rq * 8 + fkh * 4;
          if (n >= p.N) { continue; }
          if (vec4 && n + 3 < p.N) {
            floatx4 v = {acc[jt][it][rq * 4 + 0], acc[jt][it][rq * 4 + 1], acc[jt][it][rq * 4 + 2], acc[jt][it][rq * 4 + 3]};
            *reinterpret_cast<floatx4*>(prow + n) = v;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (n + e < p.N) { prow[n + e] = acc[jt][it][rq * 4 + e]; }
            }
          }
        }
      }
    }
    return;
  }
  if (p.gate_act) {
    // A register quad is (gate, up, gate, up) of features n/2 and n/2 + 1 (n is a multiple of 4):
    // the activation is register-local and a quad becomes one dword of two bf16.
    const bool pair_ok = ((p.out_stride | p.out_off) & 1) == 0;
#pragma unroll
    for (int it = 0; it < kIT; ++it) {
      const int m = m0 + wm * kWaveM + it * 32 + frow;
      if (m >= p.M) { continue; }
      uint16_t* yrow = p.y + (size_t)m * p.out_stride + p.out_off;
      bool pad_slot = false;                 // a padding slot of the grouped form: x = 0, so act(0) * 0 = +0
      if constexpr (GROUPED) {
        if (p.srow != nullptr) {
          const int src = p.srow[m];
          pad_slot = src < 0 || src >= p.rows_x;
        }
      }
#pragma unroll
      for (int jt = 0; jt < kJT; ++jt) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int n = n0 + wn * (TNK / 2) + jt * 32 + rq * 8 + fkh * 4;
          if (n >= p.N) { continue; }
          const float f0 = pad_slot ? 0.0f : gated_f32(p.gate_act, acc[jt][it][rq * 4 + 0], acc[jt][it][rq * 4 + 1]);
          const float f1 = pad_slot ? 0.0f : gated_f32(p.gate_act, acc[jt][it][rq * 4 + 2], acc[jt][it][rq * 4 + 3]);
          if (pair_ok && n + 3 < p.N) {
            *reinterpret_cast<uint32_t*>(yrow + (n >> 1)) = pack_elt2<F16>(f0, f1);
          } else {
            yrow[n >> 1] = (uint16_t)f32_to_elt_bits<F16>(f0);
            if (n + 3 < p.N) { yrow[(n >> 1) + 1] = (uint16_t)f32_to_elt_bits<F16>(f1); }
          }
        }
      }
    }
    return;
  }
  const bool vec_ok = (p.N & 3) == 0;
#pragma unroll
  for (int it = 0; it < kIT; ++it) {
    const int m = m0 + wm * kWaveM + it * 32 + frow;
    if (m >= p.M) { continue; }
    int mdst = m;
    if constexpr (GROUPED) {
      if (p.sdst != nullptr) {
        mdst = p.sdst[m];
        if (mdst < 0 || mdst >= p.rows_y) { continue; }
      }
    }
    uint16_t* yrow = p.y + (size_t)mdst * p.N;
#pragma unroll
    for (int jt = 0; jt < kJT; ++jt) {
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int n = n0 + wn * (TNK / 2) + jt * 32 + rq * 8 + fkh * 4;
        if (n >= p.N) { continue; }
        const float v0 = acc[jt][it][rq * 4 + 0], v1 = acc[jt][it][rq * 4 + 1];
        const float v2 = acc[jt][it][rq * 4 + 2], v3 = acc[jt][it][rq * 4 + 3];
        if (vec_ok && n + 3 < p.N) {
          uint2 o;
          o.x = pack_elt2<F16>(v0, v1);
          o.y = pack_elt2<F16>(v2, v3);
          *reinterpret_cast<uint2*>(yrow + n) = o;
        } else {
          const float v[4] = {v0, v1, v2, v3};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (n + e < p.N) { yrow[n + e] = (uint16_t)f32_to_elt_bits<F16>(v[e]); }
          }
        }
      }
    }
  }
}

// y[i] = bf16(plane[0][i] + plane[1][i] + ... ) in that order, i over M*N.
__global__ __launch_bounds__(256) void splitk_fold_kernel(const float* __restrict__ plane, uint16_t* __restrict__ y,
                                                          size_t count, int splits)
{
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (size_t)gridDim.x * 256) {
    float v = plane[i];
    for (int s = 1; s < splits; ++s) { v += plane[(size_t)s * count + i]; }
    y[i] = (uint16_t)f32_to_bf16_bits(v);
  }
}

// Split count by a small cost model (microseconds, from measurements on MI355X): a workgroup costs
// ~3 us to start and drain plus ~0.9 us per K step; workgroups run one per CU, so the grid takes
// ceil(workgroups / CUs) rounds; the planes are written and read once more by the fold at ~4 TB/s.
int qmm_choose_splits(int K, int N, int M, int cu_count)
{
  const int tiles = ((M + TM - 1) / TM) * ((N + TN - 1) / TN);
  const int steps = K / TK;
  const int cus = cu_count > 0 ? cu_count : 256;
  if (tiles * 2 > cus) { return 1; }                   // the tiles alone fill at least half of the chip
  auto cost = [&](int s) {
    const int per = (steps + s - 1) / s;
    const int rounds = (tiles * s + cus - 1) / cus;
    double us = rounds * (3.0 + 0.9 * per);
    if (s > 1) { us += 3.0 + (s + 0.5) * (double)M * (double)N * 4.0 / 4.0e6; }
    return us;
  };
  int best = 1;
  double best_us = cost(1);
  for (int s = 2; s <= 16 && steps / s >= 4; ++s) {
    const int per = (steps + s - 1) / s;
    if ((steps + per - 1) / per != s) { continue; }    // shares would come out uneven: another count covers it
    const double us = cost(s);
    if (us < 0.9 * best_us) { best = s; best_us = us; }
  }
  return best;
}

size_t qmm_splitk_workspace_bytes(int K, int N, int M, int cu_count)
{
  const int s = qmm_choose_splits(K, N, M, cu_count);
  return s > 1 ? (size_t)s * (size_t)M * (size_t)N * sizeof(float) : 0;
}

// The scale/bias ring's windows are 16-byte loads of 8 groups: whole windows in every row, aligned.
static bool sb_ring_ok(const GemmArgs& a)
{
  return (a.K % 512) == 0 && (reinterpret_cast<uintptr_t>(a.scales) & 15) == 0 &&
         (reinterpret_cast<uintptr_t>(a.biases) & 15) == 0;
}

hipError_t launch_qmm_tile_splitk(hipStream_t st, const GemmArgs& a, int splits, float* plane)
{
  TileParams p;
  p.w = a.w; p.scales = a.scales; p.biases = a.biases; p.x = a.x; p.y = a.y;
  p.lora_t = nullptr; p.lora_b = nullptr;
  p.K = a.K; p.N = a.N; p.M = a.M; p.r = 0;
  p.gate_act = 0; p.out_stride = a.N / 2; p.out_off = 0;
  p.tiles_m = (a.M + TM - 1) / TM;
  p.tiles_n = (a.N + TN - 1) / TN;
  const int steps = a.K / TK;
  p.steps_per_split = (steps + splits - 1) / splits;
  p.ksplit = (steps + p.steps_per_split - 1) / p.steps_per_split;
  p.plane = plane;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n * p.ksplit)), block(kThreads);
  hipError_t e = launch_kernel(qmm_tile_kernel<false>, grid, block, 0, st, p);
  if (e != hipSuccess) { return e; }
  const size_t count = (size_t)a.M * (size_t)a.N;
  size_t blocks = (count + 255) / 256;
  if (blocks > 65536) { blocks = 65536; }
  return launch_kernel(splitk_fold_kernel, dim3((unsigned)blocks), dim3(256), 0, st, plane, a.y, count, p.ksplit);
}

hipError_t launch_qmm_tile(hipStream_t st, const GemmArgs& a)
{
  TileParams p;
  p.w = a.w; p.scales = a.scales; p.biases = a.biases; p.x = a.x; p.y = a.y;
  p.lora_t = a.lora_t; p.lora_b = a.lora_b;
  p.K = a.K; p.N = a.N; p.M = a.M; p.r = a.r;
  p.gate_act = a.gate_act;
  p.out_stride = a.out_stride > 0 ? a.out_stride : a.N / 2;
  p.out_off = a.out_off;
  p.tiles_m = (a.M + TM - 1) / TM;
  p.tiles_n = (a.N + TN - 1) / TN;
  p.ksplit = 1; p.steps_per_split = a.K / TK; p.plane = nullptr;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n)), block(kThreads);
  if (a.bits == 8) {
    if (a.lora_t != nullptr || a.group != 64 || a.f16) { return hipErrorInvalidValue; }     // no 8-bit form with the adapter
    return launch_kernel(qmm_tile_kernel<false, TM, TN, false, kProducers, false, 8>, grid, block, 0, st, p);
  }
  if (a.group == 32) {
    if (a.lora_t != nullptr || a.f16) { return hipErrorInvalidValue; }
    return launch_kernel(qmm_tile_kernel<false, TM, TN, false, kProducers, false, 4, 32>, grid, block, 0, st, p);
  }
  if (a.f16) {
    return a.lora_t != nullptr
               ? launch_kernel(qmm_tile_kernel<true, TM, TN, false, kProducers, false, 4, 64, true>, grid, block, 0, st, p)
               : launch_kernel(qmm_tile_kernel<false, TM, TN, false, kProducers, false, 4, 64, true>, grid, block, 0, st, p);
  }
  return a.lora_t != nullptr ? launch_kernel(qmm_tile_kernel<true>, grid, block, 0, st, p)
                             : launch_kernel(qmm_tile_kernel<false>, grid, block, 0, st, p);
}

hipError_t launch_qmm_grouped(hipStream_t st, const GemmArgs& a, const GroupedArgs& g)
{
  TileParams p;
  p.w = a.w; p.scales = a.scales; p.biases = a.biases; p.x = a.x; p.y = a.y;
  p.lora_t = nullptr; p.lora_b = nullptr;
  p.K = a.K; p.N = a.N; p.M = a.M; p.r = 0;
  p.gate_act = a.gate_act;
  p.out_stride = a.out_stride > 0 ? a.out_stride : a.N / 2;
  p.out_off = a.out_off;
  p.tiles_m = a.M / kGroupedBlockRows;       // a.M is a whole number of blocks
  const bool wide = a.N > TN;                // 128 x 256 tiles unless one 128-wide tile holds all of N
  p.tiles_n = wide ? (a.N + 2 * TN - 1) / (2 * TN) : 1;
  p.ksplit = 1; p.steps_per_split = a.K / TK; p.plane = nullptr;
  p.tile2e = g.tile2e; p.srow = g.srow; p.sdst = g.sdst;
  p.n_experts = g.n_experts; p.rows_x = g.rows_x; p.rows_y = g.rows_y;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n)), block(kThreads);
  if (wide) {
    const dim3 block12((kConsumers + 8) * 64);
    if (a.bits == 8) {
      return sb_ring_ok(a)
                 ? launch_kernel(qmm_tile_kernel<false, kGroupedBlockRows, 2 * TN, true, 8, true, 8>, grid, block12, 0, st, p)
                 : launch_kernel(qmm_tile_kernel<false, kGroupedBlockRows, 2 * TN, true, 8, false, 8>, grid, block12, 0, st, p);
    }
    return sb_ring_ok(a) ? launch_kernel(qmm_tile_kernel<false, kGroupedBlockRows, 2 * TN, true, 8, true>, grid, block12, 0, st, p)
                         : launch_kernel(qmm_tile_kernel<false, kGroupedBlockRows, 2 * TN, true, 8>, grid, block12, 0, st, p);
  }
  if (a.bits == 8) {
    return launch_kernel(qmm_tile_kernel<false, kGroupedBlockRows, TN, true, kProducers, false, 8>, grid, block, 0, st, p);
  }
  return launch_kernel(qmm_tile_kernel<false, kGroupedBlockRows, TN, true>, grid, block, 0, st, p);
}

}  // namespace vpq

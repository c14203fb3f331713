// QMM, large-tile kernel: y[M,N] = x[M,K] . bf16(W)^T (+ t[M,r] . B[N,r]^T) for GEMMs with many
// tiles (the video-DiT projections, M in the thousands).  Same arithmetic as the 256 x 128 tile
// kernel -- W = bf16_rne(fp32(s*q+b)) (gpu-kernels/metal/quant/affine_qmm_steel.metal:78-96),
// v_mfma_f32_32x32x16_bf16 over K in ascending order, fp32 accumulators, one rounding -- and the
// same bits; what differs is who does what.
//
// A workgroup owns 256(M) x BN(N) of y, BN = 64 NT in {256, 192, 128}, and has FOUR wavefronts, one per
// SIMD, each with a 128 x (BN/2) block of accumulators (up to 256 registers, in the accumulation
// file).  A wavefront's operand reads from LDS are then (4 + NT) fragments per 4 NT MFMAs -- half the
// LDS bytes per MFMA of a 128 x 64 block -- which is what bounds the smaller tile: there the LDS
// pipe is busy longer than the matrix pipe.  With one wavefront per SIMD nothing else can fill the
// matrix pipe's shadow, so every wavefront does all three jobs and the instruction stream itself
// interleaves them: the work of a K step is cut into single instructions and dealt out over the step's MFMAs
// by a plan made at compile time, at most four issue units behind each MFMA (a fragment read for the next
// quarter step, every second time a load request, instructions of the dequantization of a coming step's
// weight tile), written as asm statements and pinned in that order by scheduling barriers.
//
// Per 64-wide K step and workgroup, everything arrives by direct-to-LDS loads:
//   x tile [256,64] bf16      8 loads per wavefront (8 rows x 128 contiguous bytes each);
//   codes  [BN rows x 32 B]   2 loads per wavefront (32 rows x 32 bytes), into a two-slot ring;
//   scales, biases            1 load each per wavefront and 8 steps (64 rows x 16 bytes), two slots.
// The BN x 8 words of a step's codes are dealt out evenly over the 256 threads for dequantization.
// The loads are written out by hand: the compiler orders every later LDS read after a direct-to-LDS
// load it knows about, whichever array that load fills, which would serialize the pipeline;
// hand-written, the only waits in the loop are the explicit ones.
// Two LDS stages of x (2 x 32 KB) and of the dequantized W (2 x 32 KB) + the rings (2 x 8 + 2 x 8 KB)
// are the whole 160 KB.
//
// A step has ONE barrier, at its 3/4 point (after the MFMAs of quarters 0..2, when every fragment of
// the step is in registers): see the pipeline's comment in the kernel.  Measured on 256 x 256 tiles
// (cycles per step; 2048 are the MFMAs alone): barrier at the step's end with the first fragment reads
// behind it 3080; this pipeline with the slot plan 2200-2250 with dense weights, 2450-2550 with the
// dequantization.  The shader clock falls as the cycles do (the part is power-limited under this load), so a
// tenth fewer cycles has been worth 1-4 % in time.
//
// Tile order: from two full rounds of the chip on, the 32 workgroups an XCD runs together form a block of
// tiles (4 x 8, 8 x 4, ...) so that they share rows of x and weight tiles through that XCD's L2; below
// that, bands of 8 rows of tiles, M first inside a band.  The store goes through LDS, a wavefront's
// block turned round 32 rows at a time, so that a store instruction covers runs of 64 NT bytes per row.
#include <string>
#include <type_traits>

#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

constexpr int BM = 256, BK = 64;
constexpr int kBigThreads = 256;
constexpr int kRow = BK * 2;                 // 128 bytes per LDS row
constexpr int kXBytes = BM * kRow;           // 32 KB per stage
constexpr int kCodeBytes = 256 * 32;         // 8 KB: the 32 bytes of codes of one K step per row
constexpr int kScaleBytes = 256 * 32;        // 8 KB: 8 scales | 8 biases (8 K steps) per row

struct BigParams {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  const uint16_t* x;
  uint16_t* y;
  const uint16_t* lora_t;   // [M,r] or nullptr
  const uint16_t* lora_b;   // [N,r]
  int K, N, M, r;
  int tiles_m, tiles_n;
  int bmt, bnt, nbn;        // tile blocks per XCD (bmt = 0: bands of 8 rows of tiles), blocks along N
  // Gated store (1 SwiGLU, 2 GEGLU): the pack is an interleaved gate|up matrix and
  // y[m * out_stride + out_off + g] = act(gate_g) * up_g (affine_qmm_steel.metal:663-768, 1460-1572).
  int gate_act, out_stride, out_off;
};

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

// Byte I of a dword as fp32 (selects v_cvt_f32_ubyteI).
template <int I>
__device__ __forceinline__ float ubyte_f32(uint32_t v) { return (float)((v >> (8 * I)) & 0xffu); }

// `when(c, f)`: f() if c -- decided at compile time for std::true_type / std::false_type, at run time for bool.
template <typename F> __device__ __forceinline__ void when(std::true_type, F&& f) { f(); }
template <typename F> __device__ __forceinline__ void when(std::false_type, F&&) {}
template <typename F> __device__ __forceinline__ void when(bool c, F&& f) { if (c) { f(); } }

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
  if constexpr (I < N) {
    f(std::integral_constant<int, I>());
    static_for<I + 1, N>(f);
  }
}

// Workgroup barrier without a memory fence: the callers wait on the counters they need.
__device__ __forceinline__ void wg_barrier()
{
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

__device__ __forceinline__ uint32_t lds_addr(const uint8_t* q)
{
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)q;
}

// 16 bytes per lane, global -> LDS at lds_dst + 16 * lane.  The LDS base travels in M0, bound as an operand: the
// compiler writes it and knows its value (the s_nop is the wait state between that write and the load).
__device__ __forceinline__ void dma16(uint32_t lds_dst, const uint8_t* src)
{
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_dst);
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "{m0}"(m0v) : "memory");
}

// The same from a wave-uniform base (scalar registers) plus a 32-bit offset per lane: stepping along K
// then costs scalar additions only.
__device__ __forceinline__ void dma16(uint32_t lds_dst, const uint8_t* base, uint32_t lane_off)
{
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_dst);
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_off), "s"(base), "{m0}"(m0v) : "memory");
}

}  // namespace

// WSRC: where the weight tile comes from.  kPacked4: 4-bit codes + scales + biases, dequantized in the kernel (the
// fused GEMM).  kDenseBf16 / kDenseF16: p.w is an expanded [N,K] matrix of 2-byte elements that goes to LDS as
// the x tile does -- the dense matrix-unit GEMM of the dequant-once route
// (gpu-kernels/metal/gemm/dense_gemm_mma.metal:44-93, 139-140, 195): same tiles, same MFMA stream, no
// dequantization pieces; any K % 32 == 0.
constexpr int kPacked4 = 0, kDenseBf16 = 1, kDenseF16 = 2, kPacked4F16 = 3, kPacked8 = 4, kPacked4G32 = 5;

template <int NT, bool LORA, int WSRC = kPacked4>
__global__ __launch_bounds__(kBigThreads) void qmm_big_kernel(const BigParams p)
{
  constexpr bool DENSE = WSRC == kDenseBf16 || WSRC == kDenseF16;
  constexpr bool F16 = WSRC == kDenseF16 || WSRC == kPacked4F16;    // elements are IEEE binary16, not bf16
  constexpr bool W8 = WSRC == kPacked8;     // one byte per code: 64 bytes per row and step, w [N, K/4] words
  constexpr bool G32 = WSRC == kPacked4G32; // groups of 32: two scales and biases per row and step
  static_assert(!(W8 && NT == 4), "byte codes: the doubled code ring fits LDS up to 192-row weight tiles");
  static_assert(!(G32 && NT == 3), "groups of 32: 256- and 128-row weight tiles only");
  constexpr int CRB = W8 ? 64 : 32;         // bytes of codes per row and step
  constexpr int NC = W8 ? 4 : 2;            // code loads per wavefront and step (1 KB each)
  constexpr int kCodeSlot = W8 ? 64 * NT * 64 : kCodeBytes;
  constexpr int kWStage = 64 * NT * kRow;   // BN rows of 128 bytes
  constexpr int SBLK = G32 ? 4 : 8;         // steps per 16-byte block of a row's scales
  constexpr int BN = 64 * NT;               // weight rows per workgroup
  constexpr int MQ = 4 * NT;                // MFMAs per quarter step (16 of K)
  __shared__ __attribute__((aligned(16))) uint8_t x_lds[2 * kXBytes];
  __shared__ __attribute__((aligned(16))) uint8_t w_lds[2 * kWStage];
  uint8_t* const x_lds0 = x_lds;
  uint8_t* const x_lds1 = x_lds + kXBytes;
  uint8_t* const w_lds0 = w_lds;
  uint8_t* const w_lds1 = w_lds + kWStage;
  __shared__ __attribute__((aligned(16))) uint8_t c_lds[2 * kCodeSlot];
  __shared__ __attribute__((aligned(16))) uint8_t sb_lds[2 * kScaleBytes];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int tm, tn;
  if (p.bmt != 0) {
    // Workgroups go to the 8 XCDs round-robin, 32 at a time each: workgroup i is number (i / 8) % 32 of the
    // (i / 256)-th set that XCD i % 8 runs.  A set is a block of bmt x bnt tiles, so that the workgroups an XCD
    // runs together share rows of x (bnt of them each) and weight tiles (bmt each) through that XCD's L2.
    const int wg = (int)blockIdx.x;
    const int slot = (wg >> 3) & 31, blk = (wg >> 8) * 8 + (wg & 7);
    tm = (blk / p.nbn) * p.bmt + slot / p.bnt;
    tn = (blk % p.nbn) * p.bnt + slot % p.bnt;
    if (tm >= p.tiles_m || tn >= p.tiles_n) { return; }
  } else {
    const int tile = (int)blockIdx.x;
    const int band = tile / (8 * p.tiles_n);
    const int in_band = tile - band * (8 * p.tiles_n);
    const int band_h = (p.tiles_m - band * 8) < 8 ? (p.tiles_m - band * 8) : 8;
    tm = band * 8 + in_band % band_h;
    tn = in_band / band_h;
  }
  const int m0 = tm * BM, n0 = tn * BN;
  const int KT = p.K / BK;                  // whole steps.  Packed: a multiple of 8 (K % 512 == 0)
  const int tail_chunks = (p.K & (BK - 1)) >> 3;   // dense: 16-byte chunks of a row in the half step after them (0: none)

  // ---- x tile: 8 direct-to-LDS loads per wavefront and step.  Load i of wavefront w covers tile rows
  // (8w + i)*8 .. +8; lane l takes row l/8 and lands at LDS position l%8 of it.
  const uint8_t* xblk = reinterpret_cast<const uint8_t*>(p.x) + (size_t)m0 * p.K * 2;
  uint32_t a_off[8];
  uint32_t tail_ok = 0;                     // bit i: this lane's chunk of load i exists in a partial last step
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = (wave * 8 + i) * 8 + (lane >> 3);
    const int chunk = swz(row, lane & 7);
    const int rg = (m0 + row < p.M) ? row : (p.M - 1 - m0);
    a_off[i] = (uint32_t)rg * (uint32_t)p.K * 2u + (uint32_t)chunk * 16u;
    if (chunk < tail_chunks) { tail_ok |= 1u << i; }
  }
  auto issue_x = [&](int step, auto stage_c) {
    const uint8_t* src = xblk + (size_t)step * (BK * 2);
    const uint32_t dst = lds_addr(decltype(stage_c)::value ? x_lds1 : x_lds0) + wave * (64 * kRow);
#pragma unroll
    for (int i = 0; i < 8; ++i) { dma16(dst + i * (8 * kRow), src, a_off[i]); }
  };
  // ---- codes, scales, biases: wavefront w brings in those of rows 64w .. 64w+63 (nothing past BN rows) ----
  const bool dq_wave = wave * 64 < BN;      // wave-uniform
  // The wavefront's offsets inside the LDS arrays, held in scalar registers for the whole kernel (the empty asm
  // keeps the compiler from recomputing them from the thread index before every request).
  uint32_t wave_x = wave * (64 * kRow), wave_c = wave * (64 * CRB), wave_s = wave * (64 * 16), wave_wd = wave * (2 * NT * 8 * kRow);
  asm volatile("" : "+s"(wave_x), "+s"(wave_c), "+s"(wave_s), "+s"(wave_wd));
  uint32_t c_off[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    // a load covers 1 KB: 32 rows of 32 bytes (two lanes a row), or 16 rows of 64 bytes (four lanes a row)
    const int row = W8 ? wave * 64 + i * 16 + (lane >> 2) : wave * 64 + i * 32 + (lane >> 1);
    const int rg = (n0 + row < p.N) ? (n0 + row) : (p.N - 1);
    c_off[i] = W8 ? (uint32_t)rg * (uint32_t)p.K + (uint32_t)(lane & 3) * 16u
                  : (uint32_t)rg * (uint32_t)(p.K >> 1) + (uint32_t)(lane & 1) * 16u;
  }
  const uint8_t* wblk = reinterpret_cast<const uint8_t*>(p.w);
  // dense W tile: as the x tile; its BN rows are dealt out evenly, wavefront w brings in rows 16 NT w .. + 16 NT
  constexpr int NWL = 2 * NT;               // loads per wavefront and step
  uint32_t wd_off[NWL];
  uint32_t wtail_ok = 0;                    // as tail_ok, for the W loads
#pragma unroll
  for (int i = 0; i < NWL; ++i) {
    const int row = (wave * NWL + i) * 8 + (lane >> 3);
    const int chunk = swz(row, lane & 7);
    const int rg = (n0 + row < p.N) ? (n0 + row) : (p.N - 1);
    wd_off[i] = DENSE ? (uint32_t)rg * (uint32_t)p.K * 2u + (uint32_t)chunk * 16u : 0u;
    if (chunk < tail_chunks) { wtail_ok |= 1u << i; }
  }
  auto issue_wdense = [&](int step, auto stage_c) {
    const uint8_t* src = wblk + (size_t)step * (BK * 2);
    const uint32_t dst = lds_addr(decltype(stage_c)::value ? w_lds1 : w_lds0) + wave * (NWL * 8 * kRow);
#pragma unroll
    for (int i = 0; i < NWL; ++i) { dma16(dst + i * (8 * kRow), src, wd_off[i]); }
  };
  auto issue_codes = [&](int u) {
    if (!dq_wave) { return; }
    const uint8_t* src = wblk + (size_t)u * CRB;
    const uint32_t dst = lds_addr(c_lds) + (u & 1) * kCodeSlot + wave * (64 * CRB);
#pragma unroll
    for (int i = 0; i < NC; ++i) { dma16(dst + i * 1024, src, c_off[i]); }
  };
  const int qrow = tid;                     // the tile row this thread dequantizes
  const int qrg = (n0 + qrow < p.N) ? (n0 + qrow) : (p.N - 1);
  const int sb_row_bytes = G32 ? (p.K >> 4) : (p.K >> 5);     // K/32 or K/64 entries of 2 bytes
  const uint8_t* srow = reinterpret_cast<const uint8_t*>(p.scales) + (size_t)qrg * sb_row_bytes;
  const uint8_t* brow = reinterpret_cast<const uint8_t*>(p.biases) + (size_t)qrg * sb_row_bytes;
  const uint32_t sb_off = (uint32_t)qrg * (uint32_t)sb_row_bytes;   // the thread's row inside the scales / biases array
  int sb_due = SBLK < KT ? 0 : 0x7fffffff;  // the window in which the next block of scales and biases is requested
  auto issue_scales = [&](int blk) {
    if (!dq_wave) { return; }
    const uint32_t dst = lds_addr(sb_lds) + (blk & 1) * kScaleBytes + wave * (64 * 16);
    dma16(dst, srow + (size_t)blk * 16);
    dma16(dst + 256 * 16, brow + (size_t)blk * 16);
  };
  // ---- dequantization: the BN x 8 pieces of a step's weight tile (a piece = 8 values of a row = one 16-byte
  // store; 4-bit codes: one word of codes, byte codes: two) are dealt out evenly, thread t takes the WPT
  // consecutive pieces from t*WPT on (row-major: piece j of row r is 8r + j).  BN = 256: its own row; BN = 128:
  // half a row; BN = 192: six pieces that may straddle two rows.  d_row is the first row, d_w0 the first piece in it.
  constexpr int WPT = 2 * NT;
  constexpr int NCW = W8 ? 2 * WPT : WPT;   // 32-bit words of codes per thread and step
  const int d_row = (tid * WPT) >> 3, d_w0 = (tid * WPT) & 7;
  int b_dst[WPT];
#pragma unroll
  for (int j = 0; j < WPT; ++j) {
    const int row = d_row + ((d_w0 + j) >> 3), word = (d_w0 + j) & 7;
    b_dst[j] = row * kRow + swz(row, word) * 16;
  }
  // A thread's pieces lie in at most two (row, group) sets of scale and bias, A before piece `sw_at` and B from it
  // on.  Group 64: rows d_row and d_row + 1 (only the 192-row tile reaches B).  Groups of 32: the change is where
  // the position in the row passes a multiple of 4: A = (d_row, the half d_w0 lies in), B = the upper half of
  // d_row if d_w0 lies in the lower one, else the lower half of d_row + 1.
  const bool starts_upper = d_w0 >= 4;
  const int sw_at = G32 ? 4 - (d_w0 & 3) : 8 - d_w0;
  constexpr bool TWO_SETS = NT == 3 || (G32 && NT == 4);   // the thread's pieces of a step can lie in two sets
  // ---- multiplier side ----
  const int wm = wave >> 1, wn = wave & 1;
  floatx16 acc[NT][4];   // [jt: 32 weight rows][it: 32 x rows]
#pragma unroll
  for (int jt = 0; jt < NT; ++jt) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
#pragma unroll
      for (int e = 0; e < 16; ++e) { acc[jt][it][e] = 0.0f; }
    }
  }
  const int frow = lane & 31;      // row of a 32-row operand fragment
  const int fkh = lane >> 5;       // which 8 of the 16 k
  int w_rd[NT], x_rd[4];           // stage-relative operand rows
#pragma unroll
  for (int jt = 0; jt < NT; ++jt) { w_rd[jt] = (wn * (BN / 2) + jt * 32 + frow) * kRow; }
#pragma unroll
  for (int it = 0; it < 4; ++it) { x_rd[it] = (wm * 128 + it * 32 + frow) * kRow; }
  const int f_sw = (frow >> 1) & 7;   // the fragment offsets are multiples of 16 rows: same swizzle for all

  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  using Yes = std::true_type;
  using No = std::false_type;

  auto mfma = [](const bf16x8& a, const bf16x8& b, const floatx16& c) {
    if constexpr (F16) {
      typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
      return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
    } else {
      return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
  };

  // ---- the pipeline.  A step's barrier stands at its 3/4 point, after the MFMAs of quarters 0..2: by then a
  // wavefront has every fragment of the step in registers and has waited for its own loads, so behind the barrier
  // the step's stage may be overwritten and the other stage (step s+1: x loaded, W loaded or dequantized) may be
  // read.  Quarter 3's MFMAs then cover the first fragment reads of step s+1, and the work of the window that
  // lasts until the next barrier starts under them:
  //   load requests  x(s+2) [8]; packed: codes(s+3) [2], on steps 8b the scales and biases of block b+1 [2];
  //                  dense: W(s+2) [2 NT] -- one request every second MFMA, all landed at the next barrier;
  //   packed         the dequantization of W(s+2) into the step's own stage, a few instructions per MFMA.
  // The state of both (fragments, codes, the piece in work) lives across steps.
  //
  // What a slot may hold.  With one wavefront per SIMD the instructions between two MFMAs issue in that MFMA's
  // shadow only up to a point: measured on this part (a loop of v_mfma_f32_32x32x16_bf16 with n other instructions
  // after each, four wavefronts), the MFMA's 32 cycles hold up to 4 further instructions of any kind at +0.5 cycles
  // each; the fifth and sixth cost 8 cycles each (4 vector instructions + 1 LDS read: 41 against 37), s_nop and
  // s_waitcnt are free, a 16-byte LDS store of a wavefront occupies the LDS write path for 16-18 cycles, and a
  // direct-to-LDS load every second slot is free while one in every slot doubles the slot (the same write path).
  // So the work of a window is cut into single instructions (ops) and dealt out so that no slot holds more than
  // 4: a fragment read counts 1, a load request 2 (the M0 write and the load; its s_nop is free), and the ops of
  // the dequantization fill what is left, in order.
  constexpr int NLOADS = DENSE ? 8 + 2 * NT : 9 + NC;           // packed: x, codes, one pair of scales and biases
  constexpr int NSLOT = 4 * MQ;                                // slots of a window (barrier to barrier)
  constexpr int LSTRIDE = 2;                                   // a load request every LSTRIDE-th slot, from slot 1 on
  // ---- the ops of a window's dequantization (of W(s+2)): NP ops that fetch the thread's codes, scales and biases
  // from the rings and convert them, then OPW ops per piece:
  //   4-bit   0 choose set A or B | 1 t = c >> 8 | 2-5 the four nibble pairs in place: c & 000f000f (q0,q4),
  //           c & 00f000f0 (q1,q5), t & 000f000f (q2,q6), t & 00f000f0 (q3,q7) | 6-13 one v_fma_mix_f32 per value |
  //           14-17 pack to bf16 pairs | 18 store
  //   bytes   0 choose | 1-2 t0 = c0 >> 8, t1 = c1 >> 8 | 3-6 c0, t0, c1, t1 & 00ff00ff | 7-14 | 15-18 | 19
  // A masked code in one half of a register, read as binary16, is the denormal q * 2^-24 (16 q * 2^-24 for the
  // nibbles left at bits 4-7), which v_fma_mix_f32 widens exactly: fma(q 2^-24, s 2^24, b) has the same exact
  // product and sum as fma(s, q, b), so the rounded weight has the same bits
  // (gpu-kernels/metal/quant/affine_qmm_steel.metal:78-96) for every |s| < 2^104 -- with 18 instructions per 8
  // weights instead of 24 (convert + fma per value).
  constexpr int RDW = NCW % 4 == 0 ? 4 : 2;                    // words per LDS read of the thread's codes (their alignment)
  constexpr int NRD = NCW / RDW;
  constexpr int NP = DENSE ? 0 : NRD + 4;                      // + raw reads A, raw reads B, convert A, convert B
  constexpr int OPW = W8 ? 20 : 19;
  constexpr int NOPS = DENSE ? 0 : NP + WPT * OPW;
  struct Plan {
    int load_of[NSLOT];        // the request made in a slot, or -1
    int op_begin[NSLOT + 1];   // the slot's ops are [op_begin[g], op_begin[g + 1])
  };
  constexpr auto make_plan = []() constexpr {
    Plan pl{};
    int next_load = 0;
    for (int g = 0; g < NSLOT; ++g) {
      pl.load_of[g] = (g % LSTRIDE == LSTRIDE - 1 && next_load < NLOADS) ? next_load++ : -1;
    }
    int u = 0;
    for (int g = 0; g < NSLOT; ++g) {
      pl.op_begin[g] = u;
      int room = 4 - ((g % MQ) < 4 + NT ? 1 : 0) - (pl.load_of[g] >= 0 ? 2 : 0);
      while (u < NOPS) {
        int wgt = 1;
        if (u < NP) {
          const int k = u - NRD;                               // 0, 1 raw reads; 2, 3 conversions
          if (k == 0) { wgt = 2; }
          if (k == 1) { wgt = (NT == 3) ? 2 : 0; }
          if (k == 2) { wgt = (W8 ? 2 : 3) + (G32 ? 1 : 0); }
          if (k == 3) { wgt = TWO_SETS ? (W8 ? 2 : 3) + (G32 ? 1 : 0) : 0; }
        } else {
          const int pc = (u - NP) / OPW, op = (u - NP) % OPW;
          if (op == 0) { wgt = (NT == 3 && pc >= 2) ? (W8 ? 2 : 3) : 0; }
        }
        if (wgt > room && room < 4) { break; }                 // does not fit beside what the slot already holds
        room -= wgt;
        ++u;
        if (room <= 0) { break; }
      }
    }
    pl.op_begin[NSLOT] = NOPS;                                 // what did not fit goes to the last slot
    return pl;
  };
  static constexpr Plan plan = make_plan();

  bf16x8 wf[2][NT], xf[2][4];                          // operand fragments of the current / the next quarter
  struct RowSet { float s24, s20, b; };                // scale * 2^24, scale * 2^20, bias
  RowSet set_a{0.0f, 0.0f, 0.0f}, set_b{0.0f, 0.0f, 0.0f}, cur{0.0f, 0.0f, 0.0f};
  uint32_t raw_a[2] = {0, 0}, raw_b[2] = {0, 0};       // scale and bias as read from the ring
  uint32_t cw[NCW];                                    // the thread's codes of the step being dequantized
#pragma unroll
  for (int j = 0; j < NCW; ++j) { cw[j] = 0; }
  uint32_t t0 = 0, t1 = 0, mk[4] = {0, 0, 0, 0};
  float v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  uint4 o = make_uint4(0, 0, 0, 0);
  auto frag = [&](const uint8_t* xb, const uint8_t* wb, int buf, int ks, int idx) {   // idx: 0 = w0, 1..4 = x0..x3, 5.. = w1..
    const int c = ((2 * ks + fkh) ^ f_sw) * 16;
    if (idx == 0) {
      wf[buf][0] = *reinterpret_cast<const bf16x8*>(wb + w_rd[0] + c);
    } else if (idx <= 4) {
      xf[buf][idx - 1] = *reinterpret_cast<const bf16x8*>(xb + x_rd[idx - 1] + c);
    } else {
      wf[buf][idx - 4] = *reinterpret_cast<const bf16x8*>(wb + w_rd[idx - 4] + c);
    }
  };
  // Single instructions of the dequantization, as volatile asm so that each stays in the slot it is written in (the
  // scheduling barriers pin machine instructions, but the compiler would still sink plain arithmetic to its first
  // use before they apply).  fma(binary16 half HI of `code` widened, scale, bias):
  auto mix = [](auto hi_c, uint32_t code, float scale, float bias) {
    float r;
    if constexpr (decltype(hi_c)::value) {
      asm volatile("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(code), "v"(scale), "v"(bias));
    } else {
      asm volatile("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(code), "v"(scale), "v"(bias));
    }
    return r;
  };
  auto shr8 = [](uint32_t c) { uint32_t r; asm volatile("v_lshrrev_b32 %0, 8, %1" : "=v"(r) : "v"(c)); return r; };
  auto andm = [](uint32_t c, uint32_t m) { uint32_t r; asm volatile("v_and_b32 %0, %1, %2" : "=v"(r) : "s"(m), "v"(c)); return r; };
  auto pk2 = [](float a, float b) {
    uint32_t r;
    if constexpr (F16) { asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b)); }
    else { asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b)); }
    return r;
  };
  auto pick = [](float a, float b, uint64_t second) {   // second ? b : a, per lane
    float r;
    asm volatile("v_cndmask_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "s"(second));
    return r;
  };
  uint32_t mask_lo = W8 ? 0x00ff00ffu : 0x000f000fu, mask_hi = 0x00f000f0u;
  asm volatile("" : "+s"(mask_lo), "+s"(mask_hi));       // in scalar registers: no literal in every instruction
  auto to_set = [](uint32_t sbits, uint32_t bbits) {
    const float sc = elt_bits_to_f32<F16>(sbits);
    return RowSet{sc * 16777216.0f, sc * 1048576.0f, elt_bits_to_f32<F16>(bbits)};
  };
  // Op U of the window that dequantizes W(u) into the stage `nb`.
  auto dq_op = [&](auto uc, int u, uint8_t* nb) {
    constexpr int U = decltype(uc)::value;
    if constexpr (U < NRD) {
      const uint8_t* cp = c_lds + (u & 1) * kCodeSlot + tid * (NCW * 4) + U * (RDW * 4);
      if constexpr (RDW == 4) {
        const uint4 c4 = *reinterpret_cast<const uint4*>(cp);
        cw[4 * U] = c4.x; cw[4 * U + 1] = c4.y; cw[4 * U + 2] = c4.z; cw[4 * U + 3] = c4.w;
      } else {
        const uint2 c2 = *reinterpret_cast<const uint2*>(cp);
        cw[2 * U] = c2.x; cw[2 * U + 1] = c2.y;
      }
    } else if constexpr (U < NP) {
      constexpr int k = U - NRD;
      // group 64: 2-byte entries, 8 steps per 16-byte block of a row; groups of 32: a dword of two entries per step
      const uint8_t* sb = G32 ? sb_lds + ((u >> 2) & 1) * kScaleBytes + d_row * 16 + (u & 3) * 4
                              : sb_lds + ((u >> 3) & 1) * kScaleBytes + d_row * 16 + (u & 7) * 2;
      if constexpr (k == 0) {
        if constexpr (G32) {
          raw_a[0] = *reinterpret_cast<const uint32_t*>(sb); raw_a[1] = *reinterpret_cast<const uint32_t*>(sb + 256 * 16);
        } else {
          raw_a[0] = *reinterpret_cast<const uint16_t*>(sb); raw_a[1] = *reinterpret_cast<const uint16_t*>(sb + 256 * 16);
        }
      } else if constexpr (k == 1) {
        if constexpr (NT == 3) {                               // the next row's
          if constexpr (G32) {
            raw_b[0] = *reinterpret_cast<const uint32_t*>(sb + 16); raw_b[1] = *reinterpret_cast<const uint32_t*>(sb + 256 * 16 + 16);
          } else {
            raw_b[0] = *reinterpret_cast<const uint16_t*>(sb + 16); raw_b[1] = *reinterpret_cast<const uint16_t*>(sb + 256 * 16 + 16);
          }
        }
      } else if constexpr (k == 2) {
        if constexpr (G32) {
          const uint32_t sh = (NT == 4 || !starts_upper) ? 0u : 16u;   // NT == 4: set A is the lower half of the row's step
          if constexpr (NT == 4) { set_a = to_set(raw_a[0] & 0xffffu, raw_a[1] & 0xffffu); }
          else { set_a = to_set((raw_a[0] >> sh) & 0xffffu, (raw_a[1] >> sh) & 0xffffu); }
        } else {
          set_a = to_set(raw_a[0], raw_a[1]);
        }
      } else {
        if constexpr (G32 && NT == 4) { set_b = to_set(raw_a[0] >> 16, raw_a[1] >> 16); }
        else if constexpr (G32 && NT == 3) {
          // the lower half of the next row, or the upper half of this one: choose the bits, convert once
          const uint32_t sbits = starts_upper ? (raw_b[0] & 0xffffu) : (raw_a[0] >> 16);
          const uint32_t bbits = starts_upper ? (raw_b[1] & 0xffffu) : (raw_a[1] >> 16);
          set_b = to_set(sbits, bbits);
        } else if constexpr (NT == 3) { set_b = to_set(raw_b[0], raw_b[1]); }
      }
    } else {
      constexpr int PC = (U - NP) / OPW, OP = (U - NP) % OPW;
      if constexpr (OP == 0) {
        if constexpr (NT == 3 && PC >= 2) {
          const uint64_t second = __builtin_amdgcn_ballot_w64(PC >= sw_at);
          cur.s24 = pick(set_a.s24, set_b.s24, second);
          if constexpr (!W8) { cur.s20 = pick(set_a.s20, set_b.s20, second); }
          cur.b = pick(set_a.b, set_b.b, second);
        } else if constexpr (G32 && NT == 4 && PC == 4) {
          cur = set_b;                                         // no instruction: the second half of the row's step
        } else if constexpr (PC == 0) {
          cur = set_a;
        }
      } else if constexpr (W8) {
        const uint32_t c0 = cw[2 * PC], c1 = cw[2 * PC + 1];   // q0 q1 q2 q3 | q4 q5 q6 q7, a byte each
        if constexpr (OP == 1) { t0 = shr8(c0); }
        if constexpr (OP == 2) { t1 = shr8(c1); }
        if constexpr (OP == 3) { mk[0] = andm(c0, mask_lo); }  // q0, q2
        if constexpr (OP == 4) { mk[1] = andm(t0, mask_lo); }  // q1, q3
        if constexpr (OP == 5) { mk[2] = andm(c1, mask_lo); }  // q4, q6
        if constexpr (OP == 6) { mk[3] = andm(t1, mask_lo); }  // q5, q7
        if constexpr (OP == 7) { v[0] = mix(No(), mk[0], cur.s24, cur.b); }
        if constexpr (OP == 8) { v[1] = mix(No(), mk[1], cur.s24, cur.b); }
        if constexpr (OP == 9) { v[2] = mix(Yes(), mk[0], cur.s24, cur.b); }
        if constexpr (OP == 10) { v[3] = mix(Yes(), mk[1], cur.s24, cur.b); }
        if constexpr (OP == 11) { v[4] = mix(No(), mk[2], cur.s24, cur.b); }
        if constexpr (OP == 12) { v[5] = mix(No(), mk[3], cur.s24, cur.b); }
        if constexpr (OP == 13) { v[6] = mix(Yes(), mk[2], cur.s24, cur.b); }
        if constexpr (OP == 14) { v[7] = mix(Yes(), mk[3], cur.s24, cur.b); }
        if constexpr (OP >= 15 && OP <= 18) {
          const uint32_t pk = pk2(v[2 * (OP - 15)], v[2 * (OP - 15) + 1]);
          if constexpr (OP == 15) { o.x = pk; } else if constexpr (OP == 16) { o.y = pk; }
          else if constexpr (OP == 17) { o.z = pk; } else { o.w = pk; }
        }
        if constexpr (OP == 19) { *reinterpret_cast<uint4*>(nb + b_dst[PC]) = o; }
      } else {
        const uint32_t c = cw[PC];
        if constexpr (OP == 1) { t0 = shr8(c); }
        if constexpr (OP == 2) { mk[0] = andm(c, mask_lo); }   // q0, q4
        if constexpr (OP == 3) { mk[1] = andm(c, mask_hi); }   // 16 q1, 16 q5
        if constexpr (OP == 4) { mk[2] = andm(t0, mask_lo); }  // q2, q6
        if constexpr (OP == 5) { mk[3] = andm(t0, mask_hi); }  // 16 q3, 16 q7
        if constexpr (OP == 6) { v[0] = mix(No(), mk[0], cur.s24, cur.b); }
        if constexpr (OP == 7) { v[1] = mix(No(), mk[1], cur.s20, cur.b); }
        if constexpr (OP == 8) { v[2] = mix(No(), mk[2], cur.s24, cur.b); }
        if constexpr (OP == 9) { v[3] = mix(No(), mk[3], cur.s20, cur.b); }
        if constexpr (OP == 10) { v[4] = mix(Yes(), mk[0], cur.s24, cur.b); }
        if constexpr (OP == 11) { v[5] = mix(Yes(), mk[1], cur.s20, cur.b); }
        if constexpr (OP == 12) { v[6] = mix(Yes(), mk[2], cur.s24, cur.b); }
        if constexpr (OP == 13) { v[7] = mix(Yes(), mk[3], cur.s20, cur.b); }
        if constexpr (OP >= 14 && OP <= 17) {
          const uint32_t pk = pk2(v[2 * (OP - 14)], v[2 * (OP - 14) + 1]);
          if constexpr (OP == 14) { o.x = pk; } else if constexpr (OP == 15) { o.y = pk; }
          else if constexpr (OP == 16) { o.z = pk; } else { o.w = pk; }
        }
        if constexpr (OP == 18) { *reinterpret_cast<uint4*>(nb + b_dst[PC]) = o; }
      }
    }
  };
  // Request I of the window that opens behind the barrier of step `win`: x(win+2) goes to the stage of step win.
  auto window_load = [&](auto ic, int win, auto stage_c) {
    constexpr int I = decltype(ic)::value;
    constexpr int STG = decltype(stage_c)::value;
    const int step_to = win + 2;
    const uint32_t xdst = lds_addr(STG ? x_lds1 : x_lds0) + wave_x;
    const uint8_t* xsrc = xblk + (size_t)step_to * (BK * 2);
    if constexpr (DENSE) {
      if constexpr (I < NWL) {
        const uint32_t wdst = lds_addr(STG ? w_lds1 : w_lds0) + wave_wd;
        dma16(wdst + I * (8 * kRow), wblk + (size_t)step_to * (BK * 2), wd_off[I]);
      } else {
        dma16(xdst + (I - NWL) * (8 * kRow), xsrc, a_off[I - NWL]);
      }
    } else {
      if constexpr (I < 8) {
        dma16(xdst + I * (8 * kRow), xsrc, a_off[I]);
      } else if constexpr (I < 8 + NC) {
        // codes(win+3) into the slot codes(win+1) have left.  Past the last step the last step's codes are read
        // again (nobody uses them) rather than branching round the request; 4-bit codes: every wavefront brings in
        // 64 rows of the 256-row slot, tile rows or not.
        const int cstep = win + 3 < KT ? win + 3 : KT - 1;
        if (!W8 || dq_wave) {
          dma16(lds_addr(c_lds) + (1 - STG) * kCodeSlot + wave_c + (I - 8) * 1024, wblk + (size_t)cstep * CRB, c_off[I - 8]);
        }
      } else {
        // scales and biases of the next block of steps, both in this slot, when the window's step starts a block
        if (win == sb_due) {
          const int blk = (win >> (G32 ? 2 : 3)) + 1;
          const uint32_t sdst = lds_addr(sb_lds) + (blk & 1) * kScaleBytes + wave_s;
          dma16(sdst, reinterpret_cast<const uint8_t*>(p.scales) + (size_t)blk * 16, sb_off);
          dma16(sdst + 256 * 16, reinterpret_cast<const uint8_t*>(p.biases) + (size_t)blk * 16, sb_off);
          sb_due = win + 2 * SBLK < KT ? win + SBLK : 0x7fffffff;
        }
      }
    }
  };
  // Slot G of the window behind the barrier of step `win`: its request, its ops (they dequantize W(win+2) into `nb`).
  auto window_slot = [&](auto gc, int win, auto stage_c, uint8_t* nb) {
    constexpr int G = decltype(gc)::value;
    if constexpr (plan.load_of[G] >= 0) { window_load(std::integral_constant<int, plan.load_of[G]>(), win, stage_c); }
    if constexpr (!DENSE) {
      static_for<plan.op_begin[G], plan.op_begin[G + 1]>([&](auto uc) { dq_op(uc, win + 2, nb); });
    }
  };
  // Step s on stage ST.  m1: a step s+1 exists, m2: a step s+2 exists (std::true_type / std::false_type).
  auto pstep = [&](auto stage_c, auto m1, auto m2, int s) {
    constexpr int ST = decltype(stage_c)::value;
    using Nx = std::integral_constant<int, 1 - ST>;
    const uint8_t* xb = ST ? x_lds1 : x_lds0;
    const uint8_t* wb = ST ? w_lds1 : w_lds0;
    const uint8_t* nxb = ST ? x_lds0 : x_lds1;
    uint8_t* nwb = ST ? w_lds0 : w_lds1;
    uint8_t* ownb = ST ? w_lds1 : w_lds0;
    static_for<0, 4>([&](auto qc) {
      constexpr int Q = decltype(qc)::value;
      constexpr int B = Q & 1;
      static_for<0, MQ>([&](auto jc) {
        constexpr int J = decltype(jc)::value;
        constexpr int JT = J >> 2, IT = J & 3;
        acc[JT][IT] = mfma(wf[B][JT], xf[B][IT], acc[JT][IT]);
        constexpr int GB = Q == 3 ? J : MQ * (Q + 1) + J;    // slot counted from the previous barrier
        if constexpr (Q == 3) { when(m2, [&] { window_slot(std::integral_constant<int, GB>(), s, stage_c, ownb); }); }
        else { when(m1, [&] { window_slot(std::integral_constant<int, GB>(), s - 1, Nx(), nwb); }); }
        // the next quarter's fragments, one read after every MFMA until they are all requested
        if constexpr (J < 4 + NT) {
          if constexpr (Q < 3) { frag(xb, wb, 1 - B, Q + 1, J); }
          else { when(m1, [&] { frag(nxb, nwb, 0, 0, J); }); }
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (Q == 2) {
        when(m1, [&] {
          asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
          wg_barrier();
        });
      }
    });
  };

  // `nq` quarter steps (16 of K each) on the tiles in stage 0, nothing overlapped: for the short extra pieces of K
  // (a dense half step, the adapter's rank).
  auto plain_quarters = [&](int nq) {
    for (int q = 0; q < nq; ++q) {
#pragma unroll
      for (int i = 0; i < 4 + NT; ++i) { frag(x_lds0, w_lds0, 0, q, i); }
#pragma unroll
      for (int j = 0; j < MQ; ++j) { acc[j >> 2][j & 3] = mfma(wf[0][j >> 2], xf[0][j & 3], acc[j >> 2][j & 3]); }
    }
  };

  if (KT > 0) {
    // Steps alternate between the two stages and the last step runs on stage 1, so that the written-out last steps
    // are the same for every K: an odd number of steps (dense weights only) starts on stage 1, as if a step on
    // stage 0 had gone before.
    const bool odd = DENSE && (KT & 1) != 0;
    // ---- prologue: the first step's stage complete (x(0); W(0) loaded or dequantized), the part of step 1's
    // window that a quarter 3 before step 0 would have done, the first fragments ----
    auto prologue = [&](auto first_c) {
      constexpr int P0 = decltype(first_c)::value;
      using Other = std::integral_constant<int, 1 - P0>;
      if constexpr (DENSE) {
        issue_wdense(0, first_c);
        issue_x(0, first_c);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        wg_barrier();
      } else {
        issue_scales(0);
        issue_codes(0);
        issue_codes(1);
        issue_x(0, first_c);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        wg_barrier();                           // the codes and scales a thread reads were brought in by any wavefront
        static_for<0, NOPS>([&](auto uc) { dq_op(uc, 0, w_lds0); });
        static_for<0, plan.op_begin[MQ]>([&](auto uc) { dq_op(uc, 1, w_lds1); });
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wg_barrier();
      }
      if (KT > 1) {
        static_for<0, MQ>([&](auto gc) {
          if constexpr (plan.load_of[decltype(gc)::value] >= 0) {
            window_load(std::integral_constant<int, plan.load_of[decltype(gc)::value]>(), -1, Other());
          }
        });
      }
#pragma unroll
      for (int i = 0; i < 4 + NT; ++i) { frag(P0 ? x_lds1 : x_lds0, P0 ? w_lds1 : w_lds0, 0, 0, i); }
    };
    if constexpr (DENSE) {
      if (odd) { prologue(S1()); } else { prologue(S0()); }
    } else {
      prologue(S0());
    }

    // ---- K loop.  No condition surrounds the arithmetic inside a step: the last two steps are written out.  With
    // an odd number of steps the count runs from -1 and the step on stage 0 that would be step -1 is skipped. ----
    int s = DENSE ? -(KT & 1) : 0;
    if constexpr (DENSE) { asm volatile("" : "+s"(s)); }   // stays in a scalar register (it feeds the request addresses)
    for (; s + 3 < KT; s += 2) {
      if (s >= 0) { pstep(S0(), Yes(), Yes(), s); }
      pstep(S1(), Yes(), Yes(), s + 1);
    }
    if (s >= 0) { pstep(S0(), Yes(), No(), s); }
    pstep(S1(), No(), No(), s + 1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the repeated last requests for codes, before LDS is reused
  }

  if constexpr (DENSE) {
    if (tail_chunks != 0) {
      // the last 32 values of K: half rows into stage 0 (only the lanes whose chunk exists), two quarter steps
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      wg_barrier();                                    // everyone done with stage 0
      const uint8_t* xsrc = xblk + (size_t)KT * (BK * 2);
      const uint8_t* wsrc = wblk + (size_t)KT * (BK * 2);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if ((tail_ok >> i) & 1u) { dma16(lds_addr(x_lds0) + wave * (64 * kRow) + i * (8 * kRow), xsrc, a_off[i]); }
      }
#pragma unroll
      for (int i = 0; i < NWL; ++i) {
        if ((wtail_ok >> i) & 1u) { dma16(lds_addr(w_lds0) + wave * (NWL * 8 * kRow) + i * (8 * kRow), wsrc, wd_off[i]); }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      wg_barrier();
      plain_quarters(tail_chunks >> 1);
    }
  }

  if (LORA) {
    // r more values of K from t[M,r] and B[N,r], dense, through stage 0
    // (gpu-kernels/metal/gemm/dense_gemm_mma.metal:297-348).
    const int steps = (p.r + BK - 1) / BK;
    for (int st = 0; st < steps; ++st) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      wg_barrier();                                    // everyone done with stage 0
      const int kleft = p.r - st * BK;                 // >= 8, a multiple of 8
      const int chunks = kleft >= BK ? 8 : (kleft >> 3);
      // An odd number of 8-value pieces (a rank of 8 mod 16): the quarter step's other half is zeros, in both tiles
      // (what lies in the stage from the K loop may be anything, a NaN pattern included).
      const int zero_chunk = (chunks & 1) ? chunks : -1;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int row = (wave * 8 + i) * 8 + (lane >> 3);
        const int chunk = swz(row, lane & 7);
        const int rg = (m0 + row < p.M) ? (m0 + row) : (p.M - 1);
        if (chunk < chunks) {
          dma16(lds_addr(x_lds0) + wave * (64 * kRow) + i * (8 * kRow),
                reinterpret_cast<const uint8_t*>(p.lora_t + (size_t)rg * p.r + st * BK + chunk * 8));
        } else if (chunk == zero_chunk) {
          *reinterpret_cast<uint4*>(x_lds0 + wave * (64 * kRow) + i * (8 * kRow) + lane * 16) = make_uint4(0, 0, 0, 0);
        }
      }
      if (dq_wave) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int row = (wave * 8 + i) * 8 + (lane >> 3);
          const int chunk = swz(row, lane & 7);
          const int rg = (n0 + row < p.N) ? (n0 + row) : (p.N - 1);
          if (chunk < chunks) {
            dma16(lds_addr(w_lds0) + wave * (64 * kRow) + i * (8 * kRow),
                  reinterpret_cast<const uint8_t*>(p.lora_b + (size_t)rg * p.r + st * BK + chunk * 8));
          } else if (chunk == zero_chunk) {
            *reinterpret_cast<uint4*>(w_lds0 + wave * (64 * kRow) + i * (8 * kRow) + lane * 16) = make_uint4(0, 0, 0, 0);
          }
        }
      }
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      wg_barrier();                                    // tiles ready
      plain_quarters((chunks + 1) >> 1);
    }
  }

  // ---- store: lane holds, for x row m = lane%32 of each it, 4 consecutive n per register quad ----
  if (!LORA && p.gate_act) {                           // never together with an adapter
    // A register quad is (gate, up, gate, up) of features n/2 and n/2 + 1 (n is a multiple of 4):
    // the activation is register-local and a quad becomes one dword of two bf16.
    const bool pair_ok = ((p.out_stride | p.out_off) & 1) == 0;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int m = m0 + wm * 128 + it * 32 + frow;
      if (m >= p.M) { continue; }
      uint16_t* yrow = p.y + (size_t)m * p.out_stride + p.out_off;
#pragma unroll
      for (int jt = 0; jt < NT; ++jt) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int n = n0 + wn * (BN / 2) + jt * 32 + rq * 8 + fkh * 4;
          if (n >= p.N) { continue; }
          const float f0 = gated_f32(p.gate_act, acc[jt][it][rq * 4 + 0], acc[jt][it][rq * 4 + 1]);
          const float f1 = gated_f32(p.gate_act, acc[jt][it][rq * 4 + 2], acc[jt][it][rq * 4 + 3]);
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
  if ((p.N & 7) == 0 && (reinterpret_cast<uintptr_t>(p.y) & 15) == 0) {
    // Rows of y in whole 16-byte pieces: each wavefront turns its block round in an LDS region of its own, 32 x
    // rows at a time -- written as the accumulators lie (lane = x row, 4 consecutive n per register quad), read back
    // along the rows -- so that a store instruction covers runs of 64 NT bytes per row instead of 16-byte pieces of
    // 32 rows.  The stages are free by now; one barrier, since other wavefronts may still be reading them.
    constexpr int kRowBytes = 64 * NT;             // the wavefront's BN/2 columns
    constexpr int kPitch = kRowBytes + 16;
    constexpr int LPR = kRowBytes / 16;            // 16-byte pieces per row
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    wg_barrier();
    uint8_t* region = wave == 0 ? x_lds0 : wave == 1 ? x_lds1 : wave == 2 ? w_lds0 : w_lds1;
    const int ncol0 = n0 + wn * (BN / 2);
#pragma unroll
    for (int it = 0; it < 4; ++it) {
#pragma unroll
      for (int jt = 0; jt < NT; ++jt) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          uint2 o;
          o.x = pack_elt2<F16>(acc[jt][it][rq * 4 + 0], acc[jt][it][rq * 4 + 1]);
          o.y = pack_elt2<F16>(acc[jt][it][rq * 4 + 2], acc[jt][it][rq * 4 + 3]);
          *reinterpret_cast<uint2*>(region + frow * kPitch + (jt * 32 + rq * 8 + fkh * 4) * 2) = o;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int idx0 = 0; idx0 < 32 * LPR; idx0 += 64) {
        const int idx = idx0 + lane;
        const int r = idx / LPR, c = idx - r * LPR;
        const int m = m0 + wm * 128 + it * 32 + r;
        const int n = ncol0 + c * 8;
        if (idx < 32 * LPR && m < p.M && n < p.N) {
          const uint4 q = *reinterpret_cast<const uint4*>(region + r * kPitch + c * 16);
          *reinterpret_cast<uint4*>(p.y + (size_t)m * p.N + n) = q;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the region is rewritten by the next block
    }
    return;
  }
  const bool vec_ok = (p.N & 3) == 0;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int m = m0 + wm * 128 + it * 32 + frow;
    if (m >= p.M) { continue; }
    uint16_t* yrow = p.y + (size_t)m * p.N;
#pragma unroll
    for (int jt = 0; jt < NT; ++jt) {
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int n = n0 + wn * (BN / 2) + jt * 32 + rq * 8 + fkh * 4;
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

bool qmm_big_supports(const GemmArgs& a)
{
  // K in blocks of 8 steps (the scale ring) with 16-byte aligned rows of scales; 32-bit offsets
  // inside the pack and inside a band of x.
  if (a.K % 512 != 0 || a.M < 1 || a.N < 1) { return false; }
  if (a.gate_act != 0 && (a.lora_t != nullptr || (a.N & 1) != 0)) { return false; }
  if ((reinterpret_cast<uintptr_t>(a.scales) & 15) != 0 || (reinterpret_cast<uintptr_t>(a.biases) & 15) != 0) { return false; }
  if ((double)a.N * (double)a.K / (a.bits == 8 ? 1.0 : 2.0) >= 4.0e9 || (double)BM * (double)a.K * 2.0 >= 4.0e9) { return false; }
  if (a.lora_t != nullptr && (a.r < 8 || a.r % 8 != 0)) { return false; }
  // the other code formats come without the adapter path; formats and element types are not combined
  const int modes = (a.bits == 8) + (a.group == 32) + (a.f16 ? 1 : 0);
  if (modes > 1 || (modes == 1 && !a.f16 && a.lora_t != nullptr)) { return false; }
  if ((a.bits != 4 && a.bits != 8) || (a.group != 64 && a.group != 32)) { return false; }
  return true;
}

// Tile width by a small cost model: workgroups run one per CU, so a launch takes ceil(tiles / CUs)
// rounds, and a round's time grows with the tile width (the MFMA work) over the width's efficiency
// (measured with whole rounds: 256 wide 1.02, 192 wide 0.98, 128 wide 0.94 PFLOP/s).  4096 -> 12288 at
// M = 2048: 384 tiles of 256 are one and a half rounds of 256 CUs, 512 tiles of 192 are two;
// N = 4096 at M = 2048 is exactly one round of 128-wide tiles.
int qmm_big_tile_n(int N, int M, int cu_count, int max_width, bool with_192)
{
  const int cus = cu_count > 0 ? cu_count : 256;
  const long tm = (M + BM - 1) / BM;
  const int widths[3] = {256, 192, 128};
  const double eff[3] = {1.0, 0.95, 0.90};
  const int first = max_width >= 256 ? 0 : 1;          // byte codes: tiles up to 192 rows of weights
  int best = widths[first];
  double best_cost = 0.0;
  for (int i = first; i < 3; ++i) {
    if (widths[i] == 192 && !with_192) { continue; }     // groups of 32: 256 and 128 wide only
    const long tiles = tm * ((N + widths[i] - 1) / widths[i]);
    const long rounds = (tiles + cus - 1) / cus;
    const double cost = (double)rounds * (double)widths[i] / eff[i];
    if (i == first || cost < best_cost) { best = widths[i]; best_cost = cost; }
  }
  return best;
}

namespace {

// Tile order and grid size.  From two full rounds of the chip on: blocks of 32 tiles per XCD, in the shape that
// leaves the fewest empty places (then the squarest); below that, bands of 8 rows of tiles.
unsigned plan_tile_order(BigParams& p)
{
  p.bmt = 0; p.bnt = 0; p.nbn = 0;
  const long tiles = (long)p.tiles_m * p.tiles_n;
  if (tiles < 512) { return (unsigned)tiles; }
  const int shapes[6][2] = {{4, 8}, {8, 4}, {2, 16}, {16, 2}, {1, 32}, {32, 1}};
  long best_sets = 0;
  for (int i = 0; i < 6; ++i) {
    const long nbm = (p.tiles_m + shapes[i][0] - 1) / shapes[i][0], nbn = (p.tiles_n + shapes[i][1] - 1) / shapes[i][1];
    const long sets = (nbm * nbn + 7) / 8;               // rounds of 8 XCDs x 32 workgroups
    if (i == 0 || sets < best_sets) { best_sets = sets; p.bmt = shapes[i][0]; p.bnt = shapes[i][1]; p.nbn = (int)nbn; }
  }
  return (unsigned)(best_sets * 256);
}

}  // namespace

hipError_t launch_qmm_big(hipStream_t st, const GemmArgs& a, int tile_n)
{
  const int widest = a.bits == 8 ? 192 : 256;
  const bool with_192 = a.group != 32;
  const int bn = tile_n == 128 || (tile_n == 192 && with_192) || (tile_n == 256 && widest == 256)
                     ? tile_n : qmm_big_tile_n(a.N, a.M, a.cu_count, widest, with_192);
  BigParams p;
  p.w = a.w; p.scales = a.scales; p.biases = a.biases; p.x = a.x; p.y = a.y;
  p.lora_t = a.lora_t; p.lora_b = a.lora_b;
  p.K = a.K; p.N = a.N; p.M = a.M; p.r = a.r;
  p.tiles_m = (a.M + BM - 1) / BM;
  p.tiles_n = (a.N + bn - 1) / bn;
  p.gate_act = a.gate_act;
  p.out_stride = a.out_stride > 0 ? a.out_stride : a.N / 2;
  p.out_off = a.out_off;
  const dim3 grid(plan_tile_order(p)), block(kBigThreads);
  const bool lora = a.lora_t != nullptr;
  if (a.bits == 8) {
    if (lora || a.f16 || a.group != 64) { return hipErrorInvalidValue; }
    if (bn == 128) { return launch_kernel(qmm_big_kernel<2, false, kPacked8>, grid, block, 0, st, p); }
    return launch_kernel(qmm_big_kernel<3, false, kPacked8>, grid, block, 0, st, p);
  }
  if (a.group == 32) {
    if (lora || a.f16) { return hipErrorInvalidValue; }
    // 256 and 128 wide only: the 192-wide tile, whose threads' pieces change between two (row, half step) sets at a
    // place that differs from thread to thread, does not fit the registers beside the accumulators
    if (bn == 128) { return launch_kernel(qmm_big_kernel<2, false, kPacked4G32>, grid, block, 0, st, p); }
    return launch_kernel(qmm_big_kernel<4, false, kPacked4G32>, grid, block, 0, st, p);
  }
  if (a.f16) {
    // IEEE binary16 elements
    if (bn == 128) {
      return lora ? launch_kernel(qmm_big_kernel<2, true, kPacked4F16>, grid, block, 0, st, p)
                  : launch_kernel(qmm_big_kernel<2, false, kPacked4F16>, grid, block, 0, st, p);
    }
    if (bn == 192) {
      return lora ? launch_kernel(qmm_big_kernel<3, true, kPacked4F16>, grid, block, 0, st, p)
                  : launch_kernel(qmm_big_kernel<3, false, kPacked4F16>, grid, block, 0, st, p);
    }
    return lora ? launch_kernel(qmm_big_kernel<4, true, kPacked4F16>, grid, block, 0, st, p)
                : launch_kernel(qmm_big_kernel<4, false, kPacked4F16>, grid, block, 0, st, p);
  }
  if (bn == 128) {
    return lora ? launch_kernel(qmm_big_kernel<2, true>, grid, block, 0, st, p)
                : launch_kernel(qmm_big_kernel<2, false>, grid, block, 0, st, p);
  }
  if (bn == 192) {
    return lora ? launch_kernel(qmm_big_kernel<3, true>, grid, block, 0, st, p)
                : launch_kernel(qmm_big_kernel<3, false>, grid, block, 0, st, p);
  }
  return lora ? launch_kernel(qmm_big_kernel<4, true>, grid, block, 0, st, p)
              : launch_kernel(qmm_big_kernel<4, false>, grid, block, 0, st, p);
}

// y[M,N] = x[M,K] . b[N,K]^T on the large-tile kernel with dense weights (2-byte elements, fp32 accumulation):
// the contraction stage of the dequant-once route.  K % 32 == 0 (a last K step of 32), 16-byte aligned rows.
bool dense_gemm_supports(int M, int N, int K)
{
  return M >= 1 && N >= 1 && K >= 32 && K % 32 == 0 && (double)N * (double)K * 2.0 < 4.0e9 &&
         (double)BM * (double)K * 2.0 < 4.0e9;
}

// lora_t [M,r] / lora_b [N,r] (nullable together, bf16 only): the adapter's second factor in the same accumulators, as in
// the fused kernel.
hipError_t launch_dense_gemm(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K,
                             bool f16, int cu_count, const uint16_t* lora_t, const uint16_t* lora_b, int r)
{
  if (!dense_gemm_supports(M, N, K)) { return hipErrorInvalidValue; }
  const bool lora = lora_t != nullptr;
  if (lora && (f16 || lora_b == nullptr || r < 8 || r % 8 != 0)) { return hipErrorInvalidValue; }
  const int bn = qmm_big_tile_n(N, M, cu_count);
  BigParams p{};
  p.w = reinterpret_cast<const uint32_t*>(b);
  p.x = x; p.y = y;
  p.lora_t = lora_t; p.lora_b = lora_b; p.r = lora ? r : 0;
  p.K = K; p.N = N; p.M = M;
  p.tiles_m = (M + BM - 1) / BM;
  p.tiles_n = (N + bn - 1) / bn;
  const dim3 grid(plan_tile_order(p)), block(kBigThreads);
#define VPQ_DENSE(NTV)                                                                      \
  (f16 ? launch_kernel(qmm_big_kernel<NTV, false, kDenseF16>, grid, block, 0, st, p)       \
       : (lora ? launch_kernel(qmm_big_kernel<NTV, true, kDenseBf16>, grid, block, 0, st, p) \
               : launch_kernel(qmm_big_kernel<NTV, false, kDenseBf16>, grid, block, 0, st, p)))
  if (bn == 128) { return VPQ_DENSE(2); }
  if (bn == 192) { return VPQ_DENSE(3); }
  return VPQ_DENSE(4);
#undef VPQ_DENSE
}

// The contraction of the dequant-once route (the reference's `gemm_mma_`,
// generative-models/minimax-h3/metal-minimax-h3-transformer.cc:2020-2160: affine_dequant into a scratch, then the
// dense matrix-unit GEMM of gpu-kernels/metal/gemm/dense_gemm_mma.metal).  There the expansion costs 2*N*K bytes
// of traffic per call; here the caller may keep the expansion of an immutable weight.  0, or -2 with *why set
// when the shape is outside the kernel or the launch failed.
int dense_gemm_elt(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K, bool f16,
                   int cu_count, std::string* why, const uint16_t* lora_t, const uint16_t* lora_b, int r)
{
  if (!dense_gemm_supports(M, N, K)) {
    if (why) { *why = "dense GEMM: K must be a multiple of 32 and the matrices below 4 GB"; }
    return -2;
  }
  const hipError_t e = launch_dense_gemm(st, x, b, y, M, N, K, f16, cu_count, lora_t, lora_b, r);
  if (e != hipSuccess) {
    if (why) { *why = hipGetErrorString(e); }
    return -2;
  }
  return 0;
}

int dense_gemm_bf16(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K, int cu_count,
                    std::string* why)
{
  return dense_gemm_elt(st, x, b, y, M, N, K, false, cu_count, why);
}

}  // namespace vpq

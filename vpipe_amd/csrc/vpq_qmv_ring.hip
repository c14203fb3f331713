// QMV (1 <= M <= 16) for K % 512 == 0: x in registers, everything else through a two-slot
// LDS ring of direct-to-LDS loads per wavefront.
//
// The [N,K] pack is cut into items of 16 weight rows x 512 k (8 quantization groups, 4 KB
// of codes).  A workgroup of NW wavefronts owns TC consecutive 16-row tiles; wavefront w
// owns the k-slices w, w+NW, ... and walks, slice by slice, over the workgroup's tiles.
//   x       The wavefront's slice of x (every row, 512 values) is brought in ONCE per slice
//           and stays in 64 registers in the MFMA A-operand layout; so does -128 * sum(x) per
//           group (two MFMAs against a constant -128 operand).  Nothing about x is repeated
//           per item, whatever M is.
//   items   One item is five 128-bit direct-to-LDS loads into a wave-private slot: four for
//           the codes (16 rows x 256 bytes, chunks XOR-swizzled so that the 64-bit reads,
//           lane = weight row, do not collide on banks) and one for the 16 rows' scales and
//           biases (8 groups each).  Two slots per wavefront; a slot's content is copied to
//           registers first, the slot is re-requested for the item after next, and only then
//           the copy is contracted: two items are in flight during the arithmetic.
//   waits   The load counter retires requests in issue order, so `s_waitcnt vmcnt(n)` with
//           n = requests issued after the item is exact.  Everything in flight during the
//           steady state is a direct-to-LDS load (for M <= 4 the slices of x come through LDS
//           the same way: four loads, requested a whole slice ahead), which keeps the counts
//           to one rule: 5 per item, 4 per slice of x.  For M > 4 the slices of x are plain
//           register loads and the queue is drained (vmcnt(0)) at each change of slice.
//           The LDS reads of what those loads wrote are written as asm so that the compiler,
//           which cannot see the counts, does not add its own wait for everything.
//   math    codes -> bf16 (128 + q) by one v_and_or_b32 per nibble pair, contracted with x
//           on v_mfma_f32_16x16x32_bf16 seeded with -128*sum(x): the result is the group's
//           sum(x*q) exactly; then y += scale*sum(x*q) + bias*sum(x) in fp32 -- the factored
//           form of gpu-kernels/metal/quant/affine_qmv.metal:151-174.  The weight is never
//           rounded to bf16.
//   sums    per item the 16 x M partial results of a wavefront go to its own row of an LDS
//           table (added to what an earlier slice left there); after the last item one
//           barrier, and the first TC*MR*64 threads add the rows in wavefront order and
//           store y.  The order is fixed, so results are bit-reproducible.
//   split   K split across workgroups (the deep-K split of generative-models/shared/mma-splitk.h:30-52: fp32
//           planes, then a fold that adds them in order and rounds once): a workgroup re-reads all M rows of x
//           over its K range, which on a narrow N (few tiles per workgroup) and many rows is several times its
//           share of the pack -- 17408 -> 5120 at 16 rows: 557 KB of x for 78 KB of codes.  With `kparts` > 1
//           grid.y is the part: the workgroup walks the slices of its part only (x over that range, `kparts` times
//           the tiles for the same number of workgroups) and writes its fp32 sums to plane [part][M][N] of the
//           caller's workspace; qmv_ring_fold_kernel adds the planes in part order and applies the store's
//           residual and rounding (plain stores only: the gated entry points take no workspace).  No atomics, no fences: a second launch.
//
// No inline-assembly VALU instruction may sit near the MFMAs (the compiler's hazard
// recogniser cannot see what such a statement writes); the asm here is loads and waits only.
#include <cstddef>
#include <type_traits>

#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

constexpr int kTileN = 16;
constexpr int kKS = 512;                 // k-values per item
constexpr int kG = kKS / kGroup;         // groups per item (8)
constexpr int kRowBytes = kKS / 2;       // code bytes per row per item (256)
constexpr int kCodeBytes = kTileN * kRowBytes;   // 4096
constexpr int kSlotBytes = kCodeBytes + 1024;    // + one 64-lane load of scales | biases (twice)
constexpr int kItemLoads = 5;            // direct-to-LDS loads per item
constexpr int kXLoads = 4;               // direct-to-LDS loads per slice of x (M <= 4)
constexpr int kXBytes = kXLoads * 1024;  // staged rows of one slice of x
// TC * MR is bounded by the LDS table of partial sums: 8 KB beside the staged x of M <= 4,
// 64 KB where x lives in registers (more tiles per workgroup = fewer reloads of x).
constexpr int max_tc_mr(int mr) { return mr == 1 ? 4 : 32; }

// The first fourteen words arrive preloaded (everything the requests need); y, residual and gate_act, which only
// the store reads, follow.
struct RingParams {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  const uint16_t* x;
  int K, N, M;
  int slices;   // K / 512
  int tiles;    // ceil(N / 16)
  int tc;       // tiles per workgroup
  void* y;
  const uint16_t* residual;
  int gate_act; // rows are interleaved gate|up; y is [M, N/2] = act(gate) * up (1 SwiGLU, 2 GEGLU)
  int kparts;   // workgroups along K (grid.y); > 1: fp32 sums go to `plane`, the fold kernel stores y
  float* plane; // [kparts][M][N]
  int part_slices;   // slices per part
  int pad_;
};
static_assert(offsetof(RingParams, y) == kPreloadWords * 4, "y starts the part that is not preloaded");

// Eight nibbles of one packed word -> eight bf16 values 128+q, element order
// [k0,k4,k1,k5,k2,k6,k3,k7].  `mask` and `magic` arrive as opaque register values so that
// each pair costs a single v_and_or_b32.  F16: binary16 values 16+q instead (the code shifted to
// mantissa bits 6..9, where a step is 1/64 of 16.0's exponent: exact).
template <bool F16>
__device__ __forceinline__ u32x4 ring_codes_to_elts(uint32_t word, uint32_t mask, uint32_t magic)
{
  u32x4 v;
  if constexpr (F16) {
    v[0] = ((word << 6) & mask) | magic;
    v[1] = ((word << 2) & mask) | magic;
    v[2] = ((word >> 2) & mask) | magic;
    v[3] = ((word >> 6) & mask) | magic;
  } else {
    v[0] = (word & mask) | magic;
    v[1] = ((word >> 4) & mask) | magic;
    v[2] = ((word >> 8) & mask) | magic;
    v[3] = ((word >> 12) & mask) | magic;
  }
  return v;
}

// D = A (16 x 32) * B (32 x 16) + C on bf16 or binary16 operands, fp32 accumulation.
template <bool F16>
__device__ __forceinline__ floatx4 ring_mfma(u32x4 a, u32x4 b, floatx4 c)
{
  if constexpr (F16) {
    typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
}

// Eight consecutive elements of x -> the element order ring_codes_to_elts produces.
__device__ __forceinline__ u32x4 ring_permute_x(u32x4 d)
{
  u32x4 v;
  v[0] = __builtin_amdgcn_perm(d[2], d[0], 0x05040100u);  // x0,x4
  v[1] = __builtin_amdgcn_perm(d[2], d[0], 0x07060302u);  // x1,x5
  v[2] = __builtin_amdgcn_perm(d[3], d[1], 0x05040100u);  // x2,x6
  v[3] = __builtin_amdgcn_perm(d[3], d[1], 0x07060302u);  // x3,x7
  return v;
}

__device__ __forceinline__ uint32_t lds_address(const void* p)
{
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}

// LDS reads the compiler does not order against the direct-to-LDS loads in flight (it would
// wait for all of them); the caller has waited for the loads that filled the address.
__device__ __forceinline__ u32x2 lds_read_b64(uint32_t addr)
{
  u32x2 v;
  asm volatile("ds_read_b64 %0, %1" : "=v"(v) : "v"(addr) : "memory");
  return v;
}

__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr)
{
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
  return v;
}

__device__ __forceinline__ void load_to_lds(const void* src, void* lds_dst)
{
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)lds_dst, 16, 0, 0);
}

template <int N>
__device__ __forceinline__ void wait_loads()
{
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// An item taken out of its slot: the lane's codes (8 groups x 2 words), scales and biases.
struct Taken {
  u32x2 cws[kG];
  u32x4 s, b;
};

}  // namespace

// MR: accumulator registers per lane = ceil(M/4).  Row m of x sits in MFMA row 4*(m%4) + m/4,
// so that output row m is register m/4 of lane group m%4.  MR == 1 (M <= 4) stages x through LDS.
// F16: x, scales, biases, y and the residual are IEEE binary16 (the reference's VPIPE_ELT = half build); the codes
// become 16+q and the offset -16*sum(x).
template <int NW, int MR, bool F32OUT, bool F16 = false>
__global__ __launch_bounds__(NW * 64) void qmv_ring_kernel(VPQ_PRELOADED_WORDS, const PreloadTail<RingParams> tail)
{
  const RingParams p = preload_assemble<RingParams>(VPQ_PRELOADED_WORD_LIST, tail);
  constexpr bool XDMA = (MR == 1);
  __shared__ __attribute__((aligned(16))) uint8_t ring0[NW * kSlotBytes];
  __shared__ __attribute__((aligned(16))) uint8_t ring1[NW * kSlotBytes];
  __shared__ __attribute__((aligned(16))) uint8_t xstage[XDMA ? NW * kXBytes : 16];
  __shared__ float sums[max_tc_mr(MR) * NW * kWave];  // [tile][wave][register][lane]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int fr = lane & 15;                 // MFMA row (A) / column (B, D) of this lane
  const int g = lane >> 4;                  // k sub-block of this lane
  const int m_real = 4 * (fr & 3) + (fr >> 2);
  // MFMA rows beyond M produce outputs nobody stores; they read the last live row.
  const int x_row = m_real < p.M ? m_real : p.M - 1;
  const int Kg = p.K >> 6;
  const uint32_t row_bytes = (uint32_t)p.K >> 1;
  const int tile0 = blockIdx.x * p.tc;
  const int TC = p.tc;

  uint8_t* slot0 = ring0 + wave * kSlotBytes;
  uint8_t* slot1 = ring1 + wave * kSlotBytes;
  uint8_t* xbuf = xstage + (XDMA ? wave * kXBytes : 0);
  // Code words of the lane, relative to a slot: row fr, chunk (2*grp + g/2) ^ fr, half g%2.
  const uint32_t code_rel = (uint32_t)(fr * kRowBytes + (g & 1) * 8);
  const int lds_chunk0 = (g >> 1) ^ fr;
  // Load j of an item covers rows 4j..4j+3: lane l takes row 4j + l/16, LDS position l%16.
  const int ld_row = lane >> 4;
  const int ld_pos = lane & 15;

  uint32_t magic = F16 ? 0x4c004c00u : 0x43004300u;   // 16.0 (binary16) or 128.0 (bf16) in both halves
  uint32_t mask = F16 ? 0x03c003c0u : 0x000f000fu;
  asm volatile("" : "+v"(magic));           // no instruction: only hides the constants
  asm volatile("" : "+s"(mask));            // from constant folding
  u32x4 neg128;                             // the offset of the codes, negated: -128.0 (bf16) or -16.0 (binary16)
  neg128[0] = neg128[1] = neg128[2] = neg128[3] = F16 ? 0xcc00cc00u : 0xc300c300u;
  constexpr float kBiasOverOffset = F16 ? -0.0625f : -0.0078125f;

  // This wavefront's items: slices s_begin + wave, + NW, ... (rounds) of the workgroup's K part x its tiles.
  const int part = (int)blockIdx.y;
  const int s_begin = part * p.part_slices;
  const int s_count = (p.slices - s_begin) < p.part_slices ? (p.slices - s_begin) : p.part_slices;
  const int rounds = (s_count - wave + NW - 1) / NW;      // <= 0 for an idle wavefront
  const int n_items = rounds > 0 ? rounds * TC : 0;

  // Requests item i into a slot (i is clamped to the last item, so that the loop can request
  // without a condition; a tile beyond the last one re-reads the last tile and its results
  // are dropped at the store).
  auto request = [&](int i, uint8_t* slot) {
    const int ii = i < n_items ? i : n_items - 1;
    const int r = ii / TC;
    const int t = ii - r * TC;
    const int sl = s_begin + wave + r * NW;
    int tile = tile0 + t;
    if (tile >= p.tiles) { tile = p.tiles - 1; }
    const int n0 = tile * kTileN;
    const uint8_t* wbase = reinterpret_cast<const uint8_t*>(p.w) + (size_t)n0 * row_bytes + (size_t)sl * kRowBytes;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = 4 * j + ld_row;
      const int rrow = (n0 + row < p.N) ? row : (p.N - 1 - n0);
      const uint32_t off = (uint32_t)rrow * row_bytes + (uint32_t)((ld_pos ^ row) & 15) * 16u;
      load_to_lds(wbase + off, slot + j * (kWave * 16));
    }
    // Lanes 0-15: the 8 scales of rows 0-15; lanes 16-31: their biases; lanes 32-63 repeat.
    const int srow = (n0 + fr < p.N) ? (n0 + fr) : (p.N - 1);
    const uint16_t* const scales_v = p.scales;       // values, not a choice between two fields' addresses
    const uint16_t* const biases_v = p.biases;
    const uint16_t* sb = ((lane & 16) ? biases_v : scales_v) + (size_t)srow * Kg + (size_t)sl * kG;
    load_to_lds(sb, slot + kCodeBytes);
  };

  // Waits until only the loads issued after the slot's item can be in flight and copies the
  // lane's part of the item out of the slot.
  auto take = [&](const uint8_t* slot, bool x_behind, Taken& it) {
    if (XDMA && x_behind) {
      wait_loads<kItemLoads + kXLoads>();
    } else {
      wait_loads<kItemLoads>();
    }
    const uint32_t base = lds_address(slot);
#pragma unroll
    for (int grp = 0; grp < kG; ++grp) {
      it.cws[grp] = lds_read_b64(base + code_rel + (uint32_t)(((2 * grp) ^ lds_chunk0) * 16));
    }
    it.s = lds_read_b128(base + kCodeBytes + (uint32_t)fr * 16);
    it.b = lds_read_b128(base + kCodeBytes + 256 + (uint32_t)fr * 16);
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(it.cws[0]), "+v"(it.cws[1]), "+v"(it.cws[2]), "+v"(it.cws[3]), "+v"(it.cws[4]), "+v"(it.cws[5]),
                   "+v"(it.cws[6]), "+v"(it.cws[7]), "+v"(it.s), "+v"(it.b)
                 :
                 : "memory");
  };

  u32x4 xq[2 * kG];         // the slice of x as A operands
  float xneg[kG][MR];       // -128 * sum(x) per group, accumulator layout

  // M <= 4: requests slice r of x, rows 0..3 (rows beyond M repeat the last one), 1 KB each.
  auto request_x = [&](int r) {
    const int sl = s_begin + wave + r * NW;
#pragma unroll
    for (int m = 0; m < kXLoads; ++m) {
      const int mm = m < p.M ? m : p.M - 1;
      load_to_lds(p.x + (size_t)mm * p.K + (size_t)sl * kKS + lane * 8, xbuf + m * 1024);
    }
  };
  // Brings slice r of x into xq and forms xneg.  `younger`: loads issued after the slice's
  // request that may stay in flight (M <= 4); for M > 4 the queue is drained.
  auto fetch_x = [&](int r, auto younger) {
    if (XDMA) {
      wait_loads<decltype(younger)::value>();
      // fragment (grp, t) of lane (fr, g): k = grp*64 + g*16 + t*8 of row x_row
      const uint32_t xa = lds_address(xbuf) + (uint32_t)(x_row * 1024 + g * 32);
#pragma unroll
      for (int grp = 0; grp < kG; ++grp) {
#pragma unroll
        for (int t = 0; t < 2; ++t) { xq[2 * grp + t] = lds_read_b128(xa + (uint32_t)(grp * 128 + t * 16)); }
      }
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(xq[0]), "+v"(xq[1]), "+v"(xq[2]), "+v"(xq[3]), "+v"(xq[4]), "+v"(xq[5]), "+v"(xq[6]),
                     "+v"(xq[7]), "+v"(xq[8]), "+v"(xq[9]), "+v"(xq[10]), "+v"(xq[11]), "+v"(xq[12]), "+v"(xq[13]),
                     "+v"(xq[14]), "+v"(xq[15])
                   :
                   : "memory");
    } else {
      const int sl = s_begin + wave + r * NW;
      const uint16_t* xp = p.x + (size_t)x_row * p.K + (size_t)sl * kKS + g * 16;
#pragma unroll
      for (int grp = 0; grp < kG; ++grp) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xq[2 * grp + t]) : "v"(xp + grp * kGroup + t * 8) : "memory");
        }
      }
      asm volatile("s_waitcnt vmcnt(0)"
                   : "+v"(xq[0]), "+v"(xq[1]), "+v"(xq[2]), "+v"(xq[3]), "+v"(xq[4]), "+v"(xq[5]), "+v"(xq[6]),
                     "+v"(xq[7]), "+v"(xq[8]), "+v"(xq[9]), "+v"(xq[10]), "+v"(xq[11]), "+v"(xq[12]), "+v"(xq[13]),
                     "+v"(xq[14]), "+v"(xq[15])
                   :
                   : "memory");
    }
#pragma unroll
    for (int i = 0; i < 2 * kG; ++i) { xq[i] = ring_permute_x(xq[i]); }
#pragma unroll
    for (int grp = 0; grp < kG; ++grp) {
      floatx4 xn = {0.f, 0.f, 0.f, 0.f};
      xn = ring_mfma<F16>(xq[2 * grp], neg128, xn);
      xn = ring_mfma<F16>(xq[2 * grp + 1], neg128, xn);
#pragma unroll
      for (int q = 0; q < MR; ++q) { xneg[grp][q] = xn[q]; }
    }
  };

  // Contracts a taken item i and adds its partial sums to this wavefront's row of `sums`.
  auto compute = [&](int i, const Taken& it) {
    const int r = i / TC;
    const int t = i - r * TC;
    const uint32_t sd[4] = {it.s[0], it.s[1], it.s[2], it.s[3]};
    const uint32_t bd[4] = {it.b[0], it.b[1], it.b[2], it.b[3]};
    float acc[MR];
#pragma unroll
    for (int q = 0; q < MR; ++q) { acc[q] = 0.0f; }
#pragma unroll
    for (int grp = 0; grp < kG; ++grp) {
      const u32x2 cw = it.cws[grp];
      floatx4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int q = 0; q < MR; ++q) { s4[q] = xneg[grp][q]; }
      s4 = ring_mfma<F16>(xq[2 * grp], ring_codes_to_elts<F16>(cw[0], mask, magic), s4);
      s4 = ring_mfma<F16>(xq[2 * grp + 1], ring_codes_to_elts<F16>(cw[1], mask, magic), s4);
      const float s = (grp & 1) ? elt_hi_to_f32<F16>(sd[grp >> 1]) : elt_lo_to_f32<F16>(sd[grp >> 1]);
      const float b = (grp & 1) ? elt_hi_to_f32<F16>(bd[grp >> 1]) : elt_lo_to_f32<F16>(bd[grp >> 1]);
      const float b2 = b * kBiasOverOffset;          // bias * sum(x) = (bias / -offset) * xneg
#pragma unroll
      for (int q = 0; q < MR; ++q) {
        acc[q] = fmaf(s, s4[q], acc[q]);
        acc[q] = fmaf(b2, xneg[grp][q], acc[q]);
      }
    }
    float* mine = sums + ((t * NW + wave) * MR) * kWave + lane;
#pragma unroll
    for (int q = 0; q < MR; ++q) {
      if (r == 0) {
        mine[q * kWave] = acc[q];
      } else {
        mine[q * kWave] += acc[q];
      }
    }
  };

  if (n_items > 0) {
    int r = 0;                          // slice (round) of the item being computed
    int left = TC;                      // items left in it
    int x_behind = 0;                   // takes whose item still has a request of x behind it
    bool fresh = false;                 // the next compute starts a new slice
    if (XDMA) { request_x(0); }
    request(0, slot0);
    request(1, slot1);
    fetch_x(0, std::integral_constant<int, 2 * kItemLoads>());
    if (XDMA && rounds > 1) { request_x(1); x_behind = 2; }
    Taken it;
    // One item: take it out of its slot, re-request the slot for the item after next, bring
    // in the next slice of x if the item starts one (and request the slice after that, a
    // whole slice ahead), contract.
    auto step = [&](int i, uint8_t* slot) {
      take(slot, x_behind > 0, it);
      if (x_behind > 0) { --x_behind; }
      if (!XDMA && fresh) {
        // x in registers: the loads of the new slice drain the queue.  Issued before the slot is re-requested they
        // wait for the one item in flight (requested an item ago) and for themselves (L2), not for a request
        // to HBM made a moment earlier.
        fetch_x(r, std::integral_constant<int, kItemLoads>());
        fresh = false;
        request(i + 2, slot);
      } else {
        request(i + 2, slot);
        if (fresh) {
          fetch_x(r, std::integral_constant<int, kItemLoads>());
          fresh = false;
          if (r + 1 < rounds) { request_x(r + 1); x_behind = 2; }
        }
      }
      compute(i, it);
      if (--left == 0) { ++r; left = TC; fresh = true; }
    };
    for (int i = 0; i < n_items; i += 2) {
      step(i, slot0);
      if (i + 1 < n_items) { step(i + 1, slot1); }
    }
    // The requests past the end are still writing this wavefront's slots.
    wait_loads<0>();
  }
  __syncthreads();

  // The TC*MR*64 outputs are dealt to the threads one wavefront's worth at a time: each adds, in
  // wavefront order, the partial sums of one (tile, register, lane) and stores
  // y[m = 4*register + lane/16][tile*16 + lane%16].
  for (int o_idx = threadIdx.x; o_idx < TC * MR * kWave; o_idx += NW * kWave) {
    const int t = o_idx / (MR * kWave);
    const int q = (o_idx / kWave) % MR;
    const int l = o_idx & 63;
    const int live = s_count < NW ? s_count : NW;
    float total = 0.0f;
    for (int wv = 0; wv < live; ++wv) { total += sums[((t * NW + wv) * MR + q) * kWave + l]; }
    const int m = 4 * q + (l >> 4);
    const int tile = tile0 + t;
    const int n = tile * kTileN + (l & 15);
    if (p.kparts > 1) {
      if (tile < p.tiles && m < p.M && n < p.N) { p.plane[((size_t)part * p.M + m) * p.N + n] = total; }
    } else if (p.gate_act) {
      // Lanes 2j and 2j+1 hold the gate and the up sum of one feature (N is even).
      const float up = from_neighbour_lane(total);
      if (tile < p.tiles && m < p.M && n < p.N && (l & 1) == 0) {
        const float v = gated_f32(p.gate_act, total, up);
        const size_t o = (size_t)m * (p.N >> 1) + (n >> 1);
        if (F32OUT) {
          reinterpret_cast<float*>(p.y)[o] = v;
        } else {
          reinterpret_cast<uint16_t*>(p.y)[o] = (uint16_t)f32_to_elt_bits<F16>(v);
        }
      }
    } else if (tile < p.tiles && m < p.M && n < p.N) {
      const size_t o = (size_t)m * p.N + n;
      if (F32OUT) {
        reinterpret_cast<float*>(p.y)[o] = total;
      } else {
        uint32_t v = f32_to_elt_bits<F16>(total);
        if (p.residual != nullptr) {
          v = f32_to_elt_bits<F16>(elt_bits_to_f32<F16>(v) + elt_bits_to_f32<F16>(p.residual[o]));
        }
        reinterpret_cast<uint16_t*>(p.y)[o] = (uint16_t)v;
      }
    }
  }
}

// y = store(plane[0] + plane[1] + ...), the parts added in order: one thread per output element.
template <bool F32OUT, bool F16>
__global__ __launch_bounds__(256) void qmv_ring_fold_kernel(const float* __restrict__ plane, void* __restrict__ y,
                                                            const uint16_t* __restrict__ residual, int M, int N, int kparts)
{
  const size_t MN = (size_t)M * N;
  const size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= MN) { return; }
  float total = 0.0f;
  for (int k = 0; k < kparts; ++k) { total += plane[k * MN + o]; }
  if (F32OUT) {
    reinterpret_cast<float*>(y)[o] = total;
  } else {
    uint32_t v = f32_to_elt_bits<F16>(total);
    if (residual != nullptr) { v = f32_to_elt_bits<F16>(elt_bits_to_f32<F16>(v) + elt_bits_to_f32<F16>(residual[o])); }
    reinterpret_cast<uint16_t*>(y)[o] = (uint16_t)v;
  }
}

bool qmv_ring_supports(int K, int N, int M)
{
  return K % kKS == 0 && N >= 1 && M >= 1 && M <= 16;
}

size_t qmv_ring_workspace_bytes(int K, int N, int M)
{
  if (!qmv_ring_supports(K, N, M) || K / kKS < 2) { return 0; }
  const int parts = K / kKS < 4 ? K / kKS : 4;
  return (size_t)parts * (size_t)M * (size_t)N * sizeof(float);
}

namespace {

template <int NW, bool F16>
hipError_t launch_nw(hipStream_t st, const RingParams& p, int mr, bool f32)
{
  const dim3 grid((unsigned)((p.tiles + p.tc - 1) / p.tc), (unsigned)p.kparts), block((unsigned)(NW * kWave));
  if (f32) {
    if (mr == 1) { return launch_preloaded(qmv_ring_kernel<NW, 1, true, F16>, grid, block, 0, st, p); }
    if (mr == 2) { return launch_preloaded(qmv_ring_kernel<NW, 2, true, F16>, grid, block, 0, st, p); }
    return launch_preloaded(qmv_ring_kernel<NW, 4, true, F16>, grid, block, 0, st, p);
  }
  if (mr == 1) { return launch_preloaded(qmv_ring_kernel<NW, 1, false, F16>, grid, block, 0, st, p); }
  if (mr == 2) { return launch_preloaded(qmv_ring_kernel<NW, 2, false, F16>, grid, block, 0, st, p); }
  return launch_preloaded(qmv_ring_kernel<NW, 4, false, F16>, grid, block, 0, st, p);
}

}  // namespace

// tc_hint > 0 forces the tiles per workgroup (measurement).  splits_hint: 0 = K across workgroups where a.ws has
// the room and the cost model says it pays, 1 = never, n > 1 = n parts (if a.ws has the room).
hipError_t launch_qmv_ring(hipStream_t st, const QmvArgs& a, int tc_hint, int splits_hint, bool f16)
{
  RingParams p;
  p.w = a.w; p.scales = a.scales; p.biases = a.biases; p.x = a.x; p.y = a.y;
  p.residual = a.residual;
  p.K = a.K; p.N = a.N; p.M = a.M;
  p.gate_act = a.gate_act;
  p.slices = a.K / kKS;
  p.tiles = (a.N + kTileN - 1) / kTileN;
  int mr = (a.M + 3) / 4;
  if (mr == 3) { mr = 4; }
  const int cus = a.cu_count > 0 ? a.cu_count : 256;
  // Tiles per workgroup.  One workgroup is resident per CU, so the launch runs in generations of `cus`
  // workgroups, each lasting about as long as a workgroup's bytes: its tiles' codes, scales and biases plus
  // all of x once.  The count that minimises generations x bytes per workgroup wins; the largest count
  // often does not (9496 tiles at 16 per workgroup: 594 workgroups, a third generation for 82 of them).
  const double tile_bytes = 16.0 * (double)a.K * 9.0 / 16.0, x_bytes = (double)a.M * (double)a.K * 2.0;
  // cost of a launch with t tiles per workgroup and K in `parts` parts, in bytes a workgroup moves per generation
  auto plan = [&](int regs, int parts, int& tc_out) {
    double best = 0.0;
    for (int t = 1; t <= max_tc_mr(regs) / regs; ++t) {
      const int wgs = ((p.tiles + t - 1) / t) * parts;
      const double cost = (double)((wgs + cus - 1) / cus) * ((double)t * tile_bytes + x_bytes) / (double)parts;
      if (t == 1 || cost <= best) { best = cost; tc_out = t; }
    }
    return best;
  };
  int tc = 1;
  double cost = plan(mr, 1, tc);
  // Up to 4 rows: the staged-x form has room for 4 tiles per workgroup; where that costs a generation the
  // two-register form (up to 16 tiles) is worth more than its idle accumulator register.
  if (mr == 1 && a.M >= 2) {
    int tc2 = 1;
    const double c2 = plan(2, 1, tc2);
    if (c2 * 1.05 < cost) { mr = 2; tc = tc2; cost = c2; }
  }
  // K across workgroups where the caller's workspace holds the planes and it pays.  Measured (kernel + fold, us,
  // unsplit / 4 parts): 17408 -> 5120 at 16 rows 26.3 / 23.5, at 8 rows 21.4 / 20.5, at 4 rows 17.2 / 22.5;
  // 5120 -> 5120 at 16 rows 11.7 / 14.8; 5120 -> 17408 at 16 rows 19.4 / 31.1; 5120 -> 151936 123.8 / 202.2: the
  // fold's launch and the shorter K walks cost more than the re-read x except for many rows over a deep K with few
  // tiles per CU.  Every element of a plane is written by exactly one workgroup before the fold reads it, so the
  // workspace needs no clearing.
  p.kparts = 1;
  p.part_slices = p.slices;
  p.plane = nullptr;
  if (splits_hint != 1 && a.ws != nullptr && p.slices >= 2 && a.gate_act == 0) {     // (the gated entry points take no workspace)
    int parts = splits_hint > 1 ? splits_hint : ((a.M >= 8 && p.slices >= 24 && p.tiles <= 2 * cus) ? 4 : 1);
    if (parts > p.slices) { parts = p.slices; }
    if (parts > 1 && (size_t)parts * (size_t)a.M * (size_t)a.N * sizeof(float) <= a.ws_bytes) {
      p.part_slices = (p.slices + parts - 1) / parts;
      p.kparts = (p.slices + p.part_slices - 1) / p.part_slices;      // no empty part
      p.plane = static_cast<float*>(a.ws);
      int tcp = 1;
      plan(mr, p.kparts, tcp);
      tc = tcp;
    } else if (splits_hint > 1) {
      return hipErrorInvalidValue;
    }
  }
  const int tc_max = max_tc_mr(mr) / mr;
  if (tc_hint > 0) { tc = tc_hint < tc_max ? tc_hint : tc_max; }
  p.tc = tc;
  p.pad_ = 0;
  if (p.kparts > 1) {
    const hipError_t e = f16 ? launch_nw<8, true>(st, p, mr, a.y_f32) : launch_nw<8, false>(st, p, mr, a.y_f32);
    if (e != hipSuccess) { return e; }
    const size_t outs = (size_t)a.M * a.N;
    const dim3 fgrid((unsigned)((outs + 255) / 256)), fblock(256);
    if (a.y_f32) {
      return f16 ? launch_kernel(qmv_ring_fold_kernel<true, true>, fgrid, fblock, 0, st, (const float*)p.plane, a.y, a.residual, a.M, a.N, p.kparts)
                 : launch_kernel(qmv_ring_fold_kernel<true, false>, fgrid, fblock, 0, st, (const float*)p.plane, a.y, a.residual, a.M, a.N, p.kparts);
    }
    return f16 ? launch_kernel(qmv_ring_fold_kernel<false, true>, fgrid, fblock, 0, st, (const float*)p.plane, a.y, a.residual, a.M, a.N, p.kparts)
               : launch_kernel(qmv_ring_fold_kernel<false, false>, fgrid, fblock, 0, st, (const float*)p.plane, a.y, a.residual, a.M, a.N, p.kparts);
  }
  return f16 ? launch_nw<8, true>(st, p, mr, a.y_f32) : launch_nw<8, false>(st, p, mr, a.y_f32);
}

}  // namespace vpq

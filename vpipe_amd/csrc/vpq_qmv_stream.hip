// QMV for M <= 4: the streaming form of the MFMA kernel in vpq_qmv_mfma.hip.
//
// Same items (16 weight rows x 512 k-values), same arithmetic, but built to keep
// the VALU work per item near its floor (nibble -> bf16 conversion and the
// per-group scale/bias combine) and to keep loads in flight while computing:
//   * a workgroup covers `tpb` 16-row tiles of N over the whole of K.  It stages
//     x ONCE into LDS (coalesced 128-bit loads, reordered for the MFMA operand
//     layout) together with -128*sum(x) of every quantization group;
//   * a wavefront owns one tile and R consecutive K slices of it (R is chosen on
//     the host so that the launch has enough wavefronts to fill the chip; with
//     a large N a wavefront takes a tile's whole K and nothing is reduced across
//     wavefronts);
//   * per item the packed codes travel global -> LDS by direct-to-LDS loads into
//     one wave-private 4 KB buffer; the wavefront copies them to registers,
//     immediately issues the loads of its NEXT item into the same buffer, and
//     only then does the arithmetic, so one item is always in flight per
//     wavefront and there is no barrier inside the loop;
//   * the partial sums of the wavefronts that share a tile meet in LDS once, at
//     the end.
// The LDS regions are separate static arrays on purpose: the compiler orders a
// ds_read after an outstanding direct-to-LDS load only when the two may alias,
// and reads of staged x must not wait for the next item's codes.
#include <cstddef>

#include "vpq_device.h"
#include "vpq_internal.h"


namespace vpq {

namespace {

constexpr int kTileN = 16;
constexpr int kKS = 512;
constexpr int kG = kKS / kGroup;
constexpr int kRowBytes = kKS / 2;
constexpr int kItemBytes = kTileN * kRowBytes;   // 4096
constexpr int kXPad = 16;                        // bytes of padding per staged 512-value slice row
constexpr int kSliceStride = kKS * 2 + kXPad;    // LDS bytes of one staged slice of one x row

// The first fourteen words arrive preloaded (what the requests need); the store's y and residual follow.
struct StreamParams {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  const uint16_t* x;
  int K, N, M;
  int slices;       // K / 512
  int tiles;        // ceil(N / 16)
  // bits 0-15: R, the K slices per wavefront; 16-23: wavefronts per tile = ceil(slices / R); 24-31: tiles per workgroup
  int plan;
  void* y;
  const uint16_t* residual;
};
static_assert(offsetof(StreamParams, y) == kPreloadWords * 4, "y starts the part that is not preloaded");

// Eight nibbles of a packed word -> eight elements 128+q (bf16) or 16+q (binary16: the code shifted to mantissa
// bits 6..9), element order [k0,k4,k1,k5,k2,k6,k3,k7]; one v_and_or_b32 per pair.
template <bool F16>
__device__ __forceinline__ u32x4 codes_to_elts(uint32_t word, uint32_t mask, uint32_t magic)
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

template <bool F16>
__device__ __forceinline__ floatx4 stream_mfma(u32x4 a, u32x4 b, floatx4 c)
{
  if constexpr (F16) {
    typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
}

__device__ __forceinline__ uint4 permute_x(uint4 d)
{
  uint4 v;
  v.x = __builtin_amdgcn_perm(d.z, d.x, 0x05040100u);  // x0,x4
  v.y = __builtin_amdgcn_perm(d.z, d.x, 0x07060302u);  // x1,x5
  v.z = __builtin_amdgcn_perm(d.w, d.y, 0x05040100u);  // x2,x6
  v.w = __builtin_amdgcn_perm(d.w, d.y, 0x07060302u);  // x3,x7
  return v;
}

}  // namespace

// NWMAX: wavefronts the static LDS is sized for (the launch may use fewer).
// XBYTES: bytes of LDS for the staged x of the whole K range, all M rows.
// F16: x, scales, biases, y and the residual are IEEE binary16; the offset of the codes is 16 instead of 128.
template <int NWMAX, int XBYTES, bool F32OUT, bool F16 = false>
__global__ __launch_bounds__(NWMAX * 64) void qmv_stream_kernel(VPQ_PRELOADED_WORDS, const PreloadTail<StreamParams> tail)
{
  const StreamParams p = preload_assemble<StreamParams>(VPQ_PRELOADED_WORD_LIST, tail);
  const int plan_R = p.plan & 0xffff, plan_wpt = (p.plan >> 16) & 0xff, plan_tpb = (p.plan >> 24) & 0xff;
  // Capacity of the per-(row, group) -128*sum(x) table: XBYTES holds M*K/512 slices of 1040
  // bytes, each with 8 groups.
  constexpr int GROUPS = XBYTES / kSliceStride * kG;
  __shared__ __attribute__((aligned(16))) uint8_t codes_lds[NWMAX * kItemBytes];
  __shared__ __attribute__((aligned(16))) uint8_t x_lds[XBYTES];
  __shared__ __attribute__((aligned(16))) float xneg_lds[GROUPS];
  // The partial sums of wavefronts that share a tile meet in the code buffers once nobody reads codes any more.
  float* red_lds = reinterpret_cast<float*>(codes_lds);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int fr = lane & 15;
  const int g = lane >> 4;
  const uint32_t Kg = (uint32_t)p.K >> 6;
  const uint32_t row_bytes_total = (uint32_t)p.K >> 1;

  // ---- this wavefront's unit: one tile, slices [sl0, sl1) ----
  const int tile_local = wave / plan_wpt;
  const int kr = wave - tile_local * plan_wpt;
  const int tile = blockIdx.x * plan_tpb + tile_local;
  const bool active = tile < p.tiles;
  const int sl0 = kr * plan_R;
  int sl1 = sl0 + plan_R;
  if (sl1 > p.slices) { sl1 = p.slices; }

  // ---- per-lane offsets.  Rows past N (ragged last tile) re-read the last real row; their
  //      outputs are never stored. ----
  constexpr int CH = kRowBytes / 16;          // 16
  constexpr int ROWS_PER_LOAD = kWave / CH;   // 4
  constexpr int NLOAD = kTileN / ROWS_PER_LOAD;
  uint8_t* wbuf = codes_lds + wave * kItemBytes;
  const int tile_c = active ? tile : p.tiles - 1;
  const int rows_here = (p.N - tile_c * kTileN) < kTileN ? (p.N - tile_c * kTileN) : kTileN;
  uint32_t code_off[NLOAD];
#pragma unroll
  for (int i = 0; i < NLOAD; ++i) {
    const int row = i * ROWS_PER_LOAD + lane / CH;
    const uint32_t chunk = (uint32_t)((lane % CH) ^ (row & (CH - 1))) * 16;
    code_off[i] = (uint32_t)(row < rows_here ? row : rows_here - 1) * row_bytes_total + chunk;
  }
  const uint8_t* wtile = reinterpret_cast<const uint8_t*>(p.w) + (size_t)tile_c * kTileN * row_bytes_total;
  const uint8_t* stile = reinterpret_cast<const uint8_t*>(p.scales) + (size_t)tile_c * kTileN * Kg * 2;
  const uint8_t* btile = reinterpret_cast<const uint8_t*>(p.biases) + (size_t)tile_c * kTileN * Kg * 2;
  // Scales and biases are fetched for four consecutive slices at a time: lane l takes the
  // 16 bytes (8 groups) of row l/4, slice l%4 of the batch, so the four lanes of a row read
  // 64 contiguous bytes.  At item j of the batch, the lane that needs row fr gets them from
  // lane 4*fr + j through the LDS crossbar (ds_bpermute).
  const int sb_row = lane >> 2, sb_pc = lane & 3;
  const uint32_t sb_off = (uint32_t)(sb_row < rows_here ? sb_row : rows_here - 1) * Kg * 2;
  uint4 sbat = make_uint4(0, 0, 0, 0), bbat = make_uint4(0, 0, 0, 0);

  // Puts the loads of slice sl in flight: codes -> this wave's LDS buffer and, at the start of
  // a batch of four slices, that batch's scales/biases -> registers.
  auto issue_item = [&](int sl) {
    const uint8_t* wbase = wtile + (size_t)sl * kRowBytes;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(wbase + code_off[i]),
          (__attribute__((address_space(3))) void*)(wbuf + i * (kWave * 16)), 16, 0, 0);
    }
    if (((sl - sl0) & 3) == 0) {
      int s = sl + sb_pc;
      if (s >= sl1) { s = sl1 - 1; }
      sbat = *reinterpret_cast<const uint4*>(stile + (size_t)s * (kG * 2) + sb_off);
      bbat = *reinterpret_cast<const uint4*>(btile + (size_t)s * (kG * 2) + sb_off);
    }
  };
  const bool work = active && sl0 < sl1;
  if (work) { issue_item(sl0); }              // first item in flight before anything else

  // ---- stage x: [M][slices][512] bf16, each 8-value piece reordered for the MFMA operand,
  //      and -128 * sum(x) per (row, group): 8 lanes hold the 64 values of a group ----
  const int xrow_stride = p.slices * kSliceStride;
  {
    const int pieces_per_row = p.K >> 3;
    const int total = p.M * pieces_per_row;                 // a multiple of 64
    for (int i = threadIdx.x; i < total; i += blockDim.x) {
      const int m = i / pieces_per_row;
      const int j = i - m * pieces_per_row;                 // 16-byte piece within the row
      const uint4 d = *reinterpret_cast<const uint4*>(p.x + (size_t)m * p.K + (size_t)j * 8);
      *reinterpret_cast<uint4*>(x_lds + m * xrow_stride + (j >> 6) * kSliceStride + (j & 63) * 16) = permute_x(d);
      float sum = ((elt_lo_to_f32<F16>(d.x) + elt_hi_to_f32<F16>(d.x)) + (elt_lo_to_f32<F16>(d.y) + elt_hi_to_f32<F16>(d.y))) +
                  ((elt_lo_to_f32<F16>(d.z) + elt_hi_to_f32<F16>(d.z)) + (elt_lo_to_f32<F16>(d.w) + elt_hi_to_f32<F16>(d.w)));
      sum += __shfl_xor(sum, 1, kWave);
      sum += __shfl_xor(sum, 2, kWave);
      sum += __shfl_xor(sum, 4, kWave);
      if ((lane & 7) == 0) { xneg_lds[m * Kg + (j >> 3)] = (F16 ? -16.0f : -128.0f) * sum; }
    }
  }
  __syncthreads();

  uint32_t magic = F16 ? 0x4c004c00u : 0x43004300u;   // 16.0 (binary16) or 128.0 (bf16) in both halves
  uint32_t mask = F16 ? 0x03c003c0u : 0x000f000fu;
  asm volatile("" : "+v"(magic));           // no instruction: hides the constants from folding
  asm volatile("" : "+s"(mask));

  // Row of x this lane's MFMA row stands for: MFMA row i = fr is x row 4*(i%4) + i/4, so that
  // output row m sits in accumulator register 0 of lane group m (M <= 4).
  const int m_real = 4 * (fr & 3) + (fr >> 2);
  const int x_row = m_real < p.M ? m_real : p.M - 1;
  const int m_out = g < p.M ? g : p.M - 1;  // accumulator register 0 of this lane is output row g
  const int lds_code0 = fr * kRowBytes + (g & 1) * 8;
  const int lds_chunk0 = (g >> 1) ^ fr;
  const uint8_t* xs_base = x_lds + x_row * xrow_stride + g * 32;
  const float* xn_base = xneg_lds + m_out * Kg;

  float acc = 0.0f;
  if (work) {
    for (int sl = sl0; sl < sl1; ++sl) {
      // The item's loads have landed: copy the codes out of the buffer ...
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      const int src = (4 * fr + ((sl - sl0) & 3)) * 4;      // byte index of the source lane
      uint4 sv, bv;
      sv.x = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)sbat.x);
      sv.y = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)sbat.y);
      sv.z = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)sbat.z);
      sv.w = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)sbat.w);
      bv.x = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bbat.x);
      bv.y = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bbat.y);
      bv.z = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bbat.z);
      bv.w = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bbat.w);
      uint2 cw[kG];
#pragma unroll
      for (int grp = 0; grp < kG; ++grp) {
        cw[grp] = *reinterpret_cast<const uint2*>(wbuf + lds_code0 + (((2 * grp) ^ lds_chunk0) * 16));
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      // ... and put the next item's loads in flight before doing the arithmetic.
      if (sl + 1 < sl1) { issue_item(sl + 1); }

      const uint8_t* xs = xs_base + sl * kSliceStride;
      const float4 xn0 = *reinterpret_cast<const float4*>(xn_base + sl * kG);
      const float4 xn1 = *reinterpret_cast<const float4*>(xn_base + sl * kG + 4);
      const float xneg[kG] = {xn0.x, xn0.y, xn0.z, xn0.w, xn1.x, xn1.y, xn1.z, xn1.w};
      const uint32_t sd[4] = {sv.x, sv.y, sv.z, sv.w};
      const uint32_t bd[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
      for (int grp = 0; grp < kG; ++grp) {
        const u32x4 a0 = *reinterpret_cast<const u32x4*>(xs + grp * 128);
        const u32x4 a1 = *reinterpret_cast<const u32x4*>(xs + grp * 128 + 16);
        floatx4 s4 = {0.f, 0.f, 0.f, 0.f};
        s4 = stream_mfma<F16>(a0, codes_to_elts<F16>(cw[grp].x, mask, magic), s4);
        s4 = stream_mfma<F16>(a1, codes_to_elts<F16>(cw[grp].y, mask, magic), s4);
        const float sc = (grp & 1) ? elt_hi_to_f32<F16>(sd[grp >> 1]) : elt_lo_to_f32<F16>(sd[grp >> 1]);
        const float bi = (grp & 1) ? elt_hi_to_f32<F16>(bd[grp >> 1]) : elt_lo_to_f32<F16>(bd[grp >> 1]);
        const float sxq = s4[0] + xneg[grp];               // sum(x*(128+q)) - 128*sum(x)
        acc = fmaf(sc, sxq, acc);
        acc = fmaf(bi * (F16 ? -0.0625f : -0.0078125f), xneg[grp], acc);      // bias * sum(x)
      }
    }
  }

  // acc of lane l is this wavefront's part of y[m = l/16][tile*16 + l%16].
  float total = acc;
  if (plan_wpt > 1) {
    __syncthreads();                         // every wavefront has taken its last item out of its buffer
    red_lds[wave * kWave + lane] = acc;
    __syncthreads();
    if (kr != 0) { return; }
    for (int i = 1; i < plan_wpt; ++i) { total += red_lds[(wave + i) * kWave + lane]; }
  }
  const int n = tile * kTileN + fr;
  if (active && g < p.M && n < p.N) {
    const size_t o = (size_t)g * p.N + n;
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

bool qmv_stream_supports(int K, int N, int M)
{
  if (K % kKS != 0 || N < 1 || M < 1 || M > 4) { return false; }
  const int slices = K / kKS;
  const int xbytes = M * slices * kSliceStride;
  return xbytes <= 72 * 1024;
}

hipError_t launch_qmv_stream(hipStream_t st, const QmvArgs& a, bool f16)
{
  StreamParams p;
  p.w = a.w; p.scales = a.scales; p.biases = a.biases; p.x = a.x; p.y = a.y; p.residual = a.residual;
  p.K = a.K; p.N = a.N; p.M = a.M;
  p.slices = a.K / kKS;
  p.tiles = (a.N + kTileN - 1) / kTileN;
  const int xbytes = a.M * p.slices * kSliceStride;
  const int cus = a.cu_count > 0 ? a.cu_count : 256;

  // K ranges (wavefronts) per tile: the fewest of 1, 2, 4, 8 that still put ~12 wavefronts
  // per CU in the launch; a workgroup is 8 wavefronts = 8 / wpt whole tiles.
  const long want_units = (long)cus * 12;
  int wpt = 1;
  while (wpt < 8 && wpt < p.slices && (long)p.tiles * wpt < want_units) { wpt *= 2; }
  if (wpt > p.slices) { wpt = p.slices; }
  if (wpt > 8) { wpt = 8; }
  const int R = (p.slices + wpt - 1) / wpt;
  wpt = (p.slices + R - 1) / R;
  int tpb = 8 / wpt;
  if (tpb > p.tiles) { tpb = p.tiles; }
  p.plan = R | (wpt << 16) | (tpb << 24);
  const int nw = tpb * wpt;
  const dim3 grid((unsigned)((p.tiles + tpb - 1) / tpb)), block((unsigned)(nw * kWave));

#define VPQ_STREAM(XB)                                                                                   \
  (f16 ? (a.y_f32 ? launch_preloaded(qmv_stream_kernel<8, XB, true, true>, grid, block, 0, st, p)          \
                  : launch_preloaded(qmv_stream_kernel<8, XB, false, true>, grid, block, 0, st, p))        \
       : (a.y_f32 ? launch_preloaded(qmv_stream_kernel<8, XB, true>, grid, block, 0, st, p)                \
                  : launch_preloaded(qmv_stream_kernel<8, XB, false>, grid, block, 0, st, p)))
  if (xbytes <= 13 * 1024) { return VPQ_STREAM(13 * 1024); }
  if (xbytes <= 26 * 1024) { return VPQ_STREAM(26 * 1024); }
  // 42 KB: four rows of K = 5120 (41600 bytes) still leave room for two workgroups per CU; the next size does not
  // (lm_head at 4 rows: 98 us with one workgroup per CU).
  if (xbytes <= 42 * 1024) { return VPQ_STREAM(42 * 1024); }
  return VPQ_STREAM(72 * 1024);
#undef VPQ_STREAM
}

}  // namespace vpq

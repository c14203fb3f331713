// Bandwidth kernels around the packed format: dense expansion, the packer,
// and the F16 -> bf16 conversion of scales/biases done once at load.
#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

// One thread per packed word: 4-byte coalesced loads, 16-byte coalesced
// stores.  out = bf16_rne(fp32(s*q + b)); s*q is exact in fp32 (8-bit x 4-bit
// significands), so the fused multiply-add below equals the two-step form of
// gpu-kernels/metal/quant/affine_dequant.metal:45-52 bit for bit.
// WS: log2 of the words per quantization group (3: group 64; 2: group 32, affine_dequant.metal:196-228).
// F16: scales, biases and the output are IEEE binary16 (the reference's VPIPE_ELT = half build).
template <int WS, bool F16 = false>
__global__ __launch_bounds__(256) void dequant_w4_kernel(
    const uint32_t* __restrict__ w, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, uint4* __restrict__ out, int Kw, size_t total_words)
{
  const int Kg = Kw >> WS;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total_words;
       idx += (size_t)gridDim.x * 256) {
    const size_t n = idx / (size_t)Kw;
    const int j = (int)(idx - n * (size_t)Kw);
    const size_t g = n * (size_t)Kg + (size_t)(j >> WS);
    const float s = elt_bits_to_f32<F16>(scales[g]);
    const float b = elt_bits_to_f32<F16>(biases[g]);
    const uint32_t p = w[idx];
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { v[i] = fmaf(s, (float)((p >> (4 * i)) & 0xfu), b); }
    uint4 o;
    o.x = pack_elt2<F16>(v[0], v[1]);
    o.y = pack_elt2<F16>(v[2], v[3]);
    o.z = pack_elt2<F16>(v[4], v[5]);
    o.w = pack_elt2<F16>(v[6], v[7]);
    out[idx] = o;
  }
}

hipError_t launch_dequant(hipStream_t st, const uint32_t* w, const uint16_t* scales,
                          const uint16_t* biases, uint16_t* out, int K, int N)
{
  const int Kw = K / 8;
  const size_t total = (size_t)N * (size_t)Kw;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536 * 4) { blocks = 65536 * 4; }
  return launch_kernel(dequant_w4_kernel<3>, dim3((unsigned)blocks), dim3(256), 0, st, w, scales,
                       biases, reinterpret_cast<uint4*>(out), Kw, total);
}

hipError_t launch_dequant_f16(hipStream_t st, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, uint16_t* out, int K, int N)
{
  const int Kw = K / 8;
  const size_t total = (size_t)N * (size_t)Kw;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536 * 4) { blocks = 65536 * 4; }
  return launch_kernel(dequant_w4_kernel<3, true>, dim3((unsigned)blocks), dim3(256), 0, st, w, scales,
                       biases, reinterpret_cast<uint4*>(out), Kw, total);
}

hipError_t launch_dequant_g32(hipStream_t st, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, uint16_t* out, int K, int N)
{
  const int Kw = K / 8;
  const size_t total = (size_t)N * (size_t)Kw;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536 * 4) { blocks = 65536 * 4; }
  return launch_kernel(dequant_w4_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, st, w, scales,
                       biases, reinterpret_cast<uint4*>(out), Kw, total);
}

// 8-bit twin (gpu-kernels/metal/quant/affine_dequant.metal:60-97): one byte per value, four per word;
// one thread per word, 8-byte stores.  s*q is exact in fp32 (8-bit x 8-bit significands).  WS: log2 of the words
// per quantization group (4: group 64; 3: group 32, affine_dequant_w8g32, :99-131).
// F16: scales, biases and the output are IEEE binary16 (the reference's VPIPE_ELT = half build, which is what its
// codec runs this expansion in); s*q stays exact in fp32 (11-bit x 8-bit significands).
template <int WS, bool F16 = false>
__global__ __launch_bounds__(256) void dequant_w8_kernel(
    const uint32_t* __restrict__ w, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, uint2* __restrict__ out, int Kw, size_t total_words)
{
  const int Kg = Kw >> WS;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total_words; idx += (size_t)gridDim.x * 256) {
    const size_t n = idx / (size_t)Kw;
    const int j = (int)(idx - n * (size_t)Kw);
    const size_t g = n * (size_t)Kg + (size_t)(j >> WS);
    const float s = elt_bits_to_f32<F16>(scales[g]);
    const float b = elt_bits_to_f32<F16>(biases[g]);
    const uint32_t p = w[idx];
    uint2 o;
    o.x = pack_elt2<F16>(fmaf(s, (float)(p & 0xffu), b), fmaf(s, (float)((p >> 8) & 0xffu), b));
    o.y = pack_elt2<F16>(fmaf(s, (float)((p >> 16) & 0xffu), b), fmaf(s, (float)(p >> 24), b));
    out[idx] = o;
  }
}

hipError_t launch_dequant8(hipStream_t st, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           uint16_t* out, int K, int N, int group, bool f16)
{
  const int Kw = K / 4;
  const size_t total = (size_t)N * (size_t)Kw;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536 * 4) { blocks = 65536 * 4; }
  const dim3 grid((unsigned)blocks), block(256);
  uint2* o = reinterpret_cast<uint2*>(out);
  if (group == 32) {
    return f16 ? launch_kernel(dequant_w8_kernel<3, true>, grid, block, 0, st, w, scales, biases, o, Kw, total)
               : launch_kernel(dequant_w8_kernel<3>, grid, block, 0, st, w, scales, biases, o, Kw, total);
  }
  return f16 ? launch_kernel(dequant_w8_kernel<4, true>, grid, block, 0, st, w, scales, biases, o, Kw, total)
             : launch_kernel(dequant_w8_kernel<4>, grid, block, 0, st, w, scales, biases, o, Kw, total);
}

// 8-bit -> 4-bit requantizer (affine_requant_w8_to_w4_g64, gpu-kernels/metal/quant/affine_dequant.metal:134-186): one
// thread per group of 64.  The group's 64 bytes come in as four 128-bit loads requested together; values are
// v = s8 * q8 + b8 in fp32 (the product is exact), scale = (max - min) / 15 and 1 / scale by IEEE division,
// q4 = round-half-away((v - min) / scale) clamped to 0..15, a constant group gives scale 0 and codes 0.  Stored
// scale / bias: bf16 roundings of scale and min.  A load-time kernel (it builds the half-width copy of an lm_head),
// bound by the 64 + 4 bytes read and 32 + 4 written per group.
__global__ __launch_bounds__(256) void requant_w8_to_w4_kernel(
    const uint4* __restrict__ w8, const uint16_t* __restrict__ s8, const uint16_t* __restrict__ b8,
    uint4* __restrict__ w4, uint16_t* __restrict__ s4, uint16_t* __restrict__ b4, size_t groups)
{
  for (size_t g = (size_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (size_t)gridDim.x * 256) {
    uint4 c[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { c[i] = w8[g * 4 + i]; }
    const float s = bf16_bits_to_f32(s8[g]);
    const float b = bf16_bits_to_f32(b8[g]);
    float v[64];
    float mn = INFINITY, mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t words[4] = {c[i].x, c[i].y, c[i].z, c[i].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float val = fmaf(s, (float)((words[j] >> (8 * k)) & 0xffu), b);
          v[16 * i + 4 * j + k] = val;
          mn = fminf(mn, val);
          mx = fmaxf(mx, val);
        }
      }
    }
    const float scale = (mx - mn) / 15.0f;
    const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
    s4[g] = (uint16_t)f32_to_bf16_bits(scale);
    b4[g] = (uint16_t)f32_to_bf16_bits(mn);
    uint32_t out[8];
#pragma unroll
    for (int wi = 0; wi < 8; ++wi) {
      uint32_t packed = 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float d = v[wi * 8 + i] - mn;
        int q = (int)roundf(d * inv);
        q = q < 0 ? 0 : (q > 15 ? 15 : q);
        packed |= (uint32_t)q << (4 * i);
      }
      out[wi] = packed;
    }
    w4[g * 2] = make_uint4(out[0], out[1], out[2], out[3]);
    w4[g * 2 + 1] = make_uint4(out[4], out[5], out[6], out[7]);
  }
}

hipError_t launch_requant_w8_to_w4(hipStream_t st, const uint32_t* w8, const uint16_t* s8, const uint16_t* b8,
                                   uint32_t* w4, uint16_t* s4, uint16_t* b4, int K, int N)
{
  const size_t groups = (size_t)N * (size_t)(K / 64);
  size_t blocks = (groups + 255) / 256;
  if (blocks > 65536 * 4) { blocks = 65536 * 4; }
  return launch_kernel(requant_w8_to_w4_kernel, dim3((unsigned)blocks), dim3(256), 0, st,
                       reinterpret_cast<const uint4*>(w8), s8, b8, reinterpret_cast<uint4*>(w4), s4, b4, groups);
}

// Dequantizing embedding gather (gpu-kernels/metal/ops/llm_elementwise.metal:1676-1701): out row t
// is the dense expansion of table row ids[t]; the arithmetic is the dequant kernel's, so a
// gathered row is bit-identical to that row of the dense table.  One thread per packed word.
// A row whose id is outside [0, vocab) is filled with zeros.
__global__ __launch_bounds__(256) void embed_gather_w4g64_kernel(
    const int* __restrict__ ids, const uint32_t* __restrict__ w, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, uint4* __restrict__ out, int Hw, int vocab, size_t total_words)
{
  const int Hg = Hw >> 3;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total_words; idx += (size_t)gridDim.x * 256) {
    const size_t t = idx / (size_t)Hw;
    const int j = (int)(idx - t * (size_t)Hw);
    const int id = ids[t];
    uint4 o = make_uint4(0, 0, 0, 0);
    if (id >= 0 && id < vocab) {
      const size_t g = (size_t)id * (size_t)Hg + (size_t)(j >> 3);
      const float s = bf16_bits_to_f32(scales[g]);
      const float b = bf16_bits_to_f32(biases[g]);
      const uint32_t p = w[(size_t)id * (size_t)Hw + (size_t)j];
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) { v[i] = fmaf(s, (float)((p >> (4 * i)) & 0xfu), b); }
      o.x = pack_bf16x2(v[0], v[1]);
      o.y = pack_bf16x2(v[2], v[3]);
      o.z = pack_bf16x2(v[4], v[5]);
      o.w = pack_bf16x2(v[6], v[7]);
    }
    out[idx] = o;
  }
}

hipError_t launch_embed_gather(hipStream_t st, const int* ids, const uint32_t* w, const uint16_t* scales,
                               const uint16_t* biases, uint16_t* out, int H, int T, int vocab)
{
  const int Hw = H / 8;
  const size_t total = (size_t)T * (size_t)Hw;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536 * 4) { blocks = 65536 * 4; }
  if (blocks == 0) { return hipSuccess; }
  return launch_kernel(embed_gather_w4g64_kernel, dim3((unsigned)blocks), dim3(256), 0, st, ids, w, scales, biases,
                       reinterpret_cast<uint4*>(out), Hw, vocab, total);
}

// One thread per group, as the reference's packer (affine_quant_impl<BITS, GROUP>,
// gpu-kernels/metal/quant/affine_dequant.metal:243-301: 4 or 8 bits, groups of 64 or 32): min/max, optional
// clip toward the midpoint, scale = (mx-mn)/(2^BITS - 1), q = clamp(round((v-mn)/scale)),
// round half away from zero, scale and min emitted as IEEE F16.  F16SRC: the source matrix is binary16 (the
// reference's quantizer runs the VPIPE_ELT = half build, generative-models/quantize/affine-quantizer.cc:25), else bf16.
template <int BITS, int GROUP, bool F16SRC>
__global__ __launch_bounds__(64) void quantize_kernel(
    const uint16_t* __restrict__ src, uint32_t* __restrict__ w, uint16_t* __restrict__ s_f16,
    uint16_t* __restrict__ b_f16, int K, int N, float clip)
{
  constexpr int VPW = 32 / BITS;             // values per word
  constexpr int WPG = GROUP / VPW;           // words per group
  constexpr int QMAX = (1 << BITS) - 1;
  const int Kg = K / GROUP;
  const int grp = blockIdx.x * 64 + threadIdx.x;
  const int n = blockIdx.y;
  if (grp >= Kg || n >= N) { return; }
  const uint16_t* xp = src + (size_t)n * K + (size_t)grp * GROUP;
  float v[GROUP];
  float mn = INFINITY, mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < GROUP / 8; ++i) {
    const uint4 d = reinterpret_cast<const uint4*>(xp)[i];
    const uint32_t dd[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[i * 8 + 2 * j] = elt_lo_to_f32<F16SRC>(dd[j]);
      v[i * 8 + 2 * j + 1] = elt_hi_to_f32<F16SRC>(dd[j]);
    }
  }
#pragma unroll
  for (int i = 0; i < GROUP; ++i) {
    mn = fminf(mn, v[i]);
    mx = fmaxf(mx, v[i]);
  }
  if (clip < 1.0f) {
    // every product rounded on its own (no fused multiply-add), as the expressions read; the CPU restatement
    // is built the same way
#pragma clang fp contract(off)
    const float mid = 0.5f * (mn + mx);
    mn = mid + (mn - mid) * clip;
    mx = mid + (mx - mid) * clip;
  }
  const float scale = (mx - mn) / (float)QMAX;
  const float inv = (scale > 0.0f) ? 1.0f / scale : 0.0f;
  s_f16[(size_t)n * Kg + grp] = __builtin_bit_cast(uint16_t, (_Float16)scale);
  b_f16[(size_t)n * Kg + grp] = __builtin_bit_cast(uint16_t, (_Float16)mn);
  uint32_t* wp = w + (size_t)n * (K / VPW) + (size_t)grp * WPG;
#pragma unroll
  for (int wi = 0; wi < WPG; ++wi) {
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < VPW; ++i) {
      int q = (int)roundf((v[wi * VPW + i] - mn) * inv);
      q = q < 0 ? 0 : (q > QMAX ? QMAX : q);
      packed |= (uint32_t)q << (BITS * i);
    }
    wp[wi] = packed;
  }
}

hipError_t launch_quantize(hipStream_t st, const uint16_t* src, uint32_t* w, uint16_t* s_f16,
                           uint16_t* b_f16, int K, int N, float clip, int bits, int group, bool f16_src)
{
  const int Kg = K / group;
  const int wpr = K * bits / 32;                 // words per row
  // grid.y carries N; rows beyond 65535 are covered by launching in bands.
  for (int n0 = 0; n0 < N; n0 += 65535) {
    const int rows = (N - n0 < 65535) ? (N - n0) : 65535;
    const dim3 grid((unsigned)((Kg + 63) / 64), (unsigned)rows), block(64);
    const uint16_t* sp = src + (size_t)n0 * K;
    uint32_t* wp = w + (size_t)n0 * wpr;
    uint16_t* ss = s_f16 + (size_t)n0 * Kg;
    uint16_t* bb = b_f16 + (size_t)n0 * Kg;
    hipError_t e = hipErrorInvalidValue;
#define VPQ_QUANT(B, G)                                                                              \
  (f16_src ? launch_kernel(quantize_kernel<B, G, true>, grid, block, 0, st, sp, wp, ss, bb, K, rows, clip) \
           : launch_kernel(quantize_kernel<B, G, false>, grid, block, 0, st, sp, wp, ss, bb, K, rows, clip))
    if (bits == 4 && group == 64) { e = VPQ_QUANT(4, 64); }
    else if (bits == 4 && group == 32) { e = VPQ_QUANT(4, 32); }
    else if (bits == 8 && group == 64) { e = VPQ_QUANT(8, 64); }
    else if (bits == 8 && group == 32) { e = VPQ_QUANT(8, 32); }
#undef VPQ_QUANT
    if (e != hipSuccess) { return e; }
  }
  return hipSuccess;
}

__global__ __launch_bounds__(256) void f16_to_bf16_kernel(const uint16_t* __restrict__ in,
                                                          uint16_t* __restrict__ out, size_t count)
{
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count;
       i += (size_t)gridDim.x * 256) {
    out[i] = (uint16_t)f32_to_bf16_bits(f16_bits_to_f32(in[i]));
  }
}

hipError_t launch_f16_to_bf16(hipStream_t st, const uint16_t* in, uint16_t* out, size_t count)
{
  size_t blocks = (count + 255) / 256;
  if (blocks > 65536) { blocks = 65536; }
  if (blocks == 0) { return hipSuccess; }
  return launch_kernel(f16_to_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, st, in, out, count);
}

// The load-time gate|up interleave of generative-models/llama3/metal-llama-model.cc:151-188 (done
// there by memcpy on unified memory): out row 2i = a row i, out row 2i+1 = b row i.  One unit
// (a dword, or a halfword where a scale row is not a multiple of 4 bytes) per thread.
template <typename T>
__global__ __launch_bounds__(256) void interleave_rows_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                              T* __restrict__ out, size_t row_units,
                                                              size_t total_units)
{
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total_units; i += (size_t)gridDim.x * 256) {
    const size_t orow = i / row_units, col = i - orow * row_units;
    const T* src = (orow & 1) ? b : a;
    out[i] = src[(orow >> 1) * row_units + col];
  }
}

template <typename T>
static hipError_t interleave_as(hipStream_t st, const void* a, const void* b, void* out, size_t row_bytes, size_t rows)
{
  const size_t row_units = row_bytes / sizeof(T), total = 2 * rows * row_units;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) { blocks = 65536; }
  if (blocks == 0) { return hipSuccess; }
  return launch_kernel(interleave_rows_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, st,
                       reinterpret_cast<const T*>(a), reinterpret_cast<const T*>(b), reinterpret_cast<T*>(out),
                       row_units, total);
}

hipError_t launch_interleave_rows(hipStream_t st, const void* a, const void* b, void* out, size_t row_bytes,
                                  size_t rows)
{
  const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                         reinterpret_cast<uintptr_t>(out) | row_bytes;
  return (bits & 3) == 0 ? interleave_as<uint32_t>(st, a, b, out, row_bytes, rows)
                         : interleave_as<uint16_t>(st, a, b, out, row_bytes, rows);
}

}  // namespace vpq

// QMV, general-shape kernel: one wavefront per output row, fp32 VALU.
// Handles every K % 64 == 0, every N and 1 <= M <= 16; used for shapes the
// MFMA kernel does not take (K not a multiple of 512, N not a multiple of 16)
// and as an independent second implementation in the tests.
//
// Arithmetic: W[n,k] = fma(s, q, b) in fp32 (never rounded to bf16),
// acc += x * W in fp32, wave reduction, one bf16 rounding on store -- the
// semantics of gpu-kernels/metal/quant/affine_qmv.metal:151-174, 228-283.
// With `gate_act` (1 SwiGLU, 2 GEGLU) the rows are an interleaved gate|up pack: wavefronts 2j and 2j+1 of a
// workgroup hold a feature's gate and up sums, the odd one hands its sum over through LDS and
// the even one stores act(gate) * up into y[M, N/2] (affine_qmv.metal:816-906, 1356-1430).
#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

// GS: log2 of the quantization group (6, or 5 for the group-32 packs); SO: scale-only (Q4_0) pack, the
// bias is -8 * scale and `biases` is never read (affine_qmv.metal:305-342, 252-256).
template <int MT, bool F32OUT, int GS = 6, bool SO = false, bool F16 = false>
__global__ __launch_bounds__(256) void qmv_simple_kernel(
    const uint32_t* __restrict__ w, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ x, void* __restrict__ y,
    const uint16_t* __restrict__ residual, int K, int N, int M, int gate_act)
{
  __shared__ float up_sum[4][MT];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int n_raw = blockIdx.x * 4 + wave;
  const bool live = n_raw < N;            // wave-uniform
  const int n = live ? n_raw : N - 1;     // idle wavefronts redo the last row and store nothing
  const int Kw = K >> 3, Kg = K >> GS;
  const uint32_t* wrow = w + (size_t)n * Kw;
  const uint16_t* srow = scales + (size_t)n * Kg;
  const uint16_t* brow = SO ? nullptr : biases + (size_t)n * Kg;

  for (int m0 = 0; m0 < M; m0 += MT) {
    float acc[MT];
#pragma unroll
    for (int mm = 0; mm < MT; ++mm) { acc[mm] = 0.0f; }
    // Each lane takes 32 consecutive k (one 128-bit load of codes, half a group of 64).
    for (int k0 = lane * 32; k0 < K; k0 += kWave * 32) {
      const uint4 c4 = *reinterpret_cast<const uint4*>(wrow + (k0 >> 3));
      const uint32_t codes[4] = {c4.x, c4.y, c4.z, c4.w};
      const float s = elt_bits_to_f32<F16>(srow[k0 >> GS]);
      const float b = SO ? -8.0f * s : elt_bits_to_f32<F16>(brow[k0 >> GS]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float wv[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) { wv[j] = fmaf(s, (float)((codes[i] >> (4 * j)) & 0xfu), b); }
#pragma unroll
        for (int mm = 0; mm < MT; ++mm) {
          const int row = (m0 + mm < M) ? (m0 + mm) : (M - 1);
          const uint4 x4 = *reinterpret_cast<const uint4*>(x + (size_t)row * K + k0 + 8 * i);
          const uint32_t xd[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc[mm] = fmaf(elt_lo_to_f32<F16>(xd[j]), wv[2 * j], acc[mm]);
            acc[mm] = fmaf(elt_hi_to_f32<F16>(xd[j]), wv[2 * j + 1], acc[mm]);
          }
        }
      }
    }
    if (gate_act == kGateSwiglu || gate_act == kGateGeglu) {
      float total[MT];
#pragma unroll
      for (int mm = 0; mm < MT; ++mm) { total[mm] = wave_sum(acc[mm]); }
      if ((wave & 1) && lane == 0) {
#pragma unroll
        for (int mm = 0; mm < MT; ++mm) { up_sum[wave][mm] = total[mm]; }
      }
      __syncthreads();
      if (!(wave & 1) && lane == 0 && live) {
#pragma unroll
        for (int mm = 0; mm < MT; ++mm) {
          const int row = m0 + mm;
          if (row < M) {
            const float v = gated_f32(gate_act, total[mm], up_sum[wave + 1][mm]);
            const size_t o = (size_t)row * (N >> 1) + (n >> 1);
            if (F32OUT) {
              reinterpret_cast<float*>(y)[o] = v;
            } else {
              reinterpret_cast<uint16_t*>(y)[o] = (uint16_t)f32_to_elt_bits<F16>(v);
            }
          }
        }
      }
      __syncthreads();   // up_sum is rewritten by the next batch of rows
      continue;
    }
#pragma unroll
    for (int mm = 0; mm < MT; ++mm) {
      const float total = wave_sum(acc[mm]);
      const int row = m0 + mm;
      if (lane == 0 && row < M && live) {
        const size_t o = (size_t)row * N + n;
        if (F32OUT) {
          reinterpret_cast<float*>(y)[o] = total;
        } else {
          uint32_t v = f32_to_elt_bits<F16>(total);
          if (gate_act == kStoreGeluMul) {          // `residual` is the multiplier, one value per output feature
            v = f32_to_elt_bits<F16>(gelu_mul_f32(elt_bits_to_f32<F16>(v), elt_bits_to_f32<F16>(residual[n])));
          } else if (residual != nullptr) {
            v = f32_to_elt_bits<F16>(elt_bits_to_f32<F16>(v) + elt_bits_to_f32<F16>(residual[o]));
          }
          reinterpret_cast<uint16_t*>(y)[o] = (uint16_t)v;
        }
      }
    }
  }
}

hipError_t launch_qmv_simple(hipStream_t st, const QmvArgs& a)
{
  const dim3 grid((unsigned)((a.N + 3) / 4)), block(256);
#define VPQ_LAUNCH(MT, F32)                                                                    \
  launch_kernel(qmv_simple_kernel<MT, F32>, grid, block, 0, st, a.w, a.scales, a.biases, a.x, a.y, \
                a.residual, a.K, a.N, a.M, a.gate_act)
  if (a.M == 1) { return a.y_f32 ? VPQ_LAUNCH(1, true) : VPQ_LAUNCH(1, false); }
  return a.y_f32 ? VPQ_LAUNCH(4, true) : VPQ_LAUNCH(4, false);
#undef VPQ_LAUNCH
}

// IEEE binary16 elements (x, scales, biases, y, residual): the reference's VPIPE_ELT = half build of
// affine_qmv_w4g64[_add] and the gated forms.
hipError_t launch_qmv_simple_f16(hipStream_t st, const QmvArgs& a)
{
  const dim3 grid((unsigned)((a.N + 3) / 4)), block(256);
#define VPQ_LAUNCH(MT, F32)                                                                                   \
  launch_kernel(qmv_simple_kernel<MT, F32, 6, false, true>, grid, block, 0, st, a.w, a.scales, a.biases, a.x, a.y, \
                a.residual, a.K, a.N, a.M, a.gate_act)
  if (a.M == 1) { return a.y_f32 ? VPQ_LAUNCH(1, true) : VPQ_LAUNCH(1, false); }
  return a.y_f32 ? VPQ_LAUNCH(4, true) : VPQ_LAUNCH(4, false);
#undef VPQ_LAUNCH
}

hipError_t launch_qmv_simple_g32(hipStream_t st, const QmvArgs& a, bool scale_only)
{
  const dim3 grid((unsigned)((a.N + 3) / 4)), block(256);
#define VPQ_LAUNCH(MT, F32, SO)                                                                       \
  launch_kernel(qmv_simple_kernel<MT, F32, 5, SO>, grid, block, 0, st, a.w, a.scales, a.biases, a.x, a.y, \
                a.residual, a.K, a.N, a.M, a.gate_act)
#define VPQ_LAUNCH_SO(MT, F32) (scale_only ? VPQ_LAUNCH(MT, F32, true) : VPQ_LAUNCH(MT, F32, false))
  if (a.M == 1) { return a.y_f32 ? VPQ_LAUNCH_SO(1, true) : VPQ_LAUNCH_SO(1, false); }
  return a.y_f32 ? VPQ_LAUNCH_SO(4, true) : VPQ_LAUNCH_SO(4, false);
#undef VPQ_LAUNCH_SO
#undef VPQ_LAUNCH
}

// 8-bit twin (affine_qmv_w8g64, gpu-kernels/metal/quant/affine_qmv.metal:3034-3050): one byte per
// value.  Each lane takes 16 consecutive k (one 128-bit load of codes, a quarter of a group) per
// pass over the row; otherwise the kernel above: W = fma(s, q, b) in fp32, never rounded.  GS: log2 of the group
// (6, or 5 for affine_qmv_w8g32, :3053-3069).  store == kStoreGeluMul: affine_qmv_gelu_mul_w8g64 (:789-805),
// `residual` is then the multiplier [N].
template <int MT, bool F32OUT, int GS = 6>
__global__ __launch_bounds__(256) void qmv_simple8_kernel(
    const uint32_t* __restrict__ w, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ x, void* __restrict__ y,
    const uint16_t* __restrict__ residual, int K, int N, int M, int store)
{
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + wave;
  if (n >= N) { return; }  // wave-uniform; no barrier in this kernel
  const int Kw = K >> 2, Kg = K >> GS;
  const uint32_t* wrow = w + (size_t)n * Kw;
  const uint16_t* srow = scales + (size_t)n * Kg;
  const uint16_t* brow = biases + (size_t)n * Kg;

  for (int m0 = 0; m0 < M; m0 += MT) {
    float acc[MT];
#pragma unroll
    for (int mm = 0; mm < MT; ++mm) { acc[mm] = 0.0f; }
    for (int k0 = lane * 16; k0 < K; k0 += kWave * 16) {
      const uint4 c4 = *reinterpret_cast<const uint4*>(wrow + (k0 >> 2));
      const uint32_t codes[4] = {c4.x, c4.y, c4.z, c4.w};
      const float s = bf16_bits_to_f32(srow[k0 >> GS]);
      const float b = bf16_bits_to_f32(brow[k0 >> GS]);
      float wv[16];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) { wv[4 * i + j] = fmaf(s, (float)((codes[i] >> (8 * j)) & 0xffu), b); }
      }
#pragma unroll
      for (int mm = 0; mm < MT; ++mm) {
        const int row = (m0 + mm < M) ? (m0 + mm) : (M - 1);
        const uint4* xp = reinterpret_cast<const uint4*>(x + (size_t)row * K + k0);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint4 x4 = xp[h];
          const uint32_t xd[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc[mm] = fmaf(bf16_lo_to_f32(xd[j]), wv[8 * h + 2 * j], acc[mm]);
            acc[mm] = fmaf(bf16_hi_to_f32(xd[j]), wv[8 * h + 2 * j + 1], acc[mm]);
          }
        }
      }
    }
#pragma unroll
    for (int mm = 0; mm < MT; ++mm) {
      const float total = wave_sum(acc[mm]);
      const int row = m0 + mm;
      if (lane == 0 && row < M) {
        const size_t o = (size_t)row * N + n;
        if (F32OUT) {
          reinterpret_cast<float*>(y)[o] = total;
        } else {
          uint32_t v = f32_to_bf16_bits(total);
          if (store == kStoreGeluMul) {          // `residual` is the multiplier, one value per output feature
            v = f32_to_bf16_bits(gelu_mul_f32(bf16_bits_to_f32(v), bf16_bits_to_f32(residual[n])));
          } else if (residual != nullptr) {
            v = f32_to_bf16_bits(bf16_bits_to_f32(v) + bf16_bits_to_f32(residual[o]));
          }
          reinterpret_cast<uint16_t*>(y)[o] = (uint16_t)v;
        }
      }
    }
  }
}

// 8-bit gated and gathered forms (affine_qmv_swiglu_w8g64 / affine_qmv_geglu_w8g64,
// gpu-kernels/metal/quant/affine_qmv.metal:3140-3178; affine_gather_qmv_swiglu_w8g64 :962-990,
// affine_gather_qmv_geglu_w8g64 :1524-1552, affine_gather_down_qmv_w8g64 :1295-1322).  One wavefront
// per output: a plain row, or (GATED) the gate and the up row of a feature of the interleaved pack,
// whose two sums meet in that wavefront's registers.  blockIdx.y is the row of x, or with pair_eid
// the (token, expert) pair: the pack is then the slab pair_eid[pair] of a batch [E, N, K/4], x row
// pair / x_div, y row pair; an id outside [0, n_experts) gives zeros.
template <bool GATED>
__global__ __launch_bounds__(256) void qmv_rows8_kernel(
    const uint32_t* __restrict__ w, const uint16_t* __restrict__ scales, const uint16_t* __restrict__ biases,
    const uint16_t* __restrict__ x, uint16_t* __restrict__ y, int K, int N, int gate_act,
    const int* __restrict__ pair_eid, int x_div, int n_experts)
{
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int outs = GATED ? (N >> 1) : N;
  const int o = blockIdx.x * 4 + wave;
  if (o >= outs) { return; }  // wave-uniform; no barrier in this kernel
  const int m = blockIdx.y;
  const int Kw = K >> 2, Kg = K >> 6;
  int xrow = m;
  if (pair_eid != nullptr) {
    const int e = pair_eid[m];
    if (e < 0 || e >= n_experts) {
      if (lane == 0) { y[(size_t)m * outs + o] = 0; }
      return;
    }
    w += (size_t)e * (size_t)N * Kw;
    scales += (size_t)e * (size_t)N * Kg;
    biases += (size_t)e * (size_t)N * Kg;
    xrow = m / x_div;
  }
  const uint16_t* xr = x + (size_t)xrow * K;
  constexpr int R = GATED ? 2 : 1;
  const int n0 = GATED ? 2 * o : o;
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) { acc[r] = 0.0f; }
  for (int k0 = lane * 16; k0 < K; k0 += kWave * 16) {
    const uint4* xp = reinterpret_cast<const uint4*>(xr + k0);
    float xv[16];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint4 x4 = xp[h];
      const uint32_t xd[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        xv[8 * h + 2 * j] = bf16_lo_to_f32(xd[j]);
        xv[8 * h + 2 * j + 1] = bf16_hi_to_f32(xd[j]);
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const size_t n = (size_t)(n0 + r);
      const uint4 c4 = *reinterpret_cast<const uint4*>(w + n * Kw + (k0 >> 2));
      const uint32_t codes[4] = {c4.x, c4.y, c4.z, c4.w};
      const float s = bf16_bits_to_f32(scales[n * Kg + (k0 >> 6)]);
      const float b = bf16_bits_to_f32(biases[n * Kg + (k0 >> 6)]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[r] = fmaf(xv[4 * i + j], fmaf(s, (float)((codes[i] >> (8 * j)) & 0xffu), b), acc[r]);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) { acc[r] = wave_sum(acc[r]); }
  if (lane == 0) {
    const float v = GATED ? gated_f32(gate_act, acc[0], acc[R - 1])
                          : (gate_act == kStoreSigmoid ? 1.0f / (1.0f + __expf(-acc[0])) : acc[0]);
    y[(size_t)m * outs + o] = (uint16_t)f32_to_bf16_bits(v);
  }
}

hipError_t launch_qmv_rows8(hipStream_t st, const QmvArgs& a, int rows, const int* pair_eid, int x_div, int n_experts)
{
  const bool gated = a.gate_act == kGateSwiglu || a.gate_act == kGateGeglu;
  const int outs = gated ? a.N / 2 : a.N;
  const dim3 grid((unsigned)((outs + 3) / 4), (unsigned)rows), block(256);
  uint16_t* y = static_cast<uint16_t*>(a.y);
  if (a.gate_act == kStoreSigmoid) {
    return launch_kernel(qmv_rows8_kernel<false>, grid, block, 0, st, a.w, a.scales, a.biases, a.x, y, a.K, a.N, a.gate_act,
                         pair_eid, x_div, n_experts);
  }
  return a.gate_act ? launch_kernel(qmv_rows8_kernel<true>, grid, block, 0, st, a.w, a.scales, a.biases, a.x, y, a.K, a.N,
                                    a.gate_act, pair_eid, x_div, n_experts)
                    : launch_kernel(qmv_rows8_kernel<false>, grid, block, 0, st, a.w, a.scales, a.biases, a.x, y, a.K, a.N, 0,
                                    pair_eid, x_div, n_experts);
}

// Expert-sorted form for a few rows per expert (gpu-kernels/metal/quant/affine_qmv.metal:2551-2719,
// `affine_grouped_swiglu_w8g64`, `affine_grouped_down_w8g64`, MAXM = 2): blockIdx.y is a tile of two slots owned by
// expert tile2e[tile] (outside [0, n_experts): unused tile, nothing written); slot s is live where srow[s] >= 0 and
// reads x row srow[s] (X_FROM_SROW: the gate|up projection gathers the hidden rows) or row s (the down projection
// reads the sorted activations), and writes y row s.  A wavefront reads its row (or gate and up rows) of the
// expert's slab once for both slots; per slot the arithmetic is qmv_rows8_kernel's, term for term.
template <bool GATED, bool X_FROM_SROW>
__global__ __launch_bounds__(256) void qmv_rows8_sorted_kernel(
    const uint32_t* __restrict__ w, const uint16_t* __restrict__ scales, const uint16_t* __restrict__ biases,
    const uint16_t* __restrict__ x, uint16_t* __restrict__ y, int K, int N, int gate_act,
    const int* __restrict__ tile2e, const int* __restrict__ srow, int n_experts)
{
  constexpr int MT = 2;                       // slots per tile
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int outs = GATED ? (N >> 1) : N;
  const int o = blockIdx.x * 4 + wave;
  if (o >= outs) { return; }  // wave-uniform; no barrier in this kernel
  const int t = blockIdx.y;
  const int e = tile2e[t];
  if (e < 0 || e >= n_experts) { return; }
  const int Kw = K >> 2, Kg = K >> 6;
  w += (size_t)e * (size_t)N * Kw;
  scales += (size_t)e * (size_t)N * Kg;
  biases += (size_t)e * (size_t)N * Kg;
  const uint16_t* xr[MT];
  bool live[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int slot = t * MT + m;
    const int rr = srow[slot];
    live[m] = rr >= 0;
    xr[m] = x + (size_t)(X_FROM_SROW ? (rr >= 0 ? rr : 0) : slot) * K;
  }
  constexpr int R = GATED ? 2 : 1;
  const int n0 = GATED ? 2 * o : o;
  float acc[MT][R];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
#pragma unroll
    for (int r = 0; r < R; ++r) { acc[m][r] = 0.0f; }
  }
  for (int k0 = lane * 16; k0 < K; k0 += kWave * 16) {
    float xv[MT][16];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const uint4* xp = reinterpret_cast<const uint4*>(xr[m] + k0);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint4 x4 = xp[h];
        const uint32_t xd[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          xv[m][8 * h + 2 * j] = bf16_lo_to_f32(xd[j]);
          xv[m][8 * h + 2 * j + 1] = bf16_hi_to_f32(xd[j]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const size_t n = (size_t)(n0 + r);
      const uint4 c4 = *reinterpret_cast<const uint4*>(w + n * Kw + (k0 >> 2));
      const uint32_t codes[4] = {c4.x, c4.y, c4.z, c4.w};
      const float s = bf16_bits_to_f32(scales[n * Kg + (k0 >> 6)]);
      const float b = bf16_bits_to_f32(biases[n * Kg + (k0 >> 6)]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float wv = fmaf(s, (float)((codes[i] >> (8 * j)) & 0xffu), b);
#pragma unroll
          for (int m = 0; m < MT; ++m) { acc[m][r] = fmaf(xv[m][4 * i + j], wv, acc[m][r]); }
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MT; ++m) {
#pragma unroll
    for (int r = 0; r < R; ++r) { acc[m][r] = wave_sum(acc[m][r]); }
  }
  if (lane == 0) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (!live[m]) { continue; }
      const float v = GATED ? gated_f32(gate_act, acc[m][0], acc[m][R - 1]) : acc[m][0];
      y[(size_t)(t * MT + m) * outs + o] = (uint16_t)f32_to_bf16_bits(v);
    }
  }
}

// a.gate_act != 0: the gate|up projection (x rows through srow); else the down projection (x in slot order).
hipError_t launch_qmv_rows8_sorted(hipStream_t st, const QmvArgs& a, const int* tile2e, const int* srow, int tiles,
                                   int n_experts)
{
  const int outs = a.gate_act ? a.N / 2 : a.N;
  const dim3 grid((unsigned)((outs + 3) / 4), (unsigned)tiles), block(256);
  uint16_t* y = static_cast<uint16_t*>(a.y);
  return a.gate_act ? launch_kernel(qmv_rows8_sorted_kernel<true, true>, grid, block, 0, st, a.w, a.scales, a.biases, a.x, y,
                                    a.K, a.N, a.gate_act, tile2e, srow, n_experts)
                    : launch_kernel(qmv_rows8_sorted_kernel<false, false>, grid, block, 0, st, a.w, a.scales, a.biases, a.x, y,
                                    a.K, a.N, 0, tile2e, srow, n_experts);
}

// Mixed-width fused gate/up (affine_gather_qmv_swiglu_w4w8g64 / _w8w4g64,
// gpu-kernels/metal/quant/affine_qmv.metal:991-1260): gate and up are SEPARATE packs [E, ffn, ...], each at
// its own width (4 or 8 bits) as a per-tensor quantizer left them; a wavefront contracts the gate row and
// the up row of one feature with x and stores act(gate) * up.  Same bytes off DRAM as a uniform layer of
// those widths, no widened copy.  blockIdx.y: the pair (pair_eid) or the row of x.
template <int BITS>
__device__ __forceinline__ float row_dot_wave(const uint32_t* __restrict__ wrow, const uint16_t* __restrict__ srow,
                                              const uint16_t* __restrict__ brow, const uint16_t* __restrict__ xr, int K,
                                              int lane)
{
  constexpr int VPL = BITS == 4 ? 32 : 16;        // values per lane and pass: one 128-bit load of codes
  float acc = 0.0f;
  for (int k0 = lane * VPL; k0 < K; k0 += kWave * VPL) {
    const uint4 c4 = *reinterpret_cast<const uint4*>(wrow + (BITS == 4 ? (k0 >> 3) : (k0 >> 2)));
    const uint32_t codes[4] = {c4.x, c4.y, c4.z, c4.w};
    const float s = bf16_bits_to_f32(srow[k0 >> 6]);
    const float b = bf16_bits_to_f32(brow[k0 >> 6]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      constexpr int PER = BITS == 4 ? 8 : 4;      // values per code word
      const uint4* xp = reinterpret_cast<const uint4*>(xr + k0 + PER * i);
      if (BITS == 4) {
        const uint4 x4 = xp[0];
        const uint32_t xd[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc = fmaf(bf16_lo_to_f32(xd[j]), fmaf(s, (float)((codes[i] >> (8 * j)) & 0xfu), b), acc);
          acc = fmaf(bf16_hi_to_f32(xd[j]), fmaf(s, (float)((codes[i] >> (8 * j + 4)) & 0xfu), b), acc);
        }
      } else {
        const uint2 x2 = *reinterpret_cast<const uint2*>(xr + k0 + 4 * i);
        acc = fmaf(bf16_lo_to_f32(x2.x), fmaf(s, (float)(codes[i] & 0xffu), b), acc);
        acc = fmaf(bf16_hi_to_f32(x2.x), fmaf(s, (float)((codes[i] >> 8) & 0xffu), b), acc);
        acc = fmaf(bf16_lo_to_f32(x2.y), fmaf(s, (float)((codes[i] >> 16) & 0xffu), b), acc);
        acc = fmaf(bf16_hi_to_f32(x2.y), fmaf(s, (float)(codes[i] >> 24), b), acc);
      }
    }
  }
  return wave_sum(acc);
}

template <int GB, int UB>
__global__ __launch_bounds__(256) void qmv_split_gate_up_kernel(
    const uint32_t* __restrict__ wg, const uint16_t* __restrict__ sg, const uint16_t* __restrict__ bg,
    const uint32_t* __restrict__ wu, const uint16_t* __restrict__ su, const uint16_t* __restrict__ bu,
    const uint16_t* __restrict__ x, uint16_t* __restrict__ y, int K, int F, int gate_act,
    const int* __restrict__ pair_eid, int x_div, int n_experts)
{
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int f = blockIdx.x * 4 + wave;
  if (f >= F) { return; }  // wave-uniform; no barrier in this kernel
  const int m = blockIdx.y;
  const int Kg = K >> 6;
  const size_t gw = (size_t)(K >> (GB == 4 ? 3 : 2)), uw = (size_t)(K >> (UB == 4 ? 3 : 2));   // words per row
  int xrow = m;
  size_t e = 0;
  if (pair_eid != nullptr) {
    const int id = pair_eid[m];
    if (id < 0 || id >= n_experts) {
      if (lane == 0) { y[(size_t)m * F + f] = 0; }
      return;
    }
    e = (size_t)id;
    xrow = m / x_div;
  }
  const size_t row = e * (size_t)F + (size_t)f;
  const uint16_t* xr = x + (size_t)xrow * K;
  const float g = row_dot_wave<GB>(wg + row * gw, sg + row * Kg, bg + row * Kg, xr, K, lane);
  const float u = row_dot_wave<UB>(wu + row * uw, su + row * Kg, bu + row * Kg, xr, K, lane);
  if (lane == 0) { y[(size_t)m * F + f] = (uint16_t)f32_to_bf16_bits(gated_f32(gate_act, g, u)); }
}

hipError_t launch_qmv_split_gate_up(hipStream_t st, const SplitGateUp& a)
{
  const dim3 grid((unsigned)((a.F + 3) / 4), (unsigned)a.rows), block(256);
#define VPQ_SPLIT(GB, UB)                                                                                       \
  launch_kernel(qmv_split_gate_up_kernel<GB, UB>, grid, block, 0, st, a.wg, a.sg, a.bg, a.wu, a.su, a.bu, a.x, a.y, a.K, \
                a.F, a.gate_act, a.pair_eid, a.x_div, a.n_experts)
  if (a.gate_bits == 4) { return a.up_bits == 4 ? VPQ_SPLIT(4, 4) : VPQ_SPLIT(4, 8); }
  return a.up_bits == 4 ? VPQ_SPLIT(8, 4) : VPQ_SPLIT(8, 8);
#undef VPQ_SPLIT
}

hipError_t launch_qmv_simple8(hipStream_t st, const QmvArgs& a, int group)
{
  const dim3 grid((unsigned)((a.N + 3) / 4)), block(256);
#define VPQ_LAUNCH8(MT, F32, GS)                                                                    \
  launch_kernel(qmv_simple8_kernel<MT, F32, GS>, grid, block, 0, st, a.w, a.scales, a.biases, a.x, a.y, \
                a.residual, a.K, a.N, a.M, a.gate_act)
  if (group == 32) {
    if (a.M == 1) { return a.y_f32 ? VPQ_LAUNCH8(1, true, 5) : VPQ_LAUNCH8(1, false, 5); }
    return a.y_f32 ? VPQ_LAUNCH8(4, true, 5) : VPQ_LAUNCH8(4, false, 5);
  }
  if (a.M == 1) { return a.y_f32 ? VPQ_LAUNCH8(1, true, 6) : VPQ_LAUNCH8(1, false, 6); }
  return a.y_f32 ? VPQ_LAUNCH8(4, true, 6) : VPQ_LAUNCH8(4, false, 6);
#undef VPQ_LAUNCH8
}

}  // namespace vpq

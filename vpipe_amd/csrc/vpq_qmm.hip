// QMM: y[M,N] = x[M,K] . bf16(W)^T on bf16 MFMA with fp32 accumulation.
//
// One workgroup (4 wavefronts, 2x2) owns a 128x128 tile of y.  Per 64-wide K
// step (= one quantization group, so one scale/bias per weight row per step):
//   x tile  [128,64] bf16   global -> registers -> LDS
//   W tile  [128,64] codes  global -> registers -> fp32 fma(s,q,b) -> bf16 RNE -> LDS
// The dequantized value is bf16_rne(fp32(s*q+b)), the tile arithmetic of
// gpu-kernels/metal/quant/affine_qmm_steel.metal:78-96 (Compute=float) and
// affine_qmm_mma.metal:96-104.  LDS is double buffered: while the MFMAs consume
// stage s, the loads of stage s+1 are in flight and are written to the other
// buffer before the single barrier of the step.
// A LoRA adds ceil(r/64) dense steps over t[M,r] and B[N,r] into the same
// accumulators before the one store (gpu-kernels/metal/gemm/dense_gemm_mma.metal:
// 297-348).  The same kernel with a dense B and the scaled epilogue computes the
// adapter's first factor t = bf16(alpha * bf16(x . A^T)) (dense_gemm_mma.metal:227-273).
#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDK = BK + 8;  // padded LDS row (bf16 elements): 144 bytes, keeps b128 reads spread over banks
constexpr int kThreads = 256;
constexpr int kStageElems = (BM + BN) * LDK;
constexpr int kLdsBytes = 2 * kStageElems * 2;

struct GemmParams {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  const uint16_t* b_dense;
  const uint16_t* x;
  uint16_t* y;
  const uint16_t* lora_t;
  const uint16_t* lora_b;
  int K, N, M, r;
  int tiles_m, tiles_n;
  float out_scale;
};

struct Stage {
  uint4 xa[4];   // x (or t) tile slice of this thread
  uint4 wb[4];   // dense B slice, or wb[0] = 32 packed codes
  float s, b;    // scale / bias of this thread's weight row for the step
};

}  // namespace

template <bool QUANT_B, bool SCALED_EPI>
__global__ __launch_bounds__(kThreads) void gemm_kernel(const GemmParams p)
{
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // Consecutive workgroups walk M first: they share one weight tile.
  const int tile = blockIdx.x;
  const int tm = tile % p.tiles_m;
  const int tn = tile / p.tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;

  const int KT = p.K / BK;
  const int RT = (p.lora_t != nullptr) ? (p.r + BK - 1) / BK : 0;
  const int nsteps = KT + RT;

  // Thread -> tile slice maps.
  const int xr = tid >> 3;          // + 32*i : row of the x tile
  const int xc = (tid & 7) * 8;     // first k (element) of the 16-byte piece
  const int qrow = tid >> 1;        // weight row for the packed path
  const int qhalf = tid & 1;        // which 32 of the 64 k

  int xrow_g[4];                    // global x rows (clamped: rows past M are never stored)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = m0 + xr + 32 * i;
    xrow_g[i] = r < p.M ? r : p.M - 1;
  }
  int brow_g[4];                    // global B rows for the dense path
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = n0 + xr + 32 * i;
    brow_g[i] = r < p.N ? r : p.N - 1;
  }
  const int qrow_g = (n0 + qrow < p.N) ? (n0 + qrow) : (p.N - 1);
  const int Kw = p.K >> 3, Kg = p.K >> 6;

  auto load_stage = [&](int s, Stage& st) {
    if (s < KT) {
      const int k0 = s * BK;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        st.xa[i] = *reinterpret_cast<const uint4*>(p.x + (size_t)xrow_g[i] * p.K + k0 + xc);
      }
      if (QUANT_B) {
        st.wb[0] = *reinterpret_cast<const uint4*>(p.w + (size_t)qrow_g * Kw + (k0 >> 3) + qhalf * 4);
        st.s = bf16_bits_to_f32(p.scales[(size_t)qrow_g * Kg + s]);
        st.b = bf16_bits_to_f32(p.biases[(size_t)qrow_g * Kg + s]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          st.wb[i] = *reinterpret_cast<const uint4*>(p.b_dense + (size_t)brow_g[i] * p.K + k0 + xc);
        }
      }
    } else {
      // LoRA step: contract t[M,r] with B[N,r]; k past r is zero on both sides.
      const int k0 = (s - KT) * BK;
      const bool in = (k0 + xc) < p.r;
      const uint4 z = make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        st.xa[i] = in ? *reinterpret_cast<const uint4*>(p.lora_t + (size_t)xrow_g[i] * p.r + k0 + xc) : z;
        st.wb[i] = in ? *reinterpret_cast<const uint4*>(p.lora_b + (size_t)brow_g[i] * p.r + k0 + xc) : z;
      }
    }
  };

  auto store_stage = [&](int s, const Stage& st, int buf) {
    uint16_t* As = lds + buf * kStageElems;
    uint16_t* Bs = As + BM * LDK;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<uint4*>(As + (xr + 32 * i) * LDK + xc) = st.xa[i];
    }
    if (QUANT_B && s < KT) {
      const uint32_t codes[4] = {st.wb[0].x, st.wb[0].y, st.wb[0].z, st.wb[0].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) { v[j] = fmaf(st.s, (float)((codes[i] >> (4 * j)) & 0xfu), st.b); }
        uint4 o;
        o.x = pack_bf16x2(v[0], v[1]);
        o.y = pack_bf16x2(v[2], v[3]);
        o.z = pack_bf16x2(v[4], v[5]);
        o.w = pack_bf16x2(v[6], v[7]);
        *reinterpret_cast<uint4*>(Bs + qrow * LDK + qhalf * 32 + i * 8) = o;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *reinterpret_cast<uint4*>(Bs + (xr + 32 * i) * LDK + xc) = st.wb[i];
      }
    }
  };

  // acc[jt][it]: D[i = n within 16][j = m within 16]; lane holds m = lane%16,
  // n = 4*(lane/16) + reg.
  floatx4 acc[4][4];
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) {
#pragma unroll
    for (int it = 0; it < 4; ++it) { acc[jt][it] = floatx4{0.f, 0.f, 0.f, 0.f}; }
  }

  Stage st;
  load_stage(0, st);
  store_stage(0, st, 0);
  __syncthreads();

  const int frag_row = lane & 15;
  const int frag_k = (lane >> 4) * 8;

  for (int s = 0; s < nsteps; ++s) {
    const int buf = s & 1;
    if (s + 1 < nsteps) { load_stage(s + 1, st); }

    const uint16_t* As = lds + buf * kStageElems;
    const uint16_t* Bs = As + BM * LDK;
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      bf16x8 wf[4], xf[4];
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) {
        wf[jt] = *reinterpret_cast<const bf16x8*>(Bs + (wn * 64 + jt * 16 + frag_row) * LDK + kh * 32 + frag_k);
      }
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        xf[it] = *reinterpret_cast<const bf16x8*>(As + (wm * 64 + it * 16 + frag_row) * LDK + kh * 32 + frag_k);
      }
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          acc[jt][it] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[jt], xf[it], acc[jt][it], 0, 0, 0);
        }
      }
    }

    if (s + 1 < nsteps) { store_stage(s + 1, st, buf ^ 1); }
    __syncthreads();
  }

  // Store: each lane owns 4 consecutive n of one row m per (jt, it).
  const bool vec_ok = (p.N & 3) == 0;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int m = m0 + wm * 64 + it * 16 + (lane & 15);
    if (m >= p.M) { continue; }
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) {
      const int n = n0 + wn * 64 + jt * 16 + (lane >> 4) * 4;
      if (n >= p.N) { continue; }
      float v[4] = {acc[jt][it][0], acc[jt][it][1], acc[jt][it][2], acc[jt][it][3]};
      if (SCALED_EPI) {
#pragma unroll
        for (int e = 0; e < 4; ++e) { v[e] = bf16_bits_to_f32(f32_to_bf16_bits(v[e])) * p.out_scale; }
      }
      uint16_t* dst = p.y + (size_t)m * p.N + n;
      if (vec_ok && n + 3 < p.N) {
        uint2 o;
        o.x = pack_bf16x2(v[0], v[1]);
        o.y = pack_bf16x2(v[2], v[3]);
        *reinterpret_cast<uint2*>(dst) = o;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (n + e < p.N) { dst[e] = (uint16_t)f32_to_bf16_bits(v[e]); }
        }
      }
    }
  }
}

hipError_t launch_gemm(hipStream_t st, const GemmArgs& a)
{
  GemmParams p;
  p.w = a.w; p.scales = a.scales; p.biases = a.biases; p.b_dense = a.b_dense;
  p.x = a.x; p.y = a.y; p.lora_t = a.lora_t; p.lora_b = a.lora_b;
  p.K = a.K; p.N = a.N; p.M = a.M; p.r = a.r;
  p.tiles_m = (a.M + BM - 1) / BM;
  p.tiles_n = (a.N + BN - 1) / BN;
  p.out_scale = a.out_scale;
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n)), block(kThreads);

  static bool attr_done[4] = {false, false, false, false};
  auto launch = [&](auto kern, int slot) -> hipError_t {
    if (!attr_done[slot]) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
      if (e != hipSuccess) { return e; }
      attr_done[slot] = true;
    }
    return launch_kernel(kern, grid, block, (size_t)kLdsBytes, st, p);
  };
  if (a.w != nullptr) {
    return a.scaled_epilogue ? launch(gemm_kernel<true, true>, 0) : launch(gemm_kernel<true, false>, 1);
  }
  return a.scaled_epilogue ? launch(gemm_kernel<false, true>, 2) : launch(gemm_kernel<false, false>, 3);
}

}  // namespace vpq

// QMV, row-streaming form (M <= 2): a wavefront owns R consecutive weight rows and walks their
// whole K; nothing goes through LDS.
//
// Every load is a full-width contiguous one: a lane takes 16 bytes of codes (32 values) of a row
// per pass, so a wavefront's load instruction covers 1 KB of one row; the two lanes that share a
// quantization group read neighbouring scales, so the scale and bias loads of a wavefront are one
// cache line each.  The lane's 32 values of x are loaded once per pass and reused for the R rows.
//
// Arithmetic (the factored form of gpu-kernels/metal/quant/affine_qmv.metal:151-174, weight never
// rounded): codes become packed bf16 pairs (128 + q_i, 128 + q_{i+4}) with one v_and_or_b32 per
// pair and are contracted against the matching pair of x with v_dot2c_f32_bf16 (products exact,
// fp32 sums); with sx = sum of the lane's 32 x,
//     y += s * (dot - 128 * sx) + b * sx
// per row and pass, then one wave reduction per row.  The gated stores (SwiGLU / GEGLU over an
// interleaved gate|up pack) are register-local: R is even, so a (gate, up) pair of rows belongs
// to one wavefront.
#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;

constexpr int kPassK = kWave * 32;     // k-values a wavefront covers per pass (2048)

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c)
{
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}

}  // namespace

// Up to four packs that share x (q|k|v, gate|up): a pack owns the workgroups from its first_block on.
struct RowsSeg {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  void* y;
  int N;
  int first_block;
};
struct RowsSegs {
  int count;
  RowsSeg seg[4];
};

// R rows per wavefront, four wavefronts (4R rows) per workgroup, MT rows of x.
template <int R, int MT, bool F32OUT>
__global__ __launch_bounds__(256) void qmv_rows_kernel(
    const RowsSegs g, const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual, int K, int M, int gate_act)
{
  RowsSeg sg = g.seg[0];
#pragma unroll
  for (int i = 1; i < 4; ++i) {
    if (i < g.count && (int)blockIdx.x >= g.seg[i].first_block) { sg = g.seg[i]; }
  }
  const uint32_t* __restrict__ w = sg.w;
  const uint16_t* __restrict__ scales = sg.scales;
  const uint16_t* __restrict__ biases = sg.biases;
  void* __restrict__ y = sg.y;
  const int N = sg.N;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n0 = (((int)blockIdx.x - sg.first_block) * 4 + wave) * R;
  if (n0 >= N) { return; }              // wave-uniform; the kernel has no barrier
  const int Kw = K >> 3, Kg = K >> 6;

  uint32_t magic = 0x43004300u;         // bf16 128.0 in both halves
  uint32_t mask = 0x000f000fu;
  asm volatile("" : "+v"(magic));       // no instruction: hides the constants from folding, so
  asm volatile("" : "+s"(mask));        // that each pair costs one v_and_or_b32
  const uint32_t ones = 0x3f803f80u;    // bf16 1.0 twice

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int m = 0; m < MT; ++m) { acc[r][m] = 0.0f; }
  }
  const uint32_t* wrow[R];
  const uint16_t* srow[R];
  const uint16_t* brow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = (n0 + r < N) ? (n0 + r) : (N - 1);     // rows past N redo the last one; never stored
    wrow[r] = w + (size_t)n * Kw;
    srow[r] = scales + (size_t)n * Kg;
    brow[r] = biases + (size_t)n * Kg;
  }

  struct Pass {
    uint4 c[R];
    uint32_t sb[R], bb[R];
    uint4 xd[MT][4];
  };
  auto fetch = [&](int k0, Pass& p) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      p.c[r] = *reinterpret_cast<const uint4*>(wrow[r] + (k0 >> 3));
      p.sb[r] = srow[r][k0 >> 6];
      p.bb[r] = brow[r][k0 >> 6];
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const int row = m < M ? m : M - 1;
      const uint4* xs = reinterpret_cast<const uint4*>(x + (size_t)row * K + k0);
#pragma unroll
      for (int t = 0; t < 4; ++t) { p.xd[m][t] = xs[t]; }
    }
  };
  auto contract = [&](const Pass& p) {
    // the lane's 32 values of x, as pairs (x_i, x_{i+4}) of each group of eight, and their sum
    uint32_t xp[MT][16];
    float sx[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      float s = 0.0f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint4 d = p.xd[m][t];
        xp[m][4 * t + 0] = __builtin_amdgcn_perm(d.z, d.x, 0x05040100u);   // x0,x4
        xp[m][4 * t + 1] = __builtin_amdgcn_perm(d.z, d.x, 0x07060302u);   // x1,x5
        xp[m][4 * t + 2] = __builtin_amdgcn_perm(d.w, d.y, 0x05040100u);   // x2,x6
        xp[m][4 * t + 3] = __builtin_amdgcn_perm(d.w, d.y, 0x07060302u);   // x3,x7
        s = dot2(d.x, ones, s);
        s = dot2(d.y, ones, s);
        s = dot2(d.z, ones, s);
        s = dot2(d.w, ones, s);
      }
      sx[m] = s;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32_t cw[4] = {p.c[r].x, p.c[r].y, p.c[r].z, p.c[r].w};
      const float s = bf16_bits_to_f32(p.sb[r]);
      const float b = bf16_bits_to_f32(p.bb[r]);
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        float d = 0.0f;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
          for (int i = 0; i < 4; ++i) { d = dot2(xp[m][4 * t + i], ((cw[t] >> (4 * i)) & mask) | magic, d); }
        }
        acc[r][m] = fmaf(s, fmaf(-128.0f, sx[m], d), acc[r][m]);
        acc[r][m] = fmaf(b, sx[m], acc[r][m]);
      }
    }
  };

  // The wavefront's passes: k0 = lane*32, then every 2048.  The next pass is fetched before the
  // current one is contracted.
  constexpr int kStep = kPassK;
  int k0 = lane * 32;
  if (k0 < K) {
    Pass cur;
    fetch(k0, cur);
    for (;;) {
      const int k1 = k0 + kStep;
      if (k1 < K) {
        Pass nxt;
        fetch(k1, nxt);
        contract(cur);
        cur = nxt;
        k0 = k1;
      } else {
        contract(cur);
        break;
      }
    }
  }

  float total[MT][R];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
#pragma unroll
    for (int r = 0; r < R; ++r) { total[m][r] = wave_sum(acc[r][m]); }
  }
  if (lane != 0) { return; }
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    if (m >= M) { continue; }
    if (gate_act) {
#pragma unroll
      for (int r = 0; r < R; r += 2) {
        const int n = n0 + r;
        if (n + 1 < N) {
          const float v = gated_f32(gate_act, total[m][r], total[m][r + 1]);
          const size_t o = (size_t)m * (N >> 1) + (n >> 1);
          if (F32OUT) {
            reinterpret_cast<float*>(y)[o] = v;
          } else {
            reinterpret_cast<uint16_t*>(y)[o] = (uint16_t)f32_to_bf16_bits(v);
          }
        }
      }
      continue;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = n0 + r;
      if (n < N) {
        const size_t o = (size_t)m * N + n;
        if (F32OUT) {
          reinterpret_cast<float*>(y)[o] = total[m][r];
        } else {
          uint32_t v = f32_to_bf16_bits(total[m][r]);
          if (residual != nullptr) { v = f32_to_bf16_bits(bf16_bits_to_f32(v) + bf16_bits_to_f32(residual[o])); }
          reinterpret_cast<uint16_t*>(y)[o] = (uint16_t)v;
        }
      }
    }
  }
}

bool qmv_rows_supports(int K, int N, int M)
{
  return K % 64 == 0 && N >= 1 && M >= 1 && M <= 2;
}

namespace {

hipError_t launch_rows_segments(hipStream_t st, RowsSegs& g, const QmvArgs& a, int rows_per_wave)
{
  double bytes = 0.0;
  for (int i = 0; i < g.count; ++i) { bytes += (double)g.seg[i].N * (double)a.K * 9.0 / 16.0; }
  // Two rows per wavefront finish sooner on layer-sized packs (more, shorter wavefronts: 4096->4096
  // 4.3 vs 4.4 us, 5120->5120 6.6 vs 7.1, 17408->5120 14.7 vs 15.9); four on lm_head-sized ones,
  // where x is re-read half as often (5120->151936: 94 vs 100 us).
  const int R = rows_per_wave == 2 || rows_per_wave == 4 ? rows_per_wave : (bytes >= 150e6 ? 4 : 2);
  int blocks = 0;
  for (int i = 0; i < g.count; ++i) {
    g.seg[i].first_block = blocks;
    blocks += (g.seg[i].N + 4 * R - 1) / (4 * R);
  }
  const dim3 grid((unsigned)blocks), block(256);
#define VPQ_ROWS(RR, MT, F32) \
  launch_kernel(qmv_rows_kernel<RR, MT, F32>, grid, block, 0, st, g, a.x, a.residual, a.K, a.M, a.gate_act)
#define VPQ_ROWS_M(RR)                                                               \
  (a.M == 1 ? (a.y_f32 ? VPQ_ROWS(RR, 1, true) : VPQ_ROWS(RR, 1, false))             \
            : (a.y_f32 ? VPQ_ROWS(RR, 2, true) : VPQ_ROWS(RR, 2, false)))
  return R == 2 ? VPQ_ROWS_M(2) : VPQ_ROWS_M(4);
#undef VPQ_ROWS_M
#undef VPQ_ROWS
}

}  // namespace

hipError_t launch_qmv_rows(hipStream_t st, const QmvArgs& a, int rows_per_wave)
{
  RowsSegs g{};
  g.count = 1;
  g.seg[0] = RowsSeg{a.w, a.scales, a.biases, a.y, a.N, 0};
  return launch_rows_segments(st, g, a, rows_per_wave);
}

hipError_t launch_qmv_rows_group(hipStream_t st, const QmvArgs& a, const QmvGroup& grp)
{
  RowsSegs g{};
  g.count = grp.count;
  for (int i = 0; i < grp.count; ++i) {
    g.seg[i] = RowsSeg{grp.seg[i].w, grp.seg[i].scales, grp.seg[i].biases, grp.seg[i].y, grp.seg[i].N, 0};
  }
  return launch_rows_segments(st, g, a, 0);
}

}  // namespace vpq

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
//
// K <= 1024 leaves half of a 2048-wide pass idle, so there a row group takes 32 lanes and a
// wavefront carries two of them (LPR = 32); the lanes past K hold zeros in the 64-lane form, so the
// sums -- a butterfly from the widest step down -- are the same bits either way.
//
// Gathered form (MoE, gpu-kernels/metal/quant/affine_qmv.metal:908-962, 1262-1292): grid.y is a
// (token, expert) pair p; the pack is a batch [E, N, K/8] of expert slabs and pair_eid[p] picks
// the slab, x row p / x_div (gate|up: top_k pairs share a token's row) or p (down), y row p.
//
// Sorted form (MoE prefill with few rows per expert, gpu-kernels/metal/quant/affine_qmv.metal:2551-2719, MAXM = 2):
// the pairs have been sorted into per-expert tiles of two slots; grid.y is a tile, its expert's slab is read once
// for both slots.  Per-row arithmetic is that of the plain kernel.
#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;


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

// Gathered launches: null pair_eid for the plain forms.
struct RowsGather {
  const int* pair_eid;
  int x_div;        // x row of pair p is p / x_div
  int n_experts;    // ids outside [0, n_experts) give zeros
  // Sorted (grouped) form: grid.y is a tile of two slots owned by expert tile2e[tile] (< 0: unused tile, nothing
  // is written); slot s is live where srow[s] >= 0 and reads x row srow[s] (x_from_srow) or row s, writes y row s.
  const int* tile2e = nullptr;
  const int* srow = nullptr;
  int x_from_srow = 0;
};

// R rows per row group, 64 / LPR row groups per wavefront, four wavefronts per workgroup, MT rows of x.
// GS: log2 of the quantization group (6: group 64; 5: group 32, a lane's 32 values are one group).
// SO: scale-only (Q4_0) pack, the bias is -8 * scale and `biases` is never read
// (gpu-kernels/metal/quant/affine_qmv.metal:252-256).
template <int R, int MT, bool F32OUT, int LPR, int GS = 6, bool SO = false>
__global__ __launch_bounds__(256) void qmv_rows_kernel(
    const RowsSegs g, const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual, int K, int M, int gate_act,
    const RowsGather gather)
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
  constexpr int SUBS = kWave / LPR;      // row groups per wavefront
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int sub = lane / LPR, ll = lane % LPR;
  const int nw = (((int)blockIdx.x - sg.first_block) * 4 + wave) * SUBS * R;
  if (nw >= N) { return; }              // wave-uniform; the kernel has no barrier
  const int n0 = nw + sub * R;
  const int Kw = K >> 3, Kg = K >> GS;
  bool expert_ok = true;
  const uint16_t* xrow[MT];
  bool live[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    xrow[m] = x + (size_t)(m < M ? m : M - 1) * K;
    live[m] = m < M;
  }
  if (gather.tile2e != nullptr) {
    const int t = (int)blockIdx.y;
    const int e = gather.tile2e[t];
    if (e < 0 || e >= gather.n_experts) { return; }      // block-uniform; the kernel has no barrier
    w += (size_t)e * (size_t)N * Kw;
    scales += (size_t)e * (size_t)N * Kg;
    biases += (size_t)e * (size_t)N * Kg;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const int slot = t * MT + m;
      const int rr = gather.srow[slot];
      live[m] = rr >= 0;
      xrow[m] = x + (size_t)(gather.x_from_srow ? (rr >= 0 ? rr : 0) : slot) * K;
    }
    const size_t yo = (size_t)t * MT * (size_t)(gate_act ? (N >> 1) : N);
    y = F32OUT ? (void*)(reinterpret_cast<float*>(y) + yo) : (void*)(reinterpret_cast<uint16_t*>(y) + yo);
  } else if (gather.pair_eid != nullptr) {
    const int p = (int)blockIdx.y;
    int e = gather.pair_eid[p];
    expert_ok = e >= 0 && e < gather.n_experts;
    e = expert_ok ? e : 0;
    w += (size_t)e * (size_t)N * Kw;
    scales += (size_t)e * (size_t)N * Kg;
    biases += (size_t)e * (size_t)N * Kg;
    xrow[0] = x + (size_t)(p / gather.x_div) * K;
    const size_t yo = (size_t)p * (size_t)(gate_act ? (N >> 1) : N);
    y = F32OUT ? (void*)(reinterpret_cast<float*>(y) + yo) : (void*)(reinterpret_cast<uint16_t*>(y) + yo);
  }

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
      p.sb[r] = srow[r][k0 >> GS];
      p.bb[r] = SO ? 0u : brow[r][k0 >> GS];
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const uint4* xs = reinterpret_cast<const uint4*>(xrow[m] + k0);
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
      const float b = SO ? -8.0f * s : bf16_bits_to_f32(p.bb[r]);
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

  // The row group's passes: k0 = ll*32, then every LPR*32.  The next pass is fetched before the
  // current one is contracted.
  constexpr int kStep = LPR * 32;
  int k0 = ll * 32;
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
    for (int r = 0; r < R; ++r) {
      float v = acc[r][m];
#pragma unroll
      for (int off = LPR / 2; off >= 1; off >>= 1) { v += __shfl_xor(v, off, kWave); }
      total[m][r] = expert_ok ? v : 0.0f;
    }
  }
  if (ll != 0) { return; }
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    if (!live[m]) { continue; }
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

hipError_t launch_rows_segments(hipStream_t st, RowsSegs& g, const QmvArgs& a, int rows_per_wave,
                                const RowsGather& gather, int pairs, int group = 64, bool scale_only = false)
{
  double bytes = 0.0;
  for (int i = 0; i < g.count; ++i) { bytes += (double)g.seg[i].N * (double)a.K * 9.0 / 16.0; }
  // Two rows per row group finish sooner on layer-sized packs (more, shorter wavefronts: 4096->4096
  // 4.3 vs 4.4 us, 5120->5120 6.6 vs 7.1, 17408->5120 14.7 vs 15.9); four on lm_head-sized ones,
  // where x is re-read half as often (5120->151936: 94 vs 100 us).
  const int R = group == 32 ? 2 : (rows_per_wave == 2 || rows_per_wave == 4 ? rows_per_wave : (bytes >= 150e6 ? 4 : 2));
  const bool half = group == 64 && a.K <= 1024 && a.M == 1 && R == 2;      // 32 lanes per row group
  const int rows_per_block = 4 * R * (half ? 2 : 1);
  int blocks = 0;
  for (int i = 0; i < g.count; ++i) {
    g.seg[i].first_block = blocks;
    blocks += (g.seg[i].N + rows_per_block - 1) / rows_per_block;
  }
  const dim3 grid((unsigned)blocks, (unsigned)pairs), block(256);
#define VPQ_ROWS(RR, MT, F32, LPR) \
  launch_kernel(qmv_rows_kernel<RR, MT, F32, LPR>, grid, block, 0, st, g, a.x, a.residual, a.K, a.M, a.gate_act, gather)
#define VPQ_ROWS_M(RR)                                                                       \
  (a.M == 1 ? (a.y_f32 ? VPQ_ROWS(RR, 1, true, 64) : VPQ_ROWS(RR, 1, false, 64))             \
            : (a.y_f32 ? VPQ_ROWS(RR, 2, true, 64) : VPQ_ROWS(RR, 2, false, 64)))
#define VPQ_ROWS32(MT, F32, SO) \
  launch_kernel(qmv_rows_kernel<2, MT, F32, 64, 5, SO>, grid, block, 0, st, g, a.x, a.residual, a.K, a.M, a.gate_act, gather)
#define VPQ_ROWS32_M(SO)                                                             \
  (a.M == 1 ? (a.y_f32 ? VPQ_ROWS32(1, true, SO) : VPQ_ROWS32(1, false, SO))         \
            : (a.y_f32 ? VPQ_ROWS32(2, true, SO) : VPQ_ROWS32(2, false, SO)))
  if (group == 32) { return scale_only ? VPQ_ROWS32_M(true) : VPQ_ROWS32_M(false); }
  if (half) { return a.y_f32 ? VPQ_ROWS(2, 1, true, 32) : VPQ_ROWS(2, 1, false, 32); }
  return R == 2 ? VPQ_ROWS_M(2) : VPQ_ROWS_M(4);
#undef VPQ_ROWS32_M
#undef VPQ_ROWS32
#undef VPQ_ROWS_M
#undef VPQ_ROWS
}

}  // namespace

hipError_t launch_qmv_rows(hipStream_t st, const QmvArgs& a, int rows_per_wave)
{
  RowsSegs g{};
  g.count = 1;
  g.seg[0] = RowsSeg{a.w, a.scales, a.biases, a.y, a.N, 0};
  return launch_rows_segments(st, g, a, rows_per_wave, RowsGather{nullptr, 1, 0}, 1);
}

hipError_t launch_qmv_rows_group(hipStream_t st, const QmvArgs& a, const QmvGroup& grp, int group, bool scale_only)
{
  RowsSegs g{};
  g.count = grp.count;
  for (int i = 0; i < grp.count; ++i) {
    g.seg[i] = RowsSeg{grp.seg[i].w, grp.seg[i].scales, grp.seg[i].biases, grp.seg[i].y, grp.seg[i].N, 0};
  }
  return launch_rows_segments(st, g, a, group == 32 ? 2 : 0, RowsGather{nullptr, 1, 0}, 1, group, scale_only);
}

hipError_t launch_qmv_rows_gather(hipStream_t st, const QmvArgs& a, const int* pair_eid, int pairs, int x_div,
                                  int n_experts)
{
  RowsSegs g{};
  g.count = 1;
  g.seg[0] = RowsSeg{a.w, a.scales, a.biases, a.y, a.N, 0};
  return launch_rows_segments(st, g, a, 2, RowsGather{pair_eid, x_div, n_experts}, pairs);
}

// a.M = 2 (slots per tile); a.x is the hidden [rows, K] (x_from_srow) or the sorted activations [2 tiles, K].
hipError_t launch_qmv_rows_sorted(hipStream_t st, const QmvArgs& a, const int* tile2e, const int* srow, int tiles,
                                  bool x_from_srow, int n_experts)
{
  RowsSegs g{};
  g.count = 1;
  g.seg[0] = RowsSeg{a.w, a.scales, a.biases, a.y, a.N, 0};
  RowsGather ga{nullptr, 1, n_experts};
  ga.tile2e = tile2e;
  ga.srow = srow;
  ga.x_from_srow = x_from_srow ? 1 : 0;
  return launch_rows_segments(st, g, a, 2, ga, tiles);
}

hipError_t launch_qmv_rows_g32(hipStream_t st, const QmvArgs& a, bool scale_only)
{
  RowsSegs g{};
  g.count = 1;
  g.seg[0] = RowsSeg{a.w, a.scales, a.biases, a.y, a.N, 0};
  return launch_rows_segments(st, g, a, 2, RowsGather{nullptr, 1, 0}, 1, 32, scale_only);
}

}  // namespace vpq
